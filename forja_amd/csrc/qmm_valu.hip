// Quantised matmul on the vector ALUs, in f32: the path of everything the matrix-core kernels do
// not take (f32 or f16 activations, 8-bit weights, groups of 32 or 128, f16 scales) as long as
// rows are contiguous.  The reference holds f32 products to its f32 tolerance
// (crates/forja-metal/tests/quant_matmul.rs:108-120), so nothing here is rounded below f32.
//
// Arithmetic of affine_quant_dot (crates/forja-cpu/src/lib.rs:1277-1310): the weight is formed
// first, `scale * q + bias` in f32 (two roundings: this file is compiled without contraction), then
// multiplied into the sum.  The sum runs in another order than the reference's left-to-right one
// (K is split over the waves of a workgroup and their sums are added in wave order), which moves
// a result by f32 rounding only.
//
// A lane owns one output column, a workgroup 64 columns x 16 rows, a wave one slice of K.  Per step
// a lane loads 16 bytes of its packed weight row (32 or 16 values, inside one group), forms the
// weights, and multiplies them into its 16 row sums; the activations of a step are the same for
// all lanes, so they arrive through scalar loads and cost no vector registers or LDS.
#include "fast_kernels.hpp"
#include "kernels.hpp"

namespace fh {

namespace {

constexpr int kValuRows = 16, kValuWaves = 8;

struct ValuArgs {
  const void *x;
  uint64_t x_row_stride;          // elements
  const uint32_t *packed;
  const uint16_t *scales, *biases;
  uint32_t params_f16;            // scales and biases are f16 (else bf16)
  void *out;
  uint64_t out_row_stride;
  uint32_t out_dtype;
  const void *residual;           // optional [rows, columns] added before the result is rounded
  uint64_t residual_row_stride;
  uint32_t residual_dtype;
  uint32_t rows, inner, columns, group_shift, steps_per_wave;
};

__device__ inline float typed_load(const void *base, uint32_t dtype, uint64_t element) {
  if (dtype == FH_F32) return ((const float *)base)[element];
  const uint16_t bits = ((const uint16_t *)base)[element];
  return dtype == FH_F16 ? f16_to_f32(bits) : bf16_to_f32(bits);
}

// The 32 (4-bit) or 16 (8-bit) weights of one 16-byte piece: scale * q + bias, value j in bits
// [kBits j, kBits (j + 1)) of the piece (low bits first).
template <int kBits>
__device__ inline void form_weights(const uint4 &piece, float scale, float bias, float (&w)[128 / kBits]) {
  constexpr int kPerWord = 32 / kBits;
#pragma unroll
  for (int j = 0; j < 128 / kBits; ++j) {
    const uint32_t word = j / kPerWord == 0 ? piece.x : (j / kPerWord == 1 ? piece.y : (j / kPerWord == 2 ? piece.z : piece.w));
    const uint32_t q = (word >> (kBits * (j % kPerWord))) & ((1u << kBits) - 1u);
    w[j] = scale * (float)q + bias;
  }
}

// sum + x[at .. at + kValues) . w, the activations read through a pointer every lane shares.
template <uint32_t kX, int kValues>
__device__ inline float row_product(const void *base, uint64_t at, const float (&w)[kValues], float sum) {
  if constexpr (kX == FH_F32) {
    const float *x = (const float *)base + at;
#pragma unroll
    for (int j = 0; j < kValues; ++j) sum = fmaf(x[j], w[j], sum);
  } else {
    const uint32_t *x = (const uint32_t *)((const uint16_t *)base + at);
#pragma unroll
    for (int j = 0; j < kValues; j += 2) {
      const uint32_t two = x[j / 2];
      float lo, hi;
      if constexpr (kX == FH_BF16) {
        lo = __uint_as_float(two << 16);
        hi = __uint_as_float(two & 0xffff0000u);
      } else {
        lo = f16_to_f32((uint16_t)(two & 0xffffu));
        hi = f16_to_f32((uint16_t)(two >> 16));
      }
      sum = fmaf(lo, w[j], sum);
      sum = fmaf(hi, w[j + 1], sum);
    }
  }
  return sum;
}

template <int kBits, uint32_t kX>
__global__ __launch_bounds__(64 * kValuWaves) void qmm_valu_kernel(ValuArgs a) {
  constexpr int kValues = 128 / kBits;   // values in a 16-byte piece of a packed row
  __shared__ float handed[kValuWaves - 1][kValuRows][64];
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t waves = blockDim.x >> 6;
  const uint32_t column = blockIdx.x * 64 + lane;
  const uint32_t column_in = min(column, a.columns - 1);
  const uint32_t row0 = blockIdx.y * kValuRows;
  const uint32_t live_rows = min((uint32_t)kValuRows, a.rows - row0);
  const uint32_t pieces_per_row = a.inner / kValues;
  const uint32_t groups_per_row = a.inner >> a.group_shift;
  const uint4 *w_row = (const uint4 *)a.packed + (uint64_t)column_in * pieces_per_row;
  const uint16_t *s_row = a.scales + (uint64_t)column_in * groups_per_row;
  const uint16_t *b_row = a.biases + (uint64_t)column_in * groups_per_row;
  float acc[kValuRows];
#pragma unroll
  for (int r = 0; r < kValuRows; ++r) acc[r] = 0.0f;
  const uint32_t first = wave * a.steps_per_wave;
  const uint32_t last = min(first + a.steps_per_wave, pieces_per_row);
  // 64 bytes of the weight row are requested at a time: with few rows a wave is a chain of
  // dependent loads, and this makes it four times shorter
  constexpr int kAhead = 4;
  for (uint32_t step = first; step < last; step += kAhead) {
    uint4 piece[kAhead];
    uint16_t scale_bits[kAhead], bias_bits[kAhead];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      const uint32_t at = min(step + i, last - 1);
      piece[i] = w_row[at];
      scale_bits[i] = s_row[(at * kValues) >> a.group_shift];
      bias_bits[i] = b_row[(at * kValues) >> a.group_shift];
    }
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      if (step + i >= last) continue;   // the same for every lane
      const uint32_t k0 = (step + i) * kValues;
      const float scale = a.params_f16 ? f16_to_f32(scale_bits[i]) : bf16_to_f32(scale_bits[i]);
      const float bias = a.params_f16 ? f16_to_f32(bias_bits[i]) : bf16_to_f32(bias_bits[i]);
      float w[kValues];
      form_weights<kBits>(piece[i], scale, bias, w);
#pragma unroll
      for (int r = 0; r < kValuRows; ++r) {
        if ((uint32_t)r >= live_rows) continue;   // the same for every lane
        const uint64_t at = (uint64_t)(row0 + r) * a.x_row_stride + k0;
        acc[r] = row_product<kX, kValues>(a.x, at, w, acc[r]);
      }
    }
  }
  if (wave != 0) {
#pragma unroll
    for (int r = 0; r < kValuRows; ++r) handed[wave - 1][r][lane] = acc[r];
  }
  __syncthreads();
  if (wave != 0 || column >= a.columns) return;
#pragma unroll
  for (int r = 0; r < kValuRows; ++r) {
    if ((uint32_t)r >= live_rows) continue;
    float value = acc[r];
    for (uint32_t other = 0; other + 1 < waves; ++other) value += handed[other][r][lane];
    const uint32_t row = row0 + r;
    if (a.residual)
      value += typed_load(a.residual, a.residual_dtype, (uint64_t)row * a.residual_row_stride + column);
    const uint64_t at = (uint64_t)row * a.out_row_stride + column;
    if (a.out_dtype == FH_F32)
      ((float *)a.out)[at] = value;
    else if (a.out_dtype == FH_F16)
      ((uint16_t *)a.out)[at] = f32_to_f16(value);
    else
      ((uint16_t *)a.out)[at] = f32_to_bf16(value);
  }
}

// Few rows and not many columns (a decode batch of at most 8 rows against a layer's projections):
// 64 columns per workgroup would leave most of the device idle, so here a wave owns one column
// and its lanes split K in 16-byte pieces, every lane reading its own slice of each activation
// row; the lanes' sums meet in a butterfly.
constexpr int kFewRows = 8;

template <int kBits, uint32_t kX>
__global__ __launch_bounds__(256) void qmm_valu_few_rows_kernel(ValuArgs a) {
  constexpr int kValues = 128 / kBits;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t column = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if (column >= a.columns) return;
  const uint32_t pieces_per_row = a.inner / kValues, groups_per_row = a.inner >> a.group_shift;
  const uint4 *w_row = (const uint4 *)a.packed + (uint64_t)column * pieces_per_row;
  const uint16_t *s_row = a.scales + (uint64_t)column * groups_per_row;
  const uint16_t *b_row = a.biases + (uint64_t)column * groups_per_row;
  float acc[kFewRows];
#pragma unroll
  for (int r = 0; r < kFewRows; ++r) acc[r] = 0.0f;
  for (uint32_t piece = lane; piece < pieces_per_row; piece += 64) {
    const uint32_t k0 = piece * kValues, group = k0 >> a.group_shift;
    const float scale = a.params_f16 ? f16_to_f32(s_row[group]) : bf16_to_f32(s_row[group]);
    const float bias = a.params_f16 ? f16_to_f32(b_row[group]) : bf16_to_f32(b_row[group]);
    float w[kValues];
    form_weights<kBits>(w_row[piece], scale, bias, w);
#pragma unroll
    for (int r = 0; r < kFewRows; ++r) {
      if ((uint32_t)r >= a.rows) continue;
      acc[r] = row_product<kX, kValues>(a.x, (uint64_t)r * a.x_row_stride + k0, w, acc[r]);
    }
  }
#pragma unroll
  for (int r = 0; r < kFewRows; ++r) {
    if ((uint32_t)r >= a.rows) continue;
    float value = acc[r];
    for (int offset = 32; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, 64);
    if (lane != 0) continue;
    if (a.residual)
      value += typed_load(a.residual, a.residual_dtype, (uint64_t)r * a.residual_row_stride + column);
    const uint64_t at = (uint64_t)r * a.out_row_stride + column;
    if (a.out_dtype == FH_F32)
      ((float *)a.out)[at] = value;
    else if (a.out_dtype == FH_F16)
      ((uint16_t *)a.out)[at] = f32_to_f16(value);
    else
      ((uint16_t *)a.out)[at] = f32_to_bf16(value);
  }
}

template <int kBits>
void launch_valu_few_rows(hipStream_t stream, const ValuArgs &a, uint32_t x_dtype) {
  const dim3 grid((a.columns + 3) / 4);
  if (x_dtype == FH_F32)
    qmm_valu_few_rows_kernel<kBits, FH_F32><<<grid, 256, 0, stream>>>(a);
  else if (x_dtype == FH_F16)
    qmm_valu_few_rows_kernel<kBits, FH_F16><<<grid, 256, 0, stream>>>(a);
  else
    qmm_valu_few_rows_kernel<kBits, FH_BF16><<<grid, 256, 0, stream>>>(a);
}

template <int kBits>
void launch_valu(hipStream_t stream, const ValuArgs &a, dim3 grid, uint32_t threads, uint32_t x_dtype) {
  if (x_dtype == FH_F32)
    qmm_valu_kernel<kBits, FH_F32><<<grid, threads, 0, stream>>>(a);
  else if (x_dtype == FH_F16)
    qmm_valu_kernel<kBits, FH_F16><<<grid, threads, 0, stream>>>(a);
  else
    qmm_valu_kernel<kBits, FH_BF16><<<grid, threads, 0, stream>>>(a);
}

// ---- routed products ------------------------------------------------------------------------
//
// gather_quant_projection_values (crates/forja-cpu/src/lib.rs:1025-1106) and
// execute_gather_quant_weighted_sum (:1108-1204) in the same arithmetic.  A wave owns 64 columns
// of one route (projection) or of one output row (weighted sum: its routes are folded in
// ascending slot order, `+= w * value`, as the reference folds them).  An
// expert id out of range is reported, lowest first; the projection writes a zero row for it, the
// weighted sum skips it.  The four waves of a workgroup take a quarter of K each (their sums are
// added in wave order) and request 64 bytes of a weight row at a time: routed decode batches are
// few waves, each a chain of dependent loads, and both shorten it.
struct GatherValuArgs {
  const void *x;
  uint64_t x_stride_row, x_stride_slot;   // elements; slot stride 0 for the projection
  const uint32_t *packed;
  const uint16_t *scales, *biases;
  uint32_t params_f16;
  View indices, weights, out;             // weights: weighted sum only
  uint32_t rows, k, inner, experts, columns, group_shift, weighted;
};

template <int kBits, uint32_t kX>
__global__ __launch_bounds__(256) void gather_valu_kernel(GatherValuArgs a, ErrorSlot *error) {
  constexpr int kValues = 128 / kBits, kAhead = 4;   // pieces requested together: 64 bytes of a row
  __shared__ float handed[3][64];
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t column = blockIdx.x * 64 + lane, column_in = min(column, a.columns - 1);
  const uint32_t unit = blockIdx.y;                     // a route, or an output row
  const uint32_t pieces_per_row = a.inner / kValues, groups_per_row = a.inner >> a.group_shift;
  // the four waves of the workgroup take a quarter of K each
  const uint32_t per_wave = (pieces_per_row + 3) / 4;
  const uint32_t first = min(wave * per_wave, pieces_per_row), last = min(first + per_wave, pieces_per_row);
  const uint32_t row = a.weighted ? unit : unit / a.k;
  const uint32_t first_slot = a.weighted ? 0 : unit % a.k, slots = a.weighted ? a.k : 1;
  float folded = 0.0f;
  uint32_t lowest_bad = 0xffffffffu;   // reported after the loads: an atomic in between would keep
                                       // the compiler from reading the activations through scalar loads
  for (uint32_t slot = first_slot; slot < first_slot + slots; ++slot) {
    const uint32_t expert = __builtin_amdgcn_readfirstlane(
        load_u32_at(a.indices, a.indices.offset + row * a.indices.stride[0] + slot * a.indices.stride[1]));
    if (expert >= a.experts) {
      lowest_bad = min(lowest_bad, expert);
      continue;
    }
    const uint64_t weight_row = (uint64_t)expert * a.columns + column_in;
    const uint4 *w_row = (const uint4 *)a.packed + weight_row * pieces_per_row;
    const uint16_t *s_row = a.scales + weight_row * groups_per_row;
    const uint16_t *b_row = a.biases + weight_row * groups_per_row;
    const uint64_t x_at = (uint64_t)row * a.x_stride_row + (uint64_t)slot * a.x_stride_slot;
    float sum = 0.0f;
    for (uint32_t step = first; step < last; step += kAhead) {
      uint4 piece[kAhead];
      uint16_t scale_bits[kAhead], bias_bits[kAhead];
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        const uint32_t at = min(step + i, last - 1);
        piece[i] = w_row[at];
        scale_bits[i] = s_row[(at * kValues) >> a.group_shift];
        bias_bits[i] = b_row[(at * kValues) >> a.group_shift];
      }
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        if (step + i >= last) continue;   // the same for every lane
        const float scale = a.params_f16 ? f16_to_f32(scale_bits[i]) : bf16_to_f32(scale_bits[i]);
        const float bias = a.params_f16 ? f16_to_f32(bias_bits[i]) : bf16_to_f32(bias_bits[i]);
        float w[kValues];
        form_weights<kBits>(piece[i], scale, bias, w);
        sum = row_product<kX, kValues>(a.x, x_at + (uint64_t)(step + i) * kValues, w, sum);
      }
    }
    if (a.weighted)
      folded += load_float_at(a.weights, a.weights.offset + row * a.weights.stride[0] +
                                             slot * a.weights.stride[1]) * sum;
    else
      folded = sum;
  }
  if (wave != 0) handed[wave - 1][lane] = folded;
  __syncthreads();
  if (wave != 0) return;
  if (lowest_bad != 0xffffffffu && lane == 0 && blockIdx.x == 0) report_error(error, lowest_bad);
  if (column >= a.columns) return;
  folded = ((folded + handed[0][lane]) + handed[1][lane]) + handed[2][lane];
  if (a.weighted)
    store_float_at(a.out, a.out.offset + row * a.out.stride[0] + column * a.out.stride[1], folded);
  else
    store_float_at(a.out, a.out.offset + row * a.out.stride[0] + first_slot * a.out.stride[1] +
                              column * a.out.stride[2], folded);
}

template <int kBits>
void launch_gather_valu(hipStream_t stream, const GatherValuArgs &a, dim3 grid, uint32_t x_dtype,
                        ErrorSlot *error) {
  if (x_dtype == FH_F32)
    gather_valu_kernel<kBits, FH_F32><<<grid, 256, 0, stream>>>(a, error);
  else if (x_dtype == FH_F16)
    gather_valu_kernel<kBits, FH_F16><<<grid, 256, 0, stream>>>(a, error);
  else
    gather_valu_kernel<kBits, FH_BF16><<<grid, 256, 0, stream>>>(a, error);
}

// ---- routed products grouped by expert ------------------------------------------------------
//
// With several routes per expert the weights are formed once per tile of routes: a workgroup owns
// 64 columns of half a packed tile (an expert and up to 16 of its routes), its four waves a
// quarter of K each.  Route r of the tile reads the activation row `route / route_div` and
// writes row `route` of a dense [routes, N] output (the [R,k,N] result, or f32 partial sums the
// weighted form folds afterwards).
struct GroupedValuArgs {
  const void *x;
  uint64_t x_row_stride;
  const uint32_t *packed;
  const uint16_t *scales, *biases;
  uint32_t params_f16;
  void *out;
  uint32_t out_dtype;
  const uint32_t *sorted_routes, *blocks, *n_blocks;
  uint32_t route_div, inner, columns, group_shift;
};

template <int kBits, uint32_t kX>
__global__ __launch_bounds__(256) void gather_grouped_valu_kernel(GroupedValuArgs a) {
  constexpr int kValues = 128 / kBits, kAhead = 4, kRows = 16;
  __shared__ float handed[3][kRows][64];
  // blockIdx.y is (tile, half): 16 of the tile's routes per workgroup.  (A loop over the halves
  // would put the first half's stores before the second half's loads, and the compiler then
  // reads the activations through vector loads instead of scalar ones.)
  const uint32_t tile = blockIdx.y >> 1, pass = (blockIdx.y & 1) * kRows;
  if (tile >= a.n_blocks[0]) return;
  const uint32_t expert = a.blocks[3 * tile], tile_first = a.blocks[3 * tile + 1], tile_count = a.blocks[3 * tile + 2];
  if (pass >= tile_count) return;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t column = blockIdx.x * 64 + lane, column_in = min(column, a.columns - 1);
  const uint32_t pieces_per_row = a.inner / kValues, groups_per_row = a.inner >> a.group_shift;
  const uint32_t per_wave = (pieces_per_row + 3) / 4;
  const uint32_t first = min(wave * per_wave, pieces_per_row), last = min(first + per_wave, pieces_per_row);
  const uint64_t weight_row = (uint64_t)expert * a.columns + column_in;
  const uint4 *w_row = (const uint4 *)a.packed + weight_row * pieces_per_row;
  const uint16_t *s_row = a.scales + weight_row * groups_per_row;
  const uint16_t *b_row = a.biases + weight_row * groups_per_row;
  {
    const uint32_t live = min((uint32_t)kRows, tile_count - pass);
    uint32_t route[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
      route[r] = a.sorted_routes[tile_first + pass + min((uint32_t)r, live - 1)];
    float acc[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) acc[r] = 0.0f;
    for (uint32_t step = first; step < last; step += kAhead) {
      uint4 piece[kAhead];
      uint16_t scale_bits[kAhead], bias_bits[kAhead];
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        const uint32_t at = min(step + i, last - 1);
        piece[i] = w_row[at];
        scale_bits[i] = s_row[(at * kValues) >> a.group_shift];
        bias_bits[i] = b_row[(at * kValues) >> a.group_shift];
      }
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        if (step + i >= last) continue;   // the same for every lane
        const float scale = a.params_f16 ? f16_to_f32(scale_bits[i]) : bf16_to_f32(scale_bits[i]);
        const float bias = a.params_f16 ? f16_to_f32(bias_bits[i]) : bf16_to_f32(bias_bits[i]);
        float w[kValues];
        form_weights<kBits>(piece[i], scale, bias, w);
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
          if ((uint32_t)r >= live) continue;
          const uint64_t at = (uint64_t)(route[r] / a.route_div) * a.x_row_stride + (uint64_t)(step + i) * kValues;
          acc[r] = row_product<kX, kValues>(a.x, at, w, acc[r]);
        }
      }
    }
    if (wave != 0) {
#pragma unroll
      for (int r = 0; r < kRows; ++r) handed[wave - 1][r][lane] = acc[r];
    }
    __syncthreads();
    if (wave == 0 && column < a.columns) {
#pragma unroll
      for (int r = 0; r < kRows; ++r) {
        if ((uint32_t)r >= live) continue;
        const float value = ((acc[r] + handed[0][r][lane]) + handed[1][r][lane]) + handed[2][r][lane];
        const uint64_t at = (uint64_t)route[r] * a.columns + column;
        if (a.out_dtype == FH_F32)
          ((float *)a.out)[at] = value;
        else if (a.out_dtype == FH_F16)
          ((uint16_t *)a.out)[at] = f32_to_f16(value);
        else
          ((uint16_t *)a.out)[at] = f32_to_bf16(value);
      }
    }
  }
}

template <int kBits>
void launch_grouped_valu(hipStream_t stream, const GroupedValuArgs &a, dim3 grid, uint32_t x_dtype) {
  if (x_dtype == FH_F32)
    gather_grouped_valu_kernel<kBits, FH_F32><<<grid, 256, 0, stream>>>(a);
  else if (x_dtype == FH_F16)
    gather_grouped_valu_kernel<kBits, FH_F16><<<grid, 256, 0, stream>>>(a);
  else
    gather_grouped_valu_kernel<kBits, FH_BF16><<<grid, 256, 0, stream>>>(a);
}

bool is_float_dtype(uint32_t dtype) { return dtype == FH_F32 || dtype == FH_F16 || dtype == FH_BF16; }

char *element_address(const View &v) { return v.base + v.offset * dtype_size(v.dtype); }

}  // namespace

bool try_valu_quant_matmul(fh_backend *backend, const QmmProblem &p) {
  if (p.bits != 4 && p.bits != 8) return false;
  if (p.group != 32 && p.group != 64 && p.group != 128) return false;
  if (p.rows == 0 || p.columns == 0 || p.inner == 0 || p.inner % p.group != 0) return false;
  if (!is_float_dtype(p.x.dtype) || !is_float_dtype(p.out.dtype)) return false;
  if ((p.scales.dtype != FH_BF16 && p.scales.dtype != FH_F16) || p.biases.dtype != p.scales.dtype)
    return false;
  // contiguous weight rows, 16-byte aligned; activation pairs word aligned
  const uint64_t words_per_row = (uint64_t)p.inner * p.bits / 32, groups_per_row = p.inner / p.group;
  if (p.packed.stride[1] != 1 || p.packed.stride[0] != words_per_row || p.packed.offset % 4 != 0) return false;
  for (const View *v : {&p.scales, &p.biases})
    if (v->stride[1] != 1 || v->stride[0] != groups_per_row) return false;
  if (p.x.stride[1] != 1 || p.out.stride[1] != 1) return false;
  if (p.x.dtype != FH_F32 && (p.x.stride[0] % 2 != 0 || p.x.offset % 2 != 0)) return false;
  if (p.residual && (!is_float_dtype(p.residual->dtype) || p.residual->stride[1] != 1)) return false;
  const uint32_t values = 128 / p.bits, pieces = p.inner / values;
  if (p.inner % values != 0) return false;
  ValuArgs a{};
  a.x = element_address(p.x);
  a.x_row_stride = p.x.stride[0];
  a.packed = (const uint32_t *)element_address(p.packed);
  a.scales = (const uint16_t *)element_address(p.scales);
  a.biases = (const uint16_t *)element_address(p.biases);
  a.params_f16 = p.scales.dtype == FH_F16;
  a.out = element_address(p.out);
  a.out_row_stride = p.out.stride[0];
  a.out_dtype = p.out.dtype;
  if (p.residual) {
    a.residual = element_address(*p.residual);
    a.residual_row_stride = p.residual->stride[0];
    a.residual_dtype = p.residual->dtype;
  }
  a.rows = p.rows;
  a.inner = p.inner;
  a.columns = p.columns;
  a.group_shift = p.group == 32 ? 5 : (p.group == 64 ? 6 : 7);
  const uint32_t waves = pieces < (uint32_t)kValuWaves ? pieces : (uint32_t)kValuWaves;
  a.steps_per_wave = (pieces + waves - 1) / waves;
  const uint64_t row_blocks = ((uint64_t)p.rows + kValuRows - 1) / kValuRows;
  if (row_blocks > 65535) return false;
  const dim3 grid((p.columns + 63) / 64, (unsigned)row_blocks);
  KernelTimer timer(backend, FH_KC_QMM_KERNEL);
  // (each wave of the few-rows kernel reads the activation rows for itself, through L1: beyond a
  // couple of thousand columns that traffic costs more than the idle compute units did)
  if (p.rows <= (uint32_t)kFewRows && p.columns <= 2048) {
    if (p.bits == 4)
      launch_valu_few_rows<4>(backend_stream(backend), a, p.x.dtype);
    else
      launch_valu_few_rows<8>(backend_stream(backend), a, p.x.dtype);
    return true;
  }
  if (p.bits == 4)
    launch_valu<4>(backend_stream(backend), a, grid, 64 * waves, p.x.dtype);
  else
    launch_valu<8>(backend_stream(backend), a, grid, 64 * waves, p.x.dtype);
  return true;
}

bool try_valu_gather(fh_backend *backend, const View &x, const View &packed, const View &scales,
                     const View &biases, const View &indices, const View *weights, const View &out,
                     uint32_t rows, uint32_t k, uint32_t inner, uint32_t experts, uint32_t columns,
                     uint32_t bits, uint32_t group, ErrorSlot *error) {
  if (bits != 4 && bits != 8) return false;
  if (group != 32 && group != 64 && group != 128) return false;
  if (rows == 0 || k == 0 || columns == 0 || inner == 0 || inner % group != 0) return false;
  if (!is_float_dtype(x.dtype) || !is_float_dtype(out.dtype)) return false;
  if ((scales.dtype != FH_BF16 && scales.dtype != FH_F16) || biases.dtype != scales.dtype) return false;
  const uint64_t words_per_row = (uint64_t)inner * bits / 32, groups_per_row = inner / group;
  if (packed.stride[2] != 1 || packed.stride[1] != words_per_row ||
      packed.stride[0] != words_per_row * columns || packed.offset % 4 != 0)
    return false;
  for (const View *v : {&scales, &biases})
    if (v->stride[2] != 1 || v->stride[1] != groups_per_row || v->stride[0] != groups_per_row * columns)
      return false;
  const uint32_t last = x.rank - 1;
  if (x.stride[last] != 1) return false;
  if (x.dtype != FH_F32)
    for (uint32_t axis = 0; axis < last; ++axis)
      if (x.stride[axis] % 2 != 0) return false;
  if (x.dtype != FH_F32 && x.offset % 2 != 0) return false;
  const uint64_t units = weights ? rows : (uint64_t)rows * k;
  if (units > 65535) return false;
  GatherValuArgs a{};
  a.x = element_address(x);
  a.x_stride_row = x.stride[0];
  a.x_stride_slot = weights ? x.stride[1] : 0;
  a.packed = (const uint32_t *)element_address(packed);
  a.scales = (const uint16_t *)element_address(scales);
  a.biases = (const uint16_t *)element_address(biases);
  a.params_f16 = scales.dtype == FH_F16;
  a.indices = indices;
  if (weights) a.weights = *weights;
  a.out = out;
  a.rows = rows;
  a.k = k;
  a.inner = inner;
  a.experts = experts;
  a.columns = columns;
  a.group_shift = group == 32 ? 5 : (group == 64 ? 6 : 7);
  a.weighted = weights != nullptr;
  const dim3 grid((columns + 63) / 64, (unsigned)units);
  KernelTimer timer(backend, FH_KC_MOE_KERNEL);
  if (bits == 4)
    launch_gather_valu<4>(backend_stream(backend), a, grid, x.dtype, error);
  else
    launch_gather_valu<8>(backend_stream(backend), a, grid, x.dtype, error);
  return true;
}

bool try_valu_gather_grouped(fh_backend *backend, const GatherProblem &p, int projection, const View &out,
                             bool weighted, const View *residual, ErrorSlot *error) {
  // worth the packing launch only when the weights formed for a tile serve several routes
  if ((uint64_t)p.rows * p.k < 4ull * p.experts) return false;
  const View &packed = p.packed[projection], &scales = p.scales[projection], &biases = p.biases[projection];
  if (p.bits != 4 && p.bits != 8) return false;
  if (p.group != 32 && p.group != 64 && p.group != 128) return false;
  if (p.inner == 0 || p.inner % p.group != 0 || p.columns == 0) return false;
  if (!is_float_dtype(p.x.dtype) || !is_float_dtype(out.dtype)) return false;
  if ((scales.dtype != FH_BF16 && scales.dtype != FH_F16) || biases.dtype != scales.dtype) return false;
  const uint64_t words_per_row = (uint64_t)p.inner * p.bits / 32, groups_per_row = p.inner / p.group;
  if (packed.stride[2] != 1 || packed.stride[1] != words_per_row ||
      packed.stride[0] != words_per_row * p.columns || packed.offset % 4 != 0)
    return false;
  for (const View *v : {&scales, &biases})
    if (v->stride[2] != 1 || v->stride[1] != groups_per_row || v->stride[0] != groups_per_row * p.columns)
      return false;
  // activation rows: [R,K] rows, or [R,k,K] dense over its first two axes so that route r*k+s is row r*k+s
  uint64_t x_row_stride;
  if (weighted) {
    if (p.x.stride[2] != 1 || p.x.stride[0] != (uint64_t)p.k * p.x.stride[1]) return false;
    x_row_stride = p.x.stride[1];
  } else {
    if (p.x.stride[1] != 1) return false;
    x_row_stride = p.x.stride[0];
  }
  if (p.x.dtype != FH_F32 && (x_row_stride % 2 != 0 || p.x.offset % 2 != 0)) return false;
  const uint64_t routes = (uint64_t)p.rows * p.k;
  if (!weighted && (out.stride[2] != 1 || out.stride[1] != p.columns || out.stride[0] != (uint64_t)p.k * p.columns))
    return false;
  if (!weighted && dtype_size(out.dtype) == 2 && ((routes * p.columns) % 2 != 0 || out.offset % 2 != 0))
    return false;
  PackedRoutes plan;
  if (!pack_routes(backend, p, weighted ? routes * p.columns * sizeof(float) : 0, error, &plan)) return false;
  if (plan.tile != 32 || 2 * plan.max_blocks > 65535) return false;   // two halves of 16 routes per tile
  hipStream_t stream = backend_stream(backend);
  GroupedValuArgs a{};
  a.x = element_address(p.x);
  a.x_row_stride = x_row_stride;
  a.packed = (const uint32_t *)element_address(packed);
  a.scales = (const uint16_t *)element_address(scales);
  a.biases = (const uint16_t *)element_address(biases);
  a.params_f16 = scales.dtype == FH_F16;
  a.sorted_routes = plan.sorted_routes;
  a.blocks = plan.blocks;
  a.n_blocks = plan.n_blocks;
  a.route_div = weighted ? 1 : p.k;
  a.inner = p.inner;
  a.columns = p.columns;
  a.group_shift = p.group == 32 ? 5 : (p.group == 64 ? 6 : 7);
  if (weighted) {
    a.out = plan.rest;       // f32 partial sums per route; rows of bad routes are never read
    a.out_dtype = FH_F32;
  } else {
    a.out = element_address(out);
    a.out_dtype = out.dtype;
    // rows of bad routes, which are never packed, read zero
    launch_fill_u32(stream, (uint32_t *)a.out, routes * p.columns * dtype_size(out.dtype) / 4, 0);
  }
  const dim3 grid((p.columns + 63) / 64, 2 * plan.max_blocks);
  {
    KernelTimer timer(backend, FH_KC_MOE_KERNEL);
    if (p.bits == 4)
      launch_grouped_valu<4>(stream, a, grid, p.x.dtype);
    else
      launch_grouped_valu<8>(stream, a, grid, p.x.dtype);
  }
  if (weighted) {
    GatherProblem folded = p;
    folded.out = out;
    launch_combine_routes(stream, (const float *)plan.rest, folded, residual);
  }
  return true;
}

}  // namespace fh
