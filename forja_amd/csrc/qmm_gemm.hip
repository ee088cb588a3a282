// MLX-4bit quantised matmul for many activation rows (prefill chunks): a tiled f16 MFMA GEMM
// whose weight tiles are dequantised on their way into LDS.
//
// y[m,n] = sum_k x[m,k] * (scale[n,k/64] * q[n,k] + bias[n,k/64])   (affine_quant_dot,
// crates/forja-cpu/src/lib.rs:1277-1310).  With hundreds of rows per weight the work is bound by
// the matrix cores, not by HBM, so the kernel is a classic GEMM:
//   * operands are fp16, not bf16: a dequantised weight scale*q+bias rounded to bf16 (8
//     significant bits) is too coarse for the stated tolerance on outputs that cancel, fp16 (11
//     bits) is not, and the matrix cores run both at the same rate.  bf16 activations convert to
//     fp16 exactly; prepare_rows_kernel does that once per product (scaling a row by a power of
//     two first if it holds values beyond the fp16 range, undone exactly in the epilogue) and
//     stores every 8 values in the order (0,4,1,5,2,6,3,7) in which nibbles unpack pairwise;
//   * workgroup tile 256 rows x 256 columns, K step 64 (one quantisation group); four waves in
//     a 2 x 2 arrangement, each owning 128 x 128 outputs = 16 accumulator tiles of
//     v_mfma_f32_32x32x16_f16 (256 accumulator registers);
//   * both operand tiles live in LDS, double buffered.  The activation tile goes from memory
//     straight into LDS (global_load_lds, no registers), its 16-byte pieces XOR-swizzled inside
//     each 128-byte row so that operand reads are bank-conflict free without padding; the weight
//     tile passes through registers to be dequantised and is stored in rows padded to 144 bytes.
//     The next K step is staged while the current one is multiplied, one barrier per step;
//     packed weights are requested two steps ahead (they are cold in HBM);
//   * a thread dequantises one weight row of the tile per step (64 nibbles): two nibbles become
//     the fp16 pair (1024+q) with one and-or, minus 1024 exactly, then one packed fused
//     multiply-add gives scale*q - c rounded once, with c ~ 7.5*scale the fp16 value that centres
//     the group.  What the centring takes out, (bias + c) * sum of the group's activations, is
//     added back exactly: the row sums per group come from prepare_rows_kernel in f32 and an f32
//     MFMA adds the rank-2 update of every two groups to the same accumulators.  Centred values
//     are half the magnitude of the weights and carry no bias, which keeps the fp16 rounding
//     inside the tolerance at the deepest contractions (K = 17408).  That needs every scale and bias to lie
//     well inside the fp16 range; check_affine_kernel scans them first and raises a flag
//     otherwise, and then a second instantiation of the kernel, which dequantises in f32, does
//     the work instead (both are launched; the one whose turn it is not returns at once).  Every weight byte is read from HBM once per 256 rows and unpacked once per
//     workgroup;
//   * the workgroup -> tile map gives the 32 workgroups that run together on one XCD a patch of
//     about 4 row tiles x 8 column tiles, so that its L2 serves each activation tile to 8
//     workgroups and each weight tile to 4, instead of every workgroup streaming its own.
// Accumulation is f32.
#include "fast_kernels.hpp"

#include <type_traits>

namespace fh {

namespace {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kBM = 256, kBN = 256, kBK = 64;
constexpr int kBand = 8;   // column tiles per band of the tile numbering
constexpr int kPitch = 2 * kBK + 16;              // bytes per staged weight row
constexpr int kATileBytes = kBM * 2 * kBK;        // activation tile, swizzled, no padding
constexpr int kBTileBytes = kBN * kPitch;         // weight tile
constexpr int kSideBytes = 4 * (kBM + kBN) * 4;  // row sums and column offsets of four groups, f32
constexpr int kGemmLds = 2 * (kATileBytes + kBTileBytes) + kSideBytes;

struct GemmArgs {
  const uint16_t *x;        // fp16 rows prepared by prepare_rows_kernel, stride = inner
  const float *row_unscale; // per row: multiply the result by this
  const float *group_sums;  // [inner / 64][rows]: sums of the prepared rows per group
  uint64_t x_row_stride;
  const uint32_t *packed;
  const uint16_t *scales, *biases;
  void *out;
  uint64_t out_row_stride;
  uint32_t out_f32;
  uint32_t rows, inner, columns;
  uint32_t row_tiles, column_tiles;
  const uint32_t *wide_flag;   // non-zero: some scale or bias does not fit fp16
};

__device__ inline uint32_t pack2(float lo, float hi) {
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ inline float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

__device__ inline uint32_t pack_f16(float lo, float hi) {
  f16x2 v = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

// Eight nibbles of `w`, dequantised to fp16, as the four pairs (0,4)(1,5)(2,6)(3,7).
// Fast form: (1024+q) pairs by and-or, minus 1024 (exact), then fused scale*q+bias per pair.
__device__ inline uint4 dequantise_word(uint32_t w, f16x2 scale2, f16x2 shift2) {
  const uint32_t mask = 0x000f000fu, magic = 0x64006400u;
  const f16x2 offset = {(_Float16)1024.0f, (_Float16)1024.0f};
  uint32_t raw[4] = {(w & mask) | magic, ((w >> 4) & mask) | magic, ((w >> 8) & mask) | magic,
                     ((w >> 12) & mask) | magic};
  uint32_t out[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const f16x2 q = __builtin_bit_cast(f16x2, raw[i]) - offset;
    out[i] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(q, scale2, shift2));
  }
  return make_uint4(out[0], out[1], out[2], out[3]);
}

// The same in f32 with one rounding to fp16, for scales or biases outside the fp16 range.
__device__ inline uint4 dequantise_word_wide(uint32_t w, float scale, float shift) {
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = __builtin_fmaf(scale, (float)((w >> (4 * i)) & 15u), shift);
  return make_uint4(pack_f16(v[0], v[4]), pack_f16(v[1], v[5]), pack_f16(v[2], v[6]),
                    pack_f16(v[3], v[7]));
}

// Scales and biases the fp16 form can take: finite and well inside the fp16 range (15 * scale +
// bias must not overflow).  Magnitudes below the fp16 normal range become fp16 subnormals, an
// absolute error under 2^-25 per weight, far below the rounding of the weight itself.
__device__ inline bool f16_safe(float scale, float bias) {
  return fabsf(scale) <= 2048.0f && fabsf(bias) <= 30000.0f;   // false for NaN too
}

// x bf16 [rows, inner] -> fp16 [rows, inner] (every 8 values stored as 0,4,1,5,2,6,3,7), each row
// multiplied by a power of two that brings its largest magnitude under 2^15; unscale[row] is the
// inverse; group_sums[g][row] is the f32 sum of the row's 64 prepared values of group g.
// One wave per row.
__global__ __launch_bounds__(256) void prepare_rows_kernel(const uint16_t *x, uint64_t x_row_stride,
                                                           uint32_t rows, uint32_t inner,
                                                           uint16_t *out, float *unscale,
                                                           float *group_sums) {
  const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= rows) return;
  const uint16_t *in_row = x + (uint64_t)row * x_row_stride;
  uint32_t top = 0;   // largest magnitude bits (bf16 without sign) in the row
  for (uint32_t piece = lane; piece < inner / 8; piece += 64) {
    const uint4 v = *(const uint4 *)(in_row + 8 * piece);
    const uint32_t words[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t lo = words[i] & 0x7fffu, hi = (words[i] >> 16) & 0x7fffu;
      // NaN and infinity (exponent 255) pass through the conversion unchanged; leave them out
      if (lo < 0x7f80u) top = max(top, lo);
      if (hi < 0x7f80u) top = max(top, hi);
    }
  }
  for (int offset = 32; offset > 0; offset >>= 1) top = max(top, (uint32_t)__shfl_xor((int)top, offset, 64));
  const int exponent = (int)(top >> 7) - 127;                    // floor(log2(max |x|))
  const int down = exponent > 14 ? exponent - 14 : 0;            // scale by 2^-down
  const float scale = __uint_as_float((uint32_t)(127 - down) << 23);
  if (lane == 0) unscale[row] = __uint_as_float((uint32_t)(127 + down) << 23);
  uint16_t *out_row = out + (uint64_t)row * inner;
  for (uint32_t piece = lane; piece < inner / 8; piece += 64) {
    const uint4 v = *(const uint4 *)(in_row + 8 * piece);
    const uint32_t words[4] = {v.x, v.y, v.z, v.w};
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(words[i] << 16) * scale;
      f[2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u) * scale;
    }
    *(uint4 *)(out_row + 8 * piece) = make_uint4(pack_f16(f[0], f[4]), pack_f16(f[1], f[5]),
                                                 pack_f16(f[2], f[6]), pack_f16(f[3], f[7]));
    // eight consecutive pieces (= lanes) make one group; the scaled values are exact in f32
    float sum = ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7]));
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);
    sum += __shfl_xor(sum, 4, 64);
    if ((piece & 7) == 0) group_sums[(uint64_t)(piece >> 3) * rows + row] = sum;
  }
}

// flag[0] = 1 if any scale or bias of the matrix is too large for (or not a number in) fp16.
__global__ void check_affine_kernel(const uint16_t *scales, const uint16_t *biases, uint64_t count,
                                    uint32_t *flag) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  if (!f16_safe(bf16_bits_to_f32(scales[i]), bf16_bits_to_f32(biases[i]))) flag[0] = 1;
}

template <bool kWide>
__global__ __launch_bounds__(256) void qmm_gemm_kernel(GemmArgs a) {
  if ((a.wide_flag[0] != 0) != kWide) return;
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_lds[];
  unsigned char *a_tiles = gemm_lds;                      // [2][kBM][128], pieces swizzled
  unsigned char *b_tiles = gemm_lds + 2 * kATileBytes;    // [2][kBN][kPitch]
  float *side_rows = (float *)(gemm_lds + 2 * (kATileBytes + kBTileBytes));   // [4][kBM], ring by group
  float *side_cols = side_rows + 4 * kBM;                                     // [4][kBN]
  const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const uint32_t wm = wave >> 1, wn = wave & 1;
  const uint32_t l32 = lane & 31, kh = lane >> 5;

  // workgroup -> tile.  Tiles are numbered band by band (a band = kBand column tiles), row
  // tile major inside a band, so 32 consecutive numbers are a 4 x 8 patch of tiles sharing
  // activation and weight tiles.  Workgroups are dealt round-robin to the 8 XCDs (workgroup b is
  // the (b / 8)-th of XCD b % 8, and 32 consecutive ones of an XCD run together): each such
  // group of 32 takes one patch, so the XCD's L2 serves an activation tile to 8 workgroups and
  // a weight tile to 4.
  const uint32_t xcd = blockIdx.x % 8, nth = blockIdx.x / 8;
  const uint32_t tile = (nth / 32) * 256 + xcd * 32 + nth % 32;
  if (tile >= a.row_tiles * a.column_tiles) return;
  const uint32_t band = tile / (a.row_tiles * kBand);
  const uint32_t band_width = min((uint32_t)kBand, a.column_tiles - band * kBand);
  const uint32_t in_band = tile - band * a.row_tiles * kBand;
  const uint32_t bm = in_band / band_width, bn = band * kBand + in_band % band_width;
  const uint32_t row0 = bm * kBM, col0 = bn * kBN;

  // Activation staging: a wave owns 64 rows of the tile; one instruction moves 8 rows (lane ->
  // row lane/8, LDS slot lane%8), and the piece a lane fetches is its slot XOR ((row >> 1) & 7).
  const uint16_t *a_src[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t in_tile = 64 * wave + 8 * i + lane / 8;
    const uint32_t row = min(row0 + in_tile, a.rows - 1);   // tail rows reload the last row; never stored
    const uint32_t piece = (lane % 8) ^ ((in_tile >> 1) & 7);
    a_src[i] = a.x + (uint64_t)row * a.x_row_stride + 8 * piece;
  }
  auto stage_a = [&](uint32_t buffer, uint32_t step) {
    unsigned char *to = a_tiles + buffer * kATileBytes + 64 * wave * 128;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void *)(a_src[i] + step * kBK),
          (__attribute__((address_space(3))) void *)(to + 8 * i * 128), 16, 0, 0);
  };
  // Weight staging: thread t dequantises row t of the tile.
  const uint32_t b_col = min(col0 + tid, a.columns - 1);
  const uint32_t steps = a.inner / kBK;
  const uint32_t *w_row = a.packed + (uint64_t)b_col * (a.inner / 8);
  const uint16_t *s_row = a.scales + (uint64_t)b_col * steps;
  const uint16_t *b_row = a.biases + (uint64_t)b_col * steps;
  uint4 w_now[2], w_next[2];
  uint32_t affine_now, affine_next;   // scale | bias << 16
  float sum_now, sum_next;            // group sum of tile row `tid`
  const float *sums_of_row = a.group_sums + min(row0 + tid, a.rows - 1);
  auto fetch_w = [&](uint32_t step) {
    const uint32_t st = min(step, steps - 1);
    w_next[0] = *(const uint4 *)(w_row + st * 8);
    w_next[1] = *(const uint4 *)(w_row + st * 8 + 4);
    affine_next = (uint32_t)s_row[st] | ((uint32_t)b_row[st] << 16);
    sum_next = sums_of_row[(uint64_t)st * a.rows];
  };
  // The group's centre c (an fp16 value near 7.5 * scale) and what it leaves to add back per
  // unit of activation sum: bias + c.
  auto centre_of = [&](float scale) { return (float)(_Float16)(7.5f * scale); };
  auto stage_side = [&](uint32_t step) {
    const float scale = bf16_bits_to_f32(affine_now & 0xffffu), bias = bf16_bits_to_f32(affine_now >> 16);
    side_rows[(step & 3) * kBM + tid] = sum_now;
    side_cols[(step & 3) * kBN + tid] = bias + (kWide ? 7.5f * scale : centre_of(scale));
  };
  // one packed word (8 values) of the weight row: `part` 0..7
  auto stage_b = [&](uint32_t buffer, int part) {
    unsigned char *bt = b_tiles + buffer * kBTileBytes + tid * kPitch + 16 * part;
    const float scale = bf16_bits_to_f32(affine_now & 0xffffu), bias = bf16_bits_to_f32(affine_now >> 16);
    const uint4 w = w_now[part / 4];
    const uint32_t word = (part & 3) == 0 ? w.x : ((part & 3) == 1 ? w.y : ((part & 3) == 2 ? w.z : w.w));
    (void)bias;
    if (kWide) {
      *(uint4 *)(bt) = dequantise_word_wide(word, scale, -7.5f * scale);
    } else {
      const _Float16 shift = (_Float16)(-centre_of(scale));
      const f16x2 scale2 = {(_Float16)scale, (_Float16)scale}, shift2 = {shift, shift};
      *(uint4 *)(bt) = dequantise_word(word, scale2, shift2);
    }
  };

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // prologue: step 0 staged, weights of step 1 in flight
  stage_a(0, 0);
  fetch_w(0);
  w_now[0] = w_next[0];
  w_now[1] = w_next[1];
  affine_now = affine_next;
  sum_now = sum_next;
  fetch_w(1);
  for (int part = 0; part < 8; ++part) stage_b(0, part);
  stage_side(0);
  __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): this wave's rows have landed in LDS
  __syncthreads();
  const uint32_t swizzle = (l32 >> 1) & 7;
  // One K step on LDS buffer kBuffer (= step & 1); the loop below runs them in pairs so that the
  // buffer, and the centring update after every second step, are fixed at compile time.
  auto k_step = [&](uint32_t step, auto parity) {
    constexpr uint32_t buffer = decltype(parity)::value;
    stage_a(buffer ^ 1, min(step + 1, steps - 1));
    w_now[0] = w_next[0];   // weights of step+1: requested a whole step ago
    w_now[1] = w_next[1];
    affine_now = affine_next;
    sum_now = sum_next;
    fetch_w(step + 2);
    const unsigned char *at = a_tiles + buffer * kATileBytes + (128 * wm + l32) * 128;
    const unsigned char *bt = b_tiles + buffer * kBTileBytes + (128 * wn + l32) * kPitch + 16 * kh;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      f16x8 a_op[4], b_op[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a_op[i] = __builtin_bit_cast(f16x8, *(const uint4 *)(at + 32 * i * 128 + 16 * ((2 * s + kh) ^ swizzle)));
        b_op[i] = __builtin_bit_cast(f16x8, *(const uint4 *)(bt + 32 * i * kPitch + 32 * s));
      }
      // eight MFMAs, then one word of the next step's weights, fenced so that the staging
      // instructions issue in the shadow of the matrix pipe instead of after all sixteen
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_op[i], b_op[j], acc[i][j], 0, 0, 0);
        if (i & 1) {
          __builtin_amdgcn_sched_barrier(0);
          stage_b(buffer ^ 1, 2 * s + (i >> 1));
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    // after the second step of a pair: the centring terms of the two groups just multiplied,
    // as one f32 MFMA per accumulator tile (lane half kh supplies group step - 1 + kh of both
    // operands)
    if (buffer == 1) {
      float row_sum[4], column_offset[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        row_sum[i] = side_rows[((step - 1 + kh) & 3) * kBM + 128 * wm + 32 * i + l32];
        column_offset[i] = side_cols[((step - 1 + kh) & 3) * kBN + 128 * wn + 32 * i + l32];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(row_sum[i], column_offset[j], acc[i][j], 0, 0, 0);
    }
    stage_side(step + 1);   // a ring slot nobody reads in this step
    __builtin_amdgcn_s_waitcnt(0x0f75);   // vmcnt(5): all but the five loads of fetch_w just issued
    __syncthreads();
  };
  for (uint32_t step = 0; step < steps; step += 2) {   // K is a multiple of 256: steps is even
    k_step(step, std::integral_constant<uint32_t, 0>{});
    k_step(step + 1, std::integral_constant<uint32_t, 1>{});
  }
  // store: lane (column l32, half kh) holds rows 8*(r/4) + 4*kh + r%4 of each 32 x 32 tile
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t column = col0 + 128 * wn + 32 * j + l32;
      if (column >= a.columns) continue;
      for (int r = 0; r < 16; ++r) {
        const uint32_t row = row0 + 128 * wm + 32 * i + 8 * (r / 4) + 4 * kh + (r % 4);
        if (row >= a.rows) continue;
        const uint64_t at_out = (uint64_t)row * a.out_row_stride + column;
        const float value = acc[i][j][r] * a.row_unscale[row];
        if (a.out_f32)
          ((float *)a.out)[at_out] = value;
        else
          ((uint16_t *)a.out)[at_out] = (uint16_t)(pack2(value, 0.0f) & 0xffffu);
      }
    }
}

}  // namespace

bool launch_quant_gemm(fh_backend *backend, const QmmProblem &p) {
  const uint64_t rows_bytes = ((uint64_t)p.rows * p.inner * 2 + 255) / 256 * 256;
  const uint64_t unscale_bytes = ((uint64_t)p.rows * sizeof(float) + 255) / 256 * 256;
  const uint64_t sums_bytes = ((uint64_t)p.rows * (p.inner / kBK) * sizeof(float) + 255) / 256 * 256;
  char *ws = backend_workspace(backend, rows_bytes + unscale_bytes + sums_bytes + 256);
  if (!ws) return false;
  hipStream_t stream = backend_stream(backend);
  GemmArgs a{};
  a.x = (const uint16_t *)ws;
  a.row_unscale = (const float *)(ws + rows_bytes);
  a.group_sums = (const float *)(ws + rows_bytes + unscale_bytes);
  a.x_row_stride = p.inner;
  a.packed = (const uint32_t *)p.packed.base + p.packed.offset;
  a.scales = (const uint16_t *)p.scales.base + p.scales.offset;
  a.biases = (const uint16_t *)p.biases.base + p.biases.offset;
  a.out = p.out.dtype == FH_F32 ? (void *)((float *)p.out.base + p.out.offset)
                                : (void *)((uint16_t *)p.out.base + p.out.offset);
  a.out_row_stride = p.out.stride[0];
  a.out_f32 = p.out.dtype == FH_F32;
  a.rows = p.rows;
  a.inner = p.inner;
  a.columns = p.columns;
  a.row_tiles = (p.rows + kBM - 1) / kBM;
  a.column_tiles = (p.columns + kBN - 1) / kBN;
  uint32_t *flag = (uint32_t *)(ws + rows_bytes + unscale_bytes + sums_bytes);
  a.wide_flag = flag;
  static bool configured = false;   // raise the dynamic LDS limit once per process
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void *>(&qmm_gemm_kernel<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLds) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void *>(&qmm_gemm_kernel<true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kGemmLds) != hipSuccess)
      return false;
    configured = true;
  }
  const uint32_t grid = (a.row_tiles * a.column_tiles + 255) / 256 * 256;
  KernelTimer timer(backend, FH_KC_QMM_KERNEL);
  prepare_rows_kernel<<<(p.rows + 3) / 4, 256, 0, stream>>>(
      (const uint16_t *)p.x.base + p.x.offset, p.x.stride[0], p.rows, p.inner, (uint16_t *)ws,
      (float *)(ws + rows_bytes), (float *)(ws + rows_bytes + unscale_bytes));
  launch_fill_u32(stream, flag, 1, 0);
  const uint64_t affine_count = (uint64_t)p.columns * (p.inner / kBK);
  check_affine_kernel<<<(uint32_t)((affine_count + 255) / 256), 256, 0, stream>>>(a.scales, a.biases,
                                                                                 affine_count, flag);
  qmm_gemm_kernel<false><<<grid, 256, kGemmLds, stream>>>(a);
  qmm_gemm_kernel<true><<<grid, 256, kGemmLds, stream>>>(a);
  return true;
}

}  // namespace fh
