// Strided, any-dtype kernels that follow the reference backend's loop order
// (crates/forja-cpu/src/lib.rs).  They are the completeness path: every legal operand layout and
// dtype lands here unless a specialised kernel claims it.  Compiled with -ffp-contract=off so a
// dot product is the same mul-then-add chain as the reference's `sum + input * weight`.
#include "kernels.hpp"

namespace fh {

namespace {

constexpr int kBlock = 256;

inline dim3 grid_for(uint64_t work, int block = kBlock) {
  uint64_t blocks = (work + block - 1) / block;
  if (blocks == 0) blocks = 1;
  return dim3((unsigned)blocks);
}

__device__ inline float wave_sum(float v) {
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
  return v;
}

__device__ inline float wave_max(float v) {
  for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, 64));
  return v;
}

// ---------------------------------------------------------------- copy (lib.rs:171-187)

__global__ void copy_kernel(View in, View out, uint64_t elements) {
  uint64_t linear = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (linear >= elements) return;
  uint64_t src = view_offset(in, linear), dst = view_offset(out, linear);
  if (in.dtype == FH_I32 || in.dtype == FH_U32) {
    ((uint32_t *)out.base)[dst] = ((const uint32_t *)in.base)[src];
  } else {
    store_float_at(out, dst, load_float_at(in, src));
  }
}

// Same dtype, both sides dense and 16-byte aligned: a flat copy, 16 bytes per thread per trip.
__global__ __launch_bounds__(256) void copy_flat_kernel(const uint4 *in, uint4 *out, uint64_t pieces) {
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < pieces; i += stride)
    out[i] = in[i];
}

// ---------------------------------------------------------------- scalar programs

__device__ inline uint32_t saturating_u32(float value) {
  if (!(value > 0.0f)) return 0u;  // NaN and non-positive
  if (value >= 4294967296.0f) return 0xffffffffu;
  return (uint32_t)value;
}

__device__ inline float propagating_min(float l, float r) {
  return (l != l || r != r) ? __uint_as_float(0x7fc00000u) : fminf(l, r);
}

__device__ inline float propagating_max(float l, float r) {
  return (l != l || r != r) ? __uint_as_float(0x7fc00000u) : fmaxf(l, r);
}

// Evaluates one non-reduce instruction (crates/forja-cpu/src/interpreter.rs:209-396).
__device__ inline uint32_t eval_inst(const DInst inst, const uint32_t *vals, const ProgramArgs &p,
                                     uint64_t linear) {
  switch (inst.kind) {
  case 0: {
    const View &v = p.inputs[inst.a];
    uint64_t off = view_offset(v, linear);
    if (v.dtype == FH_U32) return load_u32_at(v, off);
    return __float_as_uint(load_float_at(v, off));
  }
  case 1: return inst.a;
  case 2: {
    uint64_t rem = linear;
    uint32_t coordinate = 0;
    for (int axis = (int)p.rank - 1; axis >= 0; --axis) {
      coordinate = (uint32_t)(rem % p.shape[axis]);
      rem /= p.shape[axis];
      if (axis == (int)inst.op) break;
    }
    return coordinate;
  }
  case 3: return p.shape[inst.op];
  case 4: {
    float x = __uint_as_float(vals[inst.a]), y;
    switch (inst.op) {
    case 0: y = -x; break;
    case 1: y = fabsf(x); break;
    case 2: case 13: y = expf(x); break;
    case 3: y = logf(x); break;
    case 4: y = sqrtf(x); break;
    case 5: y = 1.0f / sqrtf(x); break;
    case 6: y = sinf(x); break;
    case 7: y = cosf(x); break;
    case 8: y = tanhf(x); break;
    case 9: y = 1.0f / (1.0f + expf(-x)); break;
    case 10: y = 1.0f / x; break;
    case 11: y = floorf(x); break;
    default: y = log1pf(x); break;
    }
    return __float_as_uint(y);
  }
  case 5: {
    if (inst.ty == 0) {
      float a = __uint_as_float(vals[inst.a]), b = __uint_as_float(vals[inst.b]);
      switch (inst.op) {
      case 0: return __float_as_uint(a + b);
      case 1: return __float_as_uint(a - b);
      case 2: return __float_as_uint(a * b);
      case 3: return __float_as_uint(a / b);
      case 4: return __float_as_uint(propagating_min(a, b));
      case 5: return __float_as_uint(propagating_max(a, b));
      case 6: return __float_as_uint(powf(a, b));
      case 7: return a < b;
      case 8: return a <= b;
      case 9: return a == b;
      case 10: return a != b;
      case 11: return a >= b;
      default: return a > b;
      }
    }
    uint32_t a = vals[inst.a], b = vals[inst.b];
    switch (inst.op) {
    case 0: return a + b;
    case 1: return a - b;
    case 2: return a * b;
    case 4: return a < b ? a : b;
    case 5: return a > b ? a : b;
    case 7: return a < b;
    case 8: return a <= b;
    case 9: return a == b;
    case 10: return a != b;
    case 11: return a >= b;
    default: return a > b;
    }
  }
  case 6: return vals[inst.a] ? vals[inst.b] : vals[inst.c];
  default: {  // cast: op = target type, ty = source type
    uint32_t raw = vals[inst.a];
    if (inst.op == 0) {
      if (inst.ty == 0) return raw;
      if (inst.ty == 1) return __float_as_uint((float)raw);
      return __float_as_uint(raw ? 1.0f : 0.0f);
    }
    if (inst.op == 1) {
      if (inst.ty == 0) return saturating_u32(__uint_as_float(raw));
      if (inst.ty == 1) return raw;
      return raw ? 1u : 0u;
    }
    if (inst.ty == 0) return __uint_as_float(raw) != 0.0f;
    return raw != 0;
  }
  }
}

__global__ void program_map_kernel(ProgramArgs p, uint64_t elements) {
  uint64_t linear = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (linear >= elements) return;
  uint32_t vals[256];
  for (uint32_t i = 0; i < p.n_insts; ++i) vals[i] = eval_inst(p.insts[i], vals, p, linear);
  for (uint32_t pair = 0; pair < p.n_pairs; ++pair) {
    const View &out = p.outputs[p.out_slot[pair]];
    store_float_at(out, view_offset(out, linear), __uint_as_float(vals[p.out_value[pair]]));
  }
}

// One workgroup per row.  Pass r evaluates the prefix up to reduction r with earlier reductions
// already known, folds the operand across the row, and publishes the broadcast value.  The fold
// is a tree, not the reference's left-to-right order (allowed: program.rs:8-10).
__global__ void program_row_kernel(ProgramArgs p) {
  __shared__ float reduced[kMaxReductions];
  __shared__ float partial[kBlock / 64];
  uint32_t width = p.shape[p.rank - 1];
  uint64_t row_start = (uint64_t)blockIdx.x * width;
  uint32_t vals[256];
  for (uint32_t pass = 0; pass <= p.n_reduce; ++pass) {
    uint32_t end = pass < p.n_reduce ? p.reduce_at[pass] : p.n_insts;
    uint32_t red_op = pass < p.n_reduce ? p.insts[end].op : 0;
    uint32_t red_src = pass < p.n_reduce ? p.insts[end].a : 0;
    float acc = 0.0f;
    bool have = false;
    for (uint32_t lane = threadIdx.x; lane < width; lane += blockDim.x) {
      uint64_t linear = row_start + lane;
      uint32_t next_reduce = 0;
      for (uint32_t i = 0; i < end; ++i) {
        DInst inst = p.insts[i];
        if (inst.kind == 8) {
          vals[i] = __float_as_uint(reduced[next_reduce++]);
        } else {
          vals[i] = eval_inst(inst, vals, p, linear);
        }
      }
      if (pass < p.n_reduce) {
        float v = __uint_as_float(vals[red_src]);
        if (!have) {
          acc = v;
          have = true;
        } else if (red_op == 0) {
          acc += v;
        } else if (red_op == 1) {
          acc = propagating_max(acc, v);
        } else {
          acc = propagating_min(acc, v);
        }
      } else {
        for (uint32_t pair = 0; pair < p.n_pairs; ++pair) {
          const View &out = p.outputs[p.out_slot[pair]];
          store_float_at(out, view_offset(out, linear), __uint_as_float(vals[p.out_value[pair]]));
        }
      }
    }
    if (pass < p.n_reduce) {
      // Threads with no element carry the identity of the fold.
      float identity = red_op == 0 ? 0.0f
                                   : (red_op == 1 ? -__builtin_inff() : __builtin_inff());
      if (!have) acc = identity;
      for (int offset = 32; offset > 0; offset >>= 1) {
        float other = __shfl_xor(acc, offset, 64);
        acc = red_op == 0 ? acc + other
                          : (red_op == 1 ? propagating_max(acc, other)
                                         : propagating_min(acc, other));
      }
      if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
      __syncthreads();
      if (threadIdx.x == 0) {
        float total = partial[0];
        for (uint32_t w = 1; w < blockDim.x / 64; ++w) {
          float other = partial[w];
          total = red_op == 0 ? total + other
                              : (red_op == 1 ? propagating_max(total, other)
                                             : propagating_min(total, other));
        }
        reduced[pass] = total;
      }
      __syncthreads();
    }
  }
}

// ---------------------------------------------------------------- quantised matmul

// affine_quant_dot (lib.rs:1277-1310) on strided rank-1 slices.
__device__ inline float quant_dot(const View &x, uint64_t x_base, uint64_t x_stride,
                                  const uint32_t *packed, uint64_t packed_base,
                                  uint64_t packed_stride, const View &scales, const View &biases,
                                  uint64_t scale_base, uint64_t scale_stride, uint64_t bias_base,
                                  uint64_t bias_stride, uint32_t inner, uint32_t bits,
                                  uint32_t group) {
  uint32_t values_per_word = 32u / bits;
  uint32_t mask = (1u << bits) - 1u;
  float sum = 0.0f;
  float scale = 0.0f, bias = 0.0f;
  uint32_t word = 0;
  for (uint32_t index = 0; index < inner; ++index) {
    if (index % values_per_word == 0)
      word = packed[packed_base + (uint64_t)(index / values_per_word) * packed_stride];
    if (index % group == 0) {
      scale = load_float_at(scales, scale_base + (uint64_t)(index / group) * scale_stride);
      bias = load_float_at(biases, bias_base + (uint64_t)(index / group) * bias_stride);
    }
    uint32_t quantized = (word >> ((index % values_per_word) * bits)) & mask;
    float weight = scale * (float)quantized + bias;
    sum = sum + load_float_at(x, x_base + (uint64_t)index * x_stride) * weight;
  }
  return sum;
}

__global__ void quant_matmul_generic_kernel(View x, View packed, View scales, View biases,
                                            View out, uint32_t rows, uint32_t inner,
                                            uint32_t columns, uint32_t bits, uint32_t group) {
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)rows * columns) return;
  uint32_t row = (uint32_t)(flat / columns), column = (uint32_t)(flat % columns);
  float value = quant_dot(x, x.offset + row * x.stride[0], x.stride[1],
                          (const uint32_t *)packed.base,
                          packed.offset + column * packed.stride[0], packed.stride[1], scales,
                          biases, scales.offset + column * scales.stride[0], scales.stride[1],
                          biases.offset + column * biases.stride[0], biases.stride[1], inner, bits,
                          group);
  store_float_at(out, out.offset + row * out.stride[0] + column * out.stride[1], value);
}

// gather_quant_projection_values (lib.rs:1025-1106): out [R,k,N].
__global__ void gather_projection_generic_kernel(View x, View packed, View scales, View biases,
                                                 View indices, View out, uint32_t rows,
                                                 uint32_t inner, uint32_t experts,
                                                 uint32_t columns, uint32_t k, uint32_t bits,
                                                 uint32_t group, ErrorSlot *error) {
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)rows * k * columns) return;
  uint32_t column = (uint32_t)(flat % columns);
  uint32_t route = (uint32_t)(flat / columns);
  uint32_t row = route / k, slot = route % k;
  uint32_t expert =
      load_u32_at(indices, indices.offset + row * indices.stride[0] + slot * indices.stride[1]);
  uint64_t out_at = out.offset + row * out.stride[0] + slot * out.stride[1] +
                    column * out.stride[2];
  if (expert >= experts) {
    if (column == 0) report_error(error, expert);
    store_float_at(out, out_at, 0.0f);
    return;
  }
  float value = quant_dot(
      x, x.offset + row * x.stride[0], x.stride[1], (const uint32_t *)packed.base,
      packed.offset + expert * packed.stride[0] + column * packed.stride[1], packed.stride[2],
      scales, biases, scales.offset + expert * scales.stride[0] + column * scales.stride[1],
      scales.stride[2], biases.offset + expert * biases.stride[0] + column * biases.stride[1],
      biases.stride[2], inner, bits, group);
  store_float_at(out, out_at, value);
}

// execute_gather_quant_weighted_sum (lib.rs:1108-1204): routes folded in ascending slot order.
__global__ void gather_weighted_generic_kernel(View x, View packed, View scales, View biases,
                                               View indices, View weights, View out,
                                               uint32_t rows, uint32_t routes, uint32_t inner,
                                               uint32_t experts, uint32_t columns, uint32_t bits,
                                               uint32_t group, ErrorSlot *error) {
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)rows * columns) return;
  uint32_t row = (uint32_t)(flat / columns), column = (uint32_t)(flat % columns);
  float value = 0.0f;
  for (uint32_t slot = 0; slot < routes; ++slot) {
    uint32_t expert =
        load_u32_at(indices, indices.offset + row * indices.stride[0] + slot * indices.stride[1]);
    if (expert >= experts) {
      if (column == 0) report_error(error, expert);
      continue;
    }
    float weight = load_float_at(
        weights, weights.offset + row * weights.stride[0] + slot * weights.stride[1]);
    float dot = quant_dot(
        x, x.offset + row * x.stride[0] + slot * x.stride[1], x.stride[2],
        (const uint32_t *)packed.base,
        packed.offset + expert * packed.stride[0] + column * packed.stride[1], packed.stride[2],
        scales, biases, scales.offset + expert * scales.stride[0] + column * scales.stride[1],
        scales.stride[2], biases.offset + expert * biases.stride[0] + column * biases.stride[1],
        biases.stride[2], inner, bits, group);
    value += weight * dot;
  }
  store_float_at(out, out.offset + row * out.stride[0] + column * out.stride[1], value);
}

// ---------------------------------------------------------------- selection

struct Candidate {
  int32_t key;
  uint32_t index;
};

// Order used by top-k: greater key first, then lower index (lib.rs:575-579).
__device__ inline bool before(Candidate l, Candidate r) {
  return l.key > r.key || (l.key == r.key && l.index < r.index);
}

// One wave per row.  Selection i is the first element, in (key desc, index asc) order, that
// comes strictly after selection i-1; no scratch storage is needed.
__global__ void top_k_kernel(View in, View values, View indices, uint32_t rows, uint32_t width,
                             uint32_t k, int normalize) {
  __shared__ float selected[256];
  uint32_t row = blockIdx.x;
  uint32_t lane = threadIdx.x;
  uint64_t in_row = in.offset + (uint64_t)row * in.stride[0];
  Candidate previous = {0, 0};
  for (uint32_t slot = 0; slot < k; ++slot) {
    Candidate best = {(int32_t)0x80000000, 0xffffffffu};
    bool have = false;
    for (uint32_t index = lane; index < width; index += 64) {
      Candidate c = {total_key(load_float_at(in, in_row + (uint64_t)index * in.stride[1])), index};
      if (slot > 0 && !before(previous, c)) continue;
      if (!have || before(c, best)) {
        best = c;
        have = true;
      }
    }
    for (int offset = 32; offset > 0; offset >>= 1) {
      Candidate other;
      other.key = __shfl_xor(best.key, offset, 64);
      other.index = __shfl_xor(best.index, offset, 64);
      int other_have = __shfl_xor((int)have, offset, 64);
      if (other_have && (!have || before(other, best))) {
        best = other;
        have = true;
      }
    }
    previous = best;
    if (lane == 0) {
      float value = load_float_at(in, in_row + (uint64_t)best.index * in.stride[1]);
      selected[slot] = value;
      ((uint32_t *)indices.base)[indices.offset + (uint64_t)row * indices.stride[0] +
                                 (uint64_t)slot * indices.stride[1]] = best.index;
    }
  }
  if (lane == 0) {
    if (normalize) {
      float maximum = selected[0];
      float sum = 0.0f;
      for (uint32_t slot = 0; slot < k; ++slot) {
        selected[slot] = expf(selected[slot] - maximum);
        sum += selected[slot];
      }
      for (uint32_t slot = 0; slot < k; ++slot) selected[slot] /= sum;
    }
    for (uint32_t slot = 0; slot < k; ++slot)
      store_float_at(values,
                     values.offset + (uint64_t)row * values.stride[0] +
                         (uint64_t)slot * values.stride[1],
                     selected[slot]);
  }
}

// Rows of at most 64 * kPer values (router logits): the whole row is loaded once into registers
// and the k selections run on registers only.  Same order and results as top_k_kernel.
template <int kPer>
__global__ void top_k_registers_kernel(View in, View values, View indices, uint32_t rows,
                                       uint32_t width, uint32_t k, int normalize) {
  __shared__ float selected[64 * kPer];
  const uint32_t row = blockIdx.x, lane = threadIdx.x;
  const uint64_t in_row = in.offset + (uint64_t)row * in.stride[0];
  // A candidate is one 64-bit word that orders like (key descending, index ascending): the key
  // mapped to unsigned order in the high half, the complemented index in the low half; 0 stands
  // for "none" (no element has index 0xffffffff).  A selection is then a 64-bit maximum.
  unsigned long long word[kPer];
#pragma unroll
  for (int i = 0; i < kPer; ++i) {
    const uint32_t index = lane + 64 * i;
    word[i] = 0;
    if (index < width) {
      const int32_t key = total_key(load_float_at(in, in_row + (uint64_t)index * in.stride[1]));
      word[i] = ((unsigned long long)((uint32_t)key ^ 0x80000000u) << 32) | (uint32_t)~index;
    }
  }
  for (uint32_t slot = 0; slot < k; ++slot) {
    unsigned long long best = word[0];
#pragma unroll
    for (int i = 1; i < kPer; ++i) best = word[i] > best ? word[i] : best;
    for (int offset = 32; offset > 0; offset >>= 1) {
      const unsigned long long other = __shfl_xor(best, offset, 64);
      best = other > best ? other : best;
    }
    // the owner retires the selected element
#pragma unroll
    for (int i = 0; i < kPer; ++i)
      if (word[i] == best) word[i] = 0;
    if (lane == 0) {
      const int32_t key = (int32_t)((uint32_t)(best >> 32) ^ 0x80000000u);
      const int32_t bits = key ^ (int32_t)(((uint32_t)(key >> 31)) >> 1);
      selected[slot] = __uint_as_float((uint32_t)bits);
      ((uint32_t *)indices.base)[indices.offset + (uint64_t)row * indices.stride[0] +
                                 (uint64_t)slot * indices.stride[1]] = ~(uint32_t)best;
    }
  }
  if (lane == 0) {
    if (normalize) {
      float maximum = selected[0];
      float sum = 0.0f;
      for (uint32_t slot = 0; slot < k; ++slot) {
        selected[slot] = expf(selected[slot] - maximum);
        sum += selected[slot];
      }
      for (uint32_t slot = 0; slot < k; ++slot) selected[slot] /= sum;
    }
    for (uint32_t slot = 0; slot < k; ++slot)
      store_float_at(values,
                     values.offset + (uint64_t)row * values.stride[0] +
                         (uint64_t)slot * values.stride[1],
                     selected[slot]);
  }
}

// Highest index among equal maxima under total order (lib.rs:530-539).
__global__ void argmax_kernel(View in, View out, uint32_t rows, uint32_t width) {
  __shared__ int32_t keys[kBlock / 64];
  __shared__ uint32_t idxs[kBlock / 64];
  uint32_t row = blockIdx.x;
  uint64_t in_row = in.offset + (uint64_t)row * in.stride[0];
  int32_t best_key = (int32_t)0x80000000;
  uint32_t best_index = 0;
  bool have = false;
  for (uint32_t index = threadIdx.x; index < width; index += blockDim.x) {
    int32_t key = total_key(load_float_at(in, in_row + (uint64_t)index * in.stride[1]));
    if (!have || key >= best_key) {
      best_key = key;
      best_index = index;
      have = true;
    }
  }
  for (int offset = 32; offset > 0; offset >>= 1) {
    int32_t other_key = __shfl_xor(best_key, offset, 64);
    uint32_t other_index = __shfl_xor(best_index, offset, 64);
    int other_have = __shfl_xor((int)have, offset, 64);
    if (other_have &&
        (!have || other_key > best_key || (other_key == best_key && other_index > best_index))) {
      best_key = other_key;
      best_index = other_index;
      have = true;
    }
  }
  // Every wave has at least lane 0 active with an element unless width < 64*wave; mark empties.
  if ((threadIdx.x & 63) == 0) {
    keys[threadIdx.x >> 6] = best_key;
    idxs[threadIdx.x >> 6] = have ? best_index : 0xffffffffu;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t key = keys[0];
    uint32_t index = idxs[0];
    for (uint32_t w = 1; w < blockDim.x / 64; ++w) {
      if (idxs[w] == 0xffffffffu) continue;
      if (index == 0xffffffffu || keys[w] > key || (keys[w] == key && idxs[w] > index)) {
        key = keys[w];
        index = idxs[w];
      }
    }
    ((uint32_t *)out.base)[view_offset(out, row)] = index;
  }
}

// bf16 or f32 (kWide) rows with a contiguous innermost axis: 16-byte loads of data read once,
// 1024 threads per row, eight consecutive elements a thread and step, in ascending order.
template <bool kWide>
__global__ __launch_bounds__(1024) void argmax_rows_kernel(const void *in, uint64_t row_stride,
                                                           View out, uint32_t width) {
  __shared__ int32_t keys[16];
  __shared__ uint32_t idxs[16];
  const uint32_t row = blockIdx.x;
  int32_t best_key = (int32_t)0x80000000;
  uint32_t best_index = 0xffffffffu;
  for (uint32_t c = threadIdx.x * 8; c < width; c += 1024 * 8) {
    float value[8];
    if constexpr (kWide) {
      const float *x = (const float *)in + (uint64_t)row * row_stride + c;
      const uint4 a = stream_load(x), b = stream_load(x + 4);
      const uint32_t words[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      for (int i = 0; i < 8; ++i) value[i] = __uint_as_float(words[i]);
    } else {
      const uint4 v = stream_load((const uint16_t *)in + (uint64_t)row * row_stride + c);
      const uint32_t words[4] = {v.x, v.y, v.z, v.w};
      for (int i = 0; i < 4; ++i) {
        value[2 * i] = __uint_as_float(words[i] << 16);
        value[2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u);
      }
    }
    for (int i = 0; i < 8; ++i) {
      const int32_t key = total_key(value[i]);
      if (best_index == 0xffffffffu || key >= best_key) {
        best_key = key;
        best_index = c + i;
      }
    }
  }
  for (int offset = 32; offset > 0; offset >>= 1) {
    int32_t other_key = __shfl_xor(best_key, offset, 64);
    uint32_t other_index = __shfl_xor(best_index, offset, 64);
    if (other_index != 0xffffffffu &&
        (best_index == 0xffffffffu || other_key > best_key ||
         (other_key == best_key && other_index > best_index))) {
      best_key = other_key;
      best_index = other_index;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    keys[threadIdx.x >> 6] = best_key;
    idxs[threadIdx.x >> 6] = best_index;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t key = keys[0];
    uint32_t index = idxs[0];
    for (uint32_t w = 1; w < 16; ++w) {
      if (idxs[w] == 0xffffffffu) continue;
      if (index == 0xffffffffu || keys[w] > key || (keys[w] == key && idxs[w] > index)) {
        key = keys[w];
        index = idxs[w];
      }
    }
    ((uint32_t *)out.base)[view_offset(out, row)] = index;
  }
}

// ---------------------------------------------------------------- glue

// execute_quant_embed (lib.rs:748-813).
__global__ void quant_embed_kernel(View packed, View scales, View biases, View ids, View out,
                                   uint32_t id_count, uint32_t vocab, uint32_t packed_width,
                                   uint32_t bits, uint32_t group, ErrorSlot *error) {
  uint32_t values_per_word = 32u / bits;
  uint32_t width = packed_width * values_per_word;
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)id_count * width) return;
  uint32_t item = (uint32_t)(flat / width), column = (uint32_t)(flat % width);
  uint32_t id = load_u32_at(ids, view_offset(ids, item));
  uint64_t out_at = view_offset(out, flat);
  if (id >= vocab) {
    if (column == 0) report_error(error, id);
    store_float_at(out, out_at, 0.0f);
    return;
  }
  uint32_t word = load_u32_at(packed, packed.offset + (uint64_t)id * packed.stride[0] +
                                          (uint64_t)(column / values_per_word) * packed.stride[1]);
  uint32_t quantized = (word >> ((column % values_per_word) * bits)) & ((1u << bits) - 1u);
  float scale = load_float_at(scales, scales.offset + (uint64_t)id * scales.stride[0] +
                                          (uint64_t)(column / group) * scales.stride[1]);
  float bias = load_float_at(biases, biases.offset + (uint64_t)id * biases.stride[0] +
                                         (uint64_t)(column / group) * biases.stride[1]);
  store_float_at(out, out_at, scale * (float)quantized + bias);
}

// execute_matmul (lib.rs:815-848); operands viewed as [B,M,K] x [B,K,N] with batch stride 0 for
// rank two.
__global__ void matmul_kernel(View left, View right, View out, uint32_t batches, uint32_t rows,
                              uint32_t inner, uint32_t columns) {
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)batches * rows * columns) return;
  uint32_t column = (uint32_t)(flat % columns);
  uint32_t row = (uint32_t)((flat / columns) % rows);
  uint32_t batch = (uint32_t)(flat / ((uint64_t)columns * rows));
  int r = (int)left.rank;
  uint64_t lb = r == 3 ? left.stride[0] : 0, rb = r == 3 ? right.stride[0] : 0,
           ob = r == 3 ? out.stride[0] : 0;
  uint64_t l_at = left.offset + batch * lb + row * left.stride[r - 2];
  uint64_t r_at = right.offset + batch * rb + column * right.stride[r - 1];
  float sum = 0.0f;
  for (uint32_t index = 0; index < inner; ++index)
    sum = sum + load_float_at(left, l_at + (uint64_t)index * left.stride[r - 1]) *
                    load_float_at(right, r_at + (uint64_t)index * right.stride[r - 2]);
  store_float_at(out, out.offset + batch * ob + row * out.stride[r - 2] +
                          column * out.stride[r - 1],
                 sum);
}

// execute_rms_norm (lib.rs:495-517); one workgroup per row, tree reduction.
__global__ void rms_norm_kernel(View in, View weight, View out, uint32_t rows, uint32_t width,
                                float eps) {
  __shared__ float partial[kBlock / 64];
  __shared__ float scale_shared;
  uint64_t row_start = (uint64_t)blockIdx.x * width;
  float acc = 0.0f;
  for (uint32_t lane = threadIdx.x; lane < width; lane += blockDim.x) {
    float v = load_float_at(in, view_offset(in, row_start + lane));
    acc += v * v;
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.0f;
    for (uint32_t w = 0; w < blockDim.x / 64; ++w) total += partial[w];
    scale_shared = 1.0f / sqrtf(total / (float)width + eps);
  }
  __syncthreads();
  float scale = scale_shared;
  for (uint32_t lane = threadIdx.x; lane < width; lane += blockDim.x) {
    float v = load_float_at(in, view_offset(in, row_start + lane));
    float w = load_float_at(weight, view_offset(weight, lane));
    store_float_at(out, view_offset(out, row_start + lane), v * scale * w);
  }
}

// execute_rope (lib.rs:681-710): in/out [rows, heads, width], half-split pairs.
__global__ void rope_kernel(View in, View positions, View out, uint32_t rows, uint32_t heads,
                            uint32_t width, float theta) {
  uint32_t half = width / 2;
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)rows * heads * half) return;
  uint32_t index = (uint32_t)(flat % half);
  uint32_t head = (uint32_t)((flat / half) % heads);
  uint32_t row = (uint32_t)(flat / ((uint64_t)half * heads));
  uint32_t position = load_u32_at(positions, view_offset(positions, row));
  float frequency = 1.0f / powf(theta, 2.0f * (float)index / (float)width);
  float angle = (float)position * frequency;
  float s = sinf(angle), c = cosf(angle);
  uint64_t base = ((uint64_t)row * heads + head) * width;
  float first = load_float_at(in, view_offset(in, base + index));
  float second = load_float_at(in, view_offset(in, base + index + half));
  store_float_at(out, view_offset(out, base + index), first * c - second * s);
  store_float_at(out, view_offset(out, base + index + half), second * c + first * s);
}

// ---------------------------------------------------------------- paged storage

// Entry valid iff page < P and generations[page] == entry.generation
// (crates/forja-core/src/paged.rs validate_entry).  Never dereferences a bad entry.
__device__ inline bool resolve_page(const View &table, const View &generations,
                                    uint32_t logical_page, uint32_t logical_pages,
                                    uint32_t physical_pages, uint32_t *physical) {
  if (logical_page >= logical_pages) return false;
  uint64_t at = table.offset + (uint64_t)logical_page * table.stride[0];
  uint32_t page = load_u32_at(table, at);
  uint32_t generation = load_u32_at(table, at + table.stride[1]);
  if (page >= physical_pages) return false;
  if (load_u32_at(generations, generations.offset + (uint64_t)page * generations.stride[0]) !=
      generation)
    return false;
  *physical = page;
  return true;
}

__device__ inline bool lane_active(const View &activity) {
  return activity.base == nullptr || load_u32_at(activity, activity.offset) != 0;
}

// execute_paged_copy (lib.rs:189-260) without the reference's whole-pool round trip.
__global__ void paged_copy_kernel(View ordinary, View pool, View table, View generations,
                                  View activity, int into_pages, uint32_t tokens,
                                  uint32_t elements, uint32_t start, uint32_t page_tokens,
                                  uint32_t physical_pages, uint32_t logical_pages,
                                  ErrorSlot *error) {
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)tokens * elements) return;
  if (!lane_active(activity)) return;
  uint32_t token = (uint32_t)(flat / elements), element = (uint32_t)(flat % elements);
  uint64_t logical = (uint64_t)start + token;
  uint32_t logical_page = (uint32_t)(logical / page_tokens);
  uint32_t physical;
  if (logical / page_tokens > 0xffffffffull ||
      !resolve_page(table, generations, logical_page, logical_pages, physical_pages, &physical)) {
    if (element == 0) report_error(error, logical_page);
    return;
  }
  uint64_t pool_at =
      pool.offset + ((uint64_t)physical * page_tokens + logical % page_tokens) * elements + element;
  uint64_t ordinary_at = view_offset(ordinary, flat);
  if (into_pages)
    store_float_at(pool, pool_at, load_float_at(ordinary, ordinary_at));
  else
    store_float_at(ordinary, ordinary_at, load_float_at(pool, pool_at));
}

// CpuPagePool::sdpa (crates/forja-cpu/src/paged.rs:161-259) for any dtype/width.  One wave per
// (head, query row); each lane keeps an online-softmax state over its stride of keys and the
// states are merged at the end.  q [Hq,Sq,D] and out [Hq,Sq,Dv] are strided views; pools are
// contiguous [P,pt,Hkv,D|Dv].
template <int kMaxDv>
__global__ void paged_sdpa_generic_kernel(View q, View key_pool, View value_pool, View table,
                                          View generations, View activity, View out,
                                          uint32_t query_heads, uint32_t query_length,
                                          uint32_t kv_heads, uint32_t width, uint32_t value_width,
                                          uint32_t key_length, uint32_t query_start, float scale,
                                          int causal, uint32_t page_tokens,
                                          uint32_t physical_pages, uint32_t logical_pages,
                                          ErrorSlot *error) {
  __shared__ float q_row[512];
  __shared__ int bad;
  uint32_t head = blockIdx.x / query_length, query_row = blockIdx.x % query_length;
  uint32_t lane = threadIdx.x;
  uint64_t out_base = out.offset + head * out.stride[0] + query_row * out.stride[1];
  if (!lane_active(activity)) {
    for (uint32_t c = lane; c < value_width; c += 64)
      store_float_at(out, out_base + c * out.stride[2], 0.0f);
    return;
  }
  uint32_t attended = key_length;
  if (causal) {
    uint64_t limit = (uint64_t)query_start + query_row + 1;
    if (limit < attended) attended = (uint32_t)limit;
  }
  if (lane == 0) bad = 0;
  __syncthreads();
  // Authenticate every page this row will touch before any K/V access.
  uint32_t pages = (attended + page_tokens - 1) / page_tokens;
  for (uint32_t page = lane; page < pages; page += 64) {
    uint32_t physical;
    if (!resolve_page(table, generations, page, logical_pages, physical_pages, &physical)) {
      report_error(error, page);
      bad = 1;
    }
  }
  for (uint32_t c = lane; c < width; c += 64)
    q_row[c] = load_float_at(q, q.offset + head * q.stride[0] + query_row * q.stride[1] +
                                    c * q.stride[2]);
  __syncthreads();
  if (bad) {
    for (uint32_t c = lane; c < value_width; c += 64)
      store_float_at(out, out_base + c * out.stride[2], 0.0f);
    return;
  }
  uint32_t kv_head = head / (query_heads / kv_heads);
  float m = -__builtin_inff(), l = 0.0f;
  float acc[kMaxDv];
  for (int c = 0; c < kMaxDv; ++c) acc[c] = 0.0f;
  for (uint32_t key = lane; key < attended; key += 64) {
    uint32_t physical = 0;
    resolve_page(table, generations, key / page_tokens, logical_pages, physical_pages, &physical);
    uint64_t pool_row = (uint64_t)physical * page_tokens + key % page_tokens;
    uint64_t k_at = key_pool.offset + (pool_row * kv_heads + kv_head) * width;
    float score = 0.0f;
    for (uint32_t c = 0; c < width; ++c) score += q_row[c] * load_float_at(key_pool, k_at + c);
    score *= scale;
    float m_new = fmaxf(m, score);
    float correction = m == -__builtin_inff() ? 0.0f : expf(m - m_new);
    float p = expf(score - m_new);
    l = l * correction + p;
    uint64_t v_at = value_pool.offset + (pool_row * kv_heads + kv_head) * value_width;
    for (int c = 0; c < kMaxDv; ++c)
      if ((uint32_t)c < value_width)
        acc[c] = acc[c] * correction + p * load_float_at(value_pool, v_at + c);
    m = m_new;
  }
  float m_all = wave_max(m);
  float factor = (m == -__builtin_inff()) ? 0.0f : expf(m - m_all);
  float l_all = wave_sum(l * factor);
  for (int c = 0; c < kMaxDv; ++c) {
    if ((uint32_t)c >= value_width) break;
    float total = wave_sum(acc[c] * factor);
    if (lane == 0) store_float_at(out, out_base + c * out.stride[2], total / l_all);
  }
}

// ---------------------------------------------------------------- seeded data

__device__ inline uint64_t splitmix64(uint64_t value) {
  value += 0x9e3779b97f4a7c15ull;
  value = (value ^ (value >> 30)) * 0xbf58476d1ce4e5b9ull;
  value = (value ^ (value >> 27)) * 0x94d049bb133111ebull;
  return value ^ (value >> 31);
}

__device__ inline uint64_t stream_u64(uint64_t key, uint64_t index) {
  return splitmix64(key ^ index);
}

__global__ void fill_seeded_kernel(View out, uint64_t elements, uint32_t kind, uint64_t key,
                                   uint64_t first, float lo, float hi) {
  uint64_t linear = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (linear >= elements) return;
  uint64_t index = first + linear;
  uint64_t at = out.offset + linear;
  if (kind == 0) {
    ((uint32_t *)out.base)[at] = (uint32_t)(stream_u64(key, index) >> 32);
    return;
  }
  float value;
  if (kind == 1) {
    float unit = (float)(stream_u64(key, index) >> 40) * (1.0f / 16777216.0f);
    float span = hi - lo;
    float scaled = unit * span;
    value = lo + scaled;
  } else {
    uint64_t a = stream_u64(key, 2 * index), b = stream_u64(key, 2 * index + 1);
    int32_t sum = 0;
    for (int lane = 0; lane < 4; ++lane) {
      sum += (int32_t)((a >> (16 * lane)) & 0xffff);
      sum += (int32_t)((b >> (16 * lane)) & 0xffff);
    }
    value = (float)(sum - 262140) * (1.0f / 53509.91796875f);
  }
  store_float_at(out, at, value);
}

__global__ void fill_u32_kernel(uint32_t *ptr, uint64_t count, uint32_t value) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) ptr[i] = value;
}

__global__ void init_errors_kernel(ErrorSlot *slots, uint32_t count) {
  uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count) {
    slots[i].flag = 0;
    slots[i].value = 0xffffffffu;
  }
}

}  // namespace

// ---------------------------------------------------------------- launchers

void launch_copy(hipStream_t s, const View &in, const View &out, uint64_t elements) {
  if (elements == 0) return;
  auto dense = [](const View &v) {
    uint64_t expected = 1;
    for (int axis = (int)v.rank - 1; axis >= 0; --axis) {
      if (v.shape[axis] != 1 && v.stride[axis] != expected) return false;
      expected *= v.shape[axis];
    }
    return true;
  };
  const uint64_t size = (in.dtype == FH_F16 || in.dtype == FH_BF16) ? 2 : 4;
  if (in.dtype == out.dtype && dense(in) && dense(out) && (elements * size) % 16 == 0 &&
      (in.offset * size) % 16 == 0 && (out.offset * size) % 16 == 0) {
    const uint64_t pieces = elements * size / 16;
    const uint64_t blocks = (pieces + 255) / 256;
    copy_flat_kernel<<<(unsigned)(blocks < 16384 ? blocks : 16384), 256, 0, s>>>(
        (const uint4 *)((const char *)in.base + in.offset * size),
        (uint4 *)((char *)out.base + out.offset * size), pieces);
    return;
  }
  copy_kernel<<<grid_for(elements), kBlock, 0, s>>>(in, out, elements);
}

void launch_program(hipStream_t s, const ProgramArgs &args, bool row, uint64_t elements) {
  if (elements == 0) return;
  if (row) {
    uint32_t width = args.shape[args.rank - 1];
    uint64_t rows = elements / width;
    program_row_kernel<<<dim3((unsigned)rows), kBlock, 0, s>>>(args);
  } else {
    program_map_kernel<<<grid_for(elements), kBlock, 0, s>>>(args, elements);
  }
}

void launch_quant_matmul_generic(hipStream_t s, const View &x, const View &packed,
                                 const View &scales, const View &biases, const View &out,
                                 uint32_t rows, uint32_t inner, uint32_t columns, uint32_t bits,
                                 uint32_t group) {
  uint64_t work = (uint64_t)rows * columns;
  if (work == 0) return;
  quant_matmul_generic_kernel<<<grid_for(work), kBlock, 0, s>>>(x, packed, scales, biases, out,
                                                                rows, inner, columns, bits, group);
}

void launch_gather_projection_generic(hipStream_t s, const View &x, const View &packed,
                                      const View &scales, const View &biases, const View &indices,
                                      const View &out, uint32_t rows, uint32_t inner,
                                      uint32_t experts, uint32_t columns, uint32_t k,
                                      uint32_t bits, uint32_t group, ErrorSlot *error) {
  uint64_t work = (uint64_t)rows * k * columns;
  if (work == 0) return;
  gather_projection_generic_kernel<<<grid_for(work), kBlock, 0, s>>>(
      x, packed, scales, biases, indices, out, rows, inner, experts, columns, k, bits, group,
      error);
}

void launch_gather_weighted_generic(hipStream_t s, const View &x, const View &packed,
                                    const View &scales, const View &biases, const View &indices,
                                    const View &weights, const View &out, uint32_t rows,
                                    uint32_t routes, uint32_t inner, uint32_t experts,
                                    uint32_t columns, uint32_t bits, uint32_t group,
                                    ErrorSlot *error) {
  uint64_t work = (uint64_t)rows * columns;
  if (work == 0) return;
  gather_weighted_generic_kernel<<<grid_for(work), kBlock, 0, s>>>(
      x, packed, scales, biases, indices, weights, out, rows, routes, inner, experts, columns,
      bits, group, error);
}

void launch_top_k(hipStream_t s, const View &in, const View &values, const View &indices,
                  uint32_t rows, uint32_t width, uint32_t k, bool normalize) {
  if (rows == 0) return;
  if (width <= 128) {
    top_k_registers_kernel<2><<<dim3(rows), 64, 0, s>>>(in, values, indices, rows, width, k,
                                                        normalize ? 1 : 0);
    return;
  }
  if (width <= 512) {
    top_k_registers_kernel<8><<<dim3(rows), 64, 0, s>>>(in, values, indices, rows, width, k,
                                                        normalize ? 1 : 0);
    return;
  }
  top_k_kernel<<<dim3(rows), 64, 0, s>>>(in, values, indices, rows, width, k, normalize ? 1 : 0);
}

void launch_argmax(hipStream_t s, const View &in, const View &out, uint32_t rows, uint32_t width) {
  if (rows == 0) return;
  if (in.dtype == FH_BF16 && in.stride[1] == 1 && width % 8 == 0 && in.offset % 8 == 0 &&
      (rows == 1 || in.stride[0] % 8 == 0)) {
    argmax_rows_kernel<false><<<dim3(rows), 1024, 0, s>>>((const uint16_t *)in.base + in.offset,
                                                          in.stride[0], out, width);
    return;
  }
  if (in.dtype == FH_F32 && in.stride[1] == 1 && width % 8 == 0 && in.offset % 4 == 0 &&
      (rows == 1 || in.stride[0] % 4 == 0)) {
    argmax_rows_kernel<true><<<dim3(rows), 1024, 0, s>>>((const float *)in.base + in.offset, in.stride[0],
                                                         out, width);
    return;
  }
  argmax_kernel<<<dim3(rows), kBlock, 0, s>>>(in, out, rows, width);
}

void launch_quant_embed(hipStream_t s, const View &packed, const View &scales,
                        const View &biases, const View &ids, const View &out, uint32_t id_count,
                        uint32_t vocab, uint32_t packed_width, uint32_t bits, uint32_t group,
                        ErrorSlot *error) {
  uint64_t work = (uint64_t)id_count * packed_width * (32u / bits);
  if (work == 0) return;
  quant_embed_kernel<<<grid_for(work), kBlock, 0, s>>>(packed, scales, biases, ids, out, id_count,
                                                       vocab, packed_width, bits, group, error);
}

void launch_matmul(hipStream_t s, const View &left, const View &right, const View &out,
                   uint32_t batches, uint32_t rows, uint32_t inner, uint32_t columns) {
  uint64_t work = (uint64_t)batches * rows * columns;
  if (work == 0) return;
  matmul_kernel<<<grid_for(work), kBlock, 0, s>>>(left, right, out, batches, rows, inner, columns);
}

void launch_rms_norm(hipStream_t s, const View &in, const View &weight, const View &out,
                     uint32_t rows, uint32_t width, float eps) {
  if (rows == 0) return;
  rms_norm_kernel<<<dim3(rows), kBlock, 0, s>>>(in, weight, out, rows, width, eps);
}

void launch_rope(hipStream_t s, const View &in, const View &positions, const View &out,
                 uint32_t rows, uint32_t heads, uint32_t width, float theta) {
  uint64_t work = (uint64_t)rows * heads * (width / 2);
  if (work == 0) return;
  rope_kernel<<<grid_for(work), kBlock, 0, s>>>(in, positions, out, rows, heads, width, theta);
}

void launch_paged_copy(hipStream_t s, const View &ordinary, const View &pool, const View &table,
                       const View &generations, const View &activity, bool into_pages,
                       uint32_t tokens, uint32_t elements, uint32_t start, uint32_t page_tokens,
                       uint32_t physical_pages, uint32_t logical_pages, ErrorSlot *error) {
  uint64_t work = (uint64_t)tokens * elements;
  if (work == 0) return;
  paged_copy_kernel<<<grid_for(work), kBlock, 0, s>>>(ordinary, pool, table, generations, activity,
                                                      into_pages ? 1 : 0, tokens, elements, start,
                                                      page_tokens, physical_pages, logical_pages,
                                                      error);
}

void launch_paged_sdpa_generic(hipStream_t s, const View &q, const View &key_pool,
                               const View &value_pool, const View &table,
                               const View &generations, const View &activity, const View &out,
                               uint32_t query_heads, uint32_t query_length, uint32_t kv_heads,
                               uint32_t width, uint32_t value_width, uint32_t key_length,
                               uint32_t query_start, float scale, bool causal,
                               uint32_t page_tokens, uint32_t physical_pages,
                               uint32_t logical_pages, ErrorSlot *error) {
  uint32_t blocks = query_heads * query_length;
  if (blocks == 0) return;
#define FH_SDPA_ARGS                                                                           \
  q, key_pool, value_pool, table, generations, activity, out, query_heads, query_length,      \
      kv_heads, width, value_width, key_length, query_start, scale, causal ? 1 : 0,           \
      page_tokens, physical_pages, logical_pages, error
  if (value_width <= 64)
    paged_sdpa_generic_kernel<64><<<dim3(blocks), 64, 0, s>>>(FH_SDPA_ARGS);
  else if (value_width <= 128)
    paged_sdpa_generic_kernel<128><<<dim3(blocks), 64, 0, s>>>(FH_SDPA_ARGS);
  else
    paged_sdpa_generic_kernel<256><<<dim3(blocks), 64, 0, s>>>(FH_SDPA_ARGS);
#undef FH_SDPA_ARGS
}

void launch_fill_seeded(hipStream_t s, const View &out, uint64_t elements, uint32_t kind,
                        uint64_t seed, uint64_t stream, uint64_t first, float lo, float hi) {
  if (elements == 0) return;
  // Same key derivation as the oracle's orc_stream_u64.
  uint64_t key = seed + 0x632be59bd9b4e019ull * (stream + 1);
  key += 0x9e3779b97f4a7c15ull;
  key = (key ^ (key >> 30)) * 0xbf58476d1ce4e5b9ull;
  key = (key ^ (key >> 27)) * 0x94d049bb133111ebull;
  key ^= key >> 31;
  fill_seeded_kernel<<<grid_for(elements), kBlock, 0, s>>>(out, elements, kind, key, first, lo,
                                                           hi);
}

void launch_fill_u32(hipStream_t s, uint32_t *ptr, uint64_t count, uint32_t value) {
  if (count == 0) return;
  fill_u32_kernel<<<grid_for(count), kBlock, 0, s>>>(ptr, count, value);
}

void launch_init_errors(hipStream_t s, ErrorSlot *slots, uint32_t count) {
  if (count == 0) return;
  init_errors_kernel<<<grid_for(count), kBlock, 0, s>>>(slots, count);
}

}  // namespace fh
