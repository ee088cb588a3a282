// Fused kernels for the guest programs every engine dispatches around the matmuls
// (crates/forja-sdk/src/nn/blocks.rs:380-443): the row programs rms_norm_rows, residual_norm_rows
// and qk_norm_rope_rows, and the element-wise silu_mul_elements and add_elements.  A program is recognised by its canonical expression (commutative operands
// sorted, constants captured), never by name, so any instruction order the SDK emits matches;
// everything else runs on the generic interpreter.  bf16 rows (the row programs: f32 rows too),
// innermost axis contiguous.
#include "fast_kernels.hpp"

#include <algorithm>
#include <regex>
#include <string>

namespace fh {

namespace {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

__device__ inline uint32_t pack2(float lo, float hi) {
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ inline float lo_f32(uint32_t w) { return __uint_as_float(w << 16); }
__device__ inline float hi_f32(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

__device__ inline float block_sum(float v, float *scratch) {
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  float total = 0.0f;
  for (uint32_t w = 0; w < blockDim.x / 64; ++w) total += scratch[w];
  __syncthreads();
  return total;
}

// Eight consecutive elements of bf16 (kWide false) or f32 rows.
template <bool kWide>
__device__ inline void load8(const void *base, uint64_t element, float (&v)[8]) {
  if constexpr (kWide) {
    const float4 a = *(const float4 *)((const float *)base + element);
    const float4 b = *(const float4 *)((const float *)base + element + 4);
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
  } else {
    const uint4 w = *(const uint4 *)((const uint16_t *)base + element);
    v[0] = lo_f32(w.x), v[1] = hi_f32(w.x), v[2] = lo_f32(w.y), v[3] = hi_f32(w.y);
    v[4] = lo_f32(w.z), v[5] = hi_f32(w.z), v[6] = lo_f32(w.w), v[7] = hi_f32(w.w);
  }
}

template <bool kWide>
__device__ inline void store8(void *base, uint64_t element, const float (&v)[8]) {
  if constexpr (kWide) {
    *(float4 *)((float *)base + element) = make_float4(v[0], v[1], v[2], v[3]);
    *(float4 *)((float *)base + element + 4) = make_float4(v[4], v[5], v[6], v[7]);
  } else {
    *(uint4 *)((uint16_t *)base + element) =
        make_uint4(pack2(v[0], v[1]), pack2(v[2], v[3]), pack2(v[4], v[5]), pack2(v[6], v[7]));
  }
}

struct RowArgs {
  const void *x, *update, *weight;   // bf16 or f32 rows, strides in elements
  void *out0, *out1;
  uint64_t x_stride, update_stride, weight_stride, out0_stride, out1_stride;
  uint32_t width;
  float eps;
};

// out = x * rsqrt(mean(x^2) + eps) * w            (kResidual = false)
// value = x + update; out0 = value; out1 = value * rsqrt(mean(value^2) + eps) * w
template <bool kResidual, bool kWide>
__global__ __launch_bounds__(256) void norm_rows_kernel(RowArgs a) {
  __shared__ float scratch[4];
  const uint64_t row = blockIdx.x;
  const uint64_t x_at = row * a.x_stride, u_at = row * a.update_stride, w_at = row * a.weight_stride;
  float acc = 0.0f;
  for (uint32_t c = threadIdx.x * 8; c < a.width; c += 256 * 8) {
    float v[8], u[8];
    load8<kWide>(a.x, x_at + c, v);
    if (kResidual) load8<kWide>(a.update, u_at + c, u);
    for (int i = 0; i < 8; ++i) {
      const float value = kResidual ? v[i] + u[i] : v[i];
      acc += value * value;
    }
  }
  const float total = block_sum(acc, scratch);
  const float inverse = 1.0f / sqrtf(total / (float)a.width + a.eps);
  for (uint32_t c = threadIdx.x * 8; c < a.width; c += 256 * 8) {
    float v[8], u[8], w[8], normed[8];
    load8<kWide>(a.x, x_at + c, v);
    load8<kWide>(a.weight, w_at + c, w);
    if (kResidual) load8<kWide>(a.update, u_at + c, u);
    for (int i = 0; i < 8; ++i) {
      if (kResidual) v[i] += u[i];
      normed[i] = v[i] * inverse * w[i];
    }
    if (kResidual) {
      store8<kWide>(a.out0, row * a.out0_stride + c, v);
      store8<kWide>(a.out1, row * a.out1_stride + c, normed);
    } else {
      store8<kWide>(a.out0, row * a.out0_stride + c, normed);
    }
  }
}

// The weighted sum of a row's routed partial rows (+ residual), as combine_routes_rows_kernel
// forms it, and the RMS normalisation of the stored (bf16) result, as norm_rows_kernel forms it:
// thread t owns columns 8t .. 8t+7 in both, so the sums and the reduction add in the same order.
template <bool kWide>
__global__ __launch_bounds__(256) void combine_routes_norm_kernel(
    const float *partial, View indices, View weights, const void *residual,
    uint64_t residual_row_stride, void *out, uint64_t out_row_stride, uint32_t routes,
    uint32_t columns, uint32_t experts, NormTail tail) {
  __shared__ float scratch[4];
  const uint32_t row = blockIdx.x, column = 8 * threadIdx.x;
  const bool live = column < columns;
  float value[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (live) {
    float weight[8];
    float4 part[8][2];
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {
      weight[slot] = 0.0f;
      part[slot][0] = part[slot][1] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if ((uint32_t)slot < routes) {
        const uint32_t expert = load_u32_at(indices, indices.offset + row * indices.stride[0] +
                                                         slot * indices.stride[1]);
        if (expert < experts) {
          weight[slot] = load_float_at(weights, weights.offset + row * weights.stride[0] +
                                                    slot * weights.stride[1]);
          const float4 *from = (const float4 *)(partial + ((uint64_t)row * routes + slot) * columns + column);
          part[slot][0] = from[0];
          part[slot][1] = from[1];
        }
      }
    }
#pragma unroll
    for (int slot = 0; slot < 8; ++slot) {   // a skipped route adds +0 * 0: no effect
      value[0] += weight[slot] * part[slot][0].x;
      value[1] += weight[slot] * part[slot][0].y;
      value[2] += weight[slot] * part[slot][0].z;
      value[3] += weight[slot] * part[slot][0].w;
      value[4] += weight[slot] * part[slot][1].x;
      value[5] += weight[slot] * part[slot][1].y;
      value[6] += weight[slot] * part[slot][1].z;
      value[7] += weight[slot] * part[slot][1].w;
    }
    if (residual) {
      float r[8];
      load8<kWide>(residual, (uint64_t)row * residual_row_stride + column, r);
      for (int i = 0; i < 8; ++i) value[i] += r[i];
    }
    store8<kWide>(out, (uint64_t)row * out_row_stride + column, value);
    // the normalisation reads what was stored
    if (!kWide)
      for (int i = 0; i < 8; ++i) value[i] = lo_f32(pack2(value[i], 0.0f));
  }
  float acc = 0.0f;
  for (int i = 0; i < 8; ++i) acc += value[i] * value[i];
  const float total = block_sum(acc, scratch);
  const float inverse = 1.0f / sqrtf(total / (float)columns + tail.eps);
  if (live) {
    float w[8], normed[8];
    load8<kWide>(tail.weight, (uint64_t)row * tail.weight_stride + column, w);
    for (int i = 0; i < 8; ++i) normed[i] = value[i] * inverse * w[i];
    store8<kWide>(tail.out, (uint64_t)row * tail.out_stride + column, normed);
  }
}

struct QkArgs {
  const void *lo, *hi, *w_lo, *w_hi;   // bf16 or f32, strides in elements
  const float *positions;
  void *out_lo, *out_hi;
  uint64_t lo_s[2], hi_s[2], wlo_s[2], whi_s[2], pos_s[3], olo_s[2], ohi_s[2];
  uint32_t rows, heads, width;
  float head_dim, eps, theta, exponent_scale;
};

// blockIdx.x is the row; the waves of its gridDim.y workgroups take the heads in turn (one head per
// wave for small batches, many for long ones): RMS-normalise the head over both halves, scale,
// rotate the (lo, hi) pair by angle = position * theta^(i * exponent_scale).  The rotation is the
// same for every head of a row when the positions do not vary along the head axis (the usual
// broadcast view), and is then computed once per wave.
template <bool kWide>
__device__ inline float load1(const void *base, uint64_t element) {
  if constexpr (kWide) return ((const float *)base)[element];
  return __uint_as_float((uint32_t)((const uint16_t *)base)[element] << 16);
}

template <bool kWide>
__device__ inline void store1(void *base, uint64_t element, float value) {
  if constexpr (kWide)
    ((float *)base)[element] = value;
  else
    ((uint16_t *)base)[element] = (uint16_t)(pack2(value, 0.0f) & 0xffffu);
}

template <bool kWide>
__global__ __launch_bounds__(256) void qk_norm_rope_kernel(QkArgs a) {
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t row = blockIdx.x;
  const bool live = lane < a.width;
  const bool shared_angle = a.pos_s[1] == 0;
  float c = 1.0f, s = 0.0f;
  const float frequency = powf(a.theta, (float)lane * a.exponent_scale);
  if (shared_angle && live) {
    const float angle = a.positions[row * a.pos_s[0] + lane * a.pos_s[2]] * frequency;
    c = cosf(angle);
    s = sinf(angle);
  }
  for (uint32_t head = blockIdx.y * 4 + wave; head < a.heads; head += 4 * gridDim.y) {
    float lo = 0.0f, hi = 0.0f;
    if (live) {
      lo = load1<kWide>(a.lo, row * a.lo_s[0] + head * a.lo_s[1] + lane);
      hi = load1<kWide>(a.hi, row * a.hi_s[0] + head * a.hi_s[1] + lane);
    }
    float square_sum = lo * lo + hi * hi;
    for (int offset = 32; offset > 0; offset >>= 1) square_sum += __shfl_xor(square_sum, offset, 64);
    if (!live) continue;
    const float inverse = 1.0f / sqrtf(square_sum / a.head_dim + a.eps);
    const float w_lo = load1<kWide>(a.w_lo, row * a.wlo_s[0] + head * a.wlo_s[1] + lane);
    const float w_hi = load1<kWide>(a.w_hi, row * a.whi_s[0] + head * a.whi_s[1] + lane);
    const float n_lo = lo * inverse * w_lo, n_hi = hi * inverse * w_hi;
    if (!shared_angle) {
      const float angle = a.positions[row * a.pos_s[0] + head * a.pos_s[1] + lane * a.pos_s[2]] * frequency;
      c = cosf(angle);
      s = sinf(angle);
    }
    const float r_lo = n_lo * c - n_hi * s, r_hi = n_hi * c + n_lo * s;
    store1<kWide>(a.out_lo, row * a.olo_s[0] + head * a.olo_s[1] + lane, r_lo);
    store1<kWide>(a.out_hi, row * a.ohi_s[0] + head * a.ohi_s[1] + lane, r_hi);
  }
}

struct PairArgs {
  const uint16_t *a, *b;
  uint16_t *out;
  uint64_t a_stride, b_stride, out_stride;   // elements between rows
  uint32_t rows, pieces_per_row;             // 8-element pieces
};

// out = a * sigmoid(a) * b (kSilu) or a + b, eight bf16 values per thread and trip; the
// arithmetic is the interpreter's: f32 throughout, sigmoid(x) = 1 / (1 + exp(-x)), one rounding.
template <bool kSilu>
__global__ __launch_bounds__(256) void map_pair_kernel(PairArgs p) {
  const uint64_t pieces = (uint64_t)p.rows * p.pieces_per_row;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t piece = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; piece < pieces;
       piece += stride) {
    const uint64_t row = piece / p.pieces_per_row, at = 8 * (piece % p.pieces_per_row);
    const uint4 av = *(const uint4 *)(p.a + row * p.a_stride + at);
    const uint4 bv = *(const uint4 *)(p.b + row * p.b_stride + at);
    const uint32_t aw[4] = {av.x, av.y, av.z, av.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
    uint32_t ow[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a_lo = lo_f32(aw[i]), a_hi = hi_f32(aw[i]);
      const float b_lo = lo_f32(bw[i]), b_hi = hi_f32(bw[i]);
      if (kSilu)
        ow[i] = pack2(a_lo * (1.0f / (1.0f + expf(-a_lo))) * b_lo,
                      a_hi * (1.0f / (1.0f + expf(-a_hi))) * b_hi);
      else
        ow[i] = pack2(a_lo + b_lo, a_hi + b_hi);
    }
    *(uint4 *)(p.out + row * p.out_stride + at) = make_uint4(ow[0], ow[1], ow[2], ow[3]);
  }
}

// Canonical expression of value v: commutative operands sorted; constants carry their bits.
std::string canonical(const fh_inst *insts, uint32_t count, uint32_t v, int depth = 0) {
  if (v >= count || depth > 24) return "?";
  const fh_inst &inst = insts[v];
  char buffer[32];
  switch (inst.kind) {
  case 0: return "in" + std::to_string(inst.a);
  case 1: snprintf(buffer, sizeof(buffer), "c%08x", inst.a); return buffer;
  case 2: return "i" + std::to_string(inst.op);
  case 3: return "e" + std::to_string(inst.op);
  case 4: return "u" + std::to_string(inst.op) + "(" + canonical(insts, count, inst.a, depth + 1) + ")";
  case 5: {
    std::string l = canonical(insts, count, inst.a, depth + 1),
                r = canonical(insts, count, inst.b, depth + 1);
    if ((inst.op == 0 || inst.op == 2) && r < l) std::swap(l, r);
    return "b" + std::to_string(inst.op) + "(" + l + "," + r + ")";
  }
  case 7: return "k" + std::to_string(inst.op) + "(" + canonical(insts, count, inst.a, depth + 1) + ")";
  case 8: return "r" + std::to_string(inst.op) + "(" + canonical(insts, count, inst.a, depth + 1) + ")";
  default: return "?";
  }
}

float const_of(const std::string &hex) {
  uint32_t bits = (uint32_t)strtoul(hex.c_str(), nullptr, 16);
  float value;
  memcpy(&value, &bits, 4);
  return value;
}

std::string escape(const std::string &s) {
  std::string out;
  for (char ch : s) {
    if (ch == '(' || ch == ')') out += '\\';
    out += ch;
  }
  return out;
}

const std::string kConst = "c([0-9a-f]{8})";

bool bf16_rows(const View &v, uint32_t rank) {
  return v.dtype == FH_BF16 && v.rank == rank && v.stride[rank - 1] == 1;
}

// Rows of `dtype` (bf16 or f32) with a contiguous innermost axis.
bool typed_rows(const View &v, uint32_t rank, uint32_t dtype) {
  return v.dtype == dtype && v.rank == rank && v.stride[rank - 1] == 1;
}

}  // namespace

ProgramClass classify_program(uint32_t kind, const fh_inst *insts, uint32_t n_insts,
                              const uint32_t *pairs, uint32_t n_pairs) {
  ProgramClass result{};
  result.kind = kProgramGeneric;
  if (kind == 0) {   // element-wise programs with one output
    if (n_pairs != 1 || pairs[0] != 0) return result;
    const std::string e = canonical(insts, n_insts, pairs[1]);
    if (e == "b2(b2(in0,u9(in0)),in1)") result.kind = kProgramSiluMul;
    if (e == "b0(in0,in1)") result.kind = kProgramAdd;
    return result;
  }
  if (kind != 1) return result;
  std::smatch m;
  auto value_of = [&](uint32_t slot) -> std::string {
    for (uint32_t p = 0; p < n_pairs; ++p)
      if (pairs[2 * p] == slot) return canonical(insts, n_insts, pairs[2 * p + 1]);
    return "";
  };
  // x * rsqrt(sum(x*x) / f32(extent) + eps) * w
  auto norm_of = [&](const std::string &x, const std::string &w) {
    std::string xe = escape(x);
    return "b2\\(b2\\(" + xe + ",u5\\(b0\\(b3\\(r0\\(b2\\(" + xe + "," + xe + "\\)\\),k0\\(e(\\d)\\)\\)," +
           kConst + "\\)\\)\\)," + w + "\\)";
  };
  if (n_pairs == 1) {
    std::string e = value_of(0);
    if (std::regex_match(e, m, std::regex("^" + norm_of("in0", "in1") + "$"))) {
      result.kind = kProgramRmsNorm;
      result.axis = (uint32_t)atoi(m[1].str().c_str());
      result.c[0] = const_of(m[2].str());
    }
    return result;
  }
  if (n_pairs != 2) return result;
  std::string first = value_of(0), second = value_of(1);
  if (first == "b0(in0,in1)" &&
      std::regex_match(second, m, std::regex("^" + norm_of("b0(in0,in1)", "in2") + "$"))) {
    result.kind = kProgramResidualNorm;
    result.axis = (uint32_t)atoi(m[1].str().c_str());
    result.c[0] = const_of(m[2].str());
    return result;
  }
  // qk_norm_rope_rows(lo, hi, w_lo, w_hi, positions)
  const std::string ss = "r0\\(b0\\(b2\\(in0,in0\\),b2\\(in1,in1\\)\\)\\)";
  const std::string inv = "u5\\(b0\\(b3\\(" + ss + "," + kConst + "\\)," + kConst + "\\)\\)";
  // later occurrences of the same sub-expression must repeat the captured constants
  const std::string inv_again = "u5\\(b0\\(b3\\(" + ss + ",c\\1\\),c\\2\\)\\)";
  const std::string angle = "b2\\(b6\\(" + kConst + ",b2\\(" + kConst + ",k0\\(i(\\d)\\)\\)\\),in4\\)";
  const std::string angle_again = "b2\\(b6\\(c\\3,b2\\(c\\4,k0\\(i\\5\\)\\)\\),in4\\)";
  const std::string n_lo = "b2\\(b2\\(in0," + inv + "\\),in2\\)";
  const std::string n_lo_again = "b2\\(b2\\(in0," + inv_again + "\\),in2\\)";
  const std::string n_hi_again = "b2\\(b2\\(in1," + inv_again + "\\),in3\\)";
  const std::string out0 = "^b1\\(b2\\(" + n_lo + ",u7\\(" + angle + "\\)\\),b2\\(" + n_hi_again +
                           ",u6\\(" + angle_again + "\\)\\)\\)$";
  if (std::regex_match(first, m, std::regex(out0))) {
    float head_dim = const_of(m[1].str()), eps = const_of(m[2].str()), theta = const_of(m[3].str()),
          exponent_scale = const_of(m[4].str());
    uint32_t axis = (uint32_t)atoi(m[5].str().c_str());
    // second output: n_hi*cos + n_lo*sin with the same constants (sorted: the n_lo product first)
    auto hex = [](float f) {
      uint32_t bits;
      memcpy(&bits, &f, 4);
      char b[16];
      snprintf(b, sizeof(b), "c%08x", bits);
      return std::string(b);
    };
    std::string inv_s = "u5(b0(b3(r0(b0(b2(in0,in0),b2(in1,in1)))," + hex(head_dim) + ")," + hex(eps) + "))";
    std::string angle_s = "b2(b6(" + hex(theta) + ",b2(" + hex(exponent_scale) + ",k0(i" +
                          std::to_string(axis) + "))),in4)";
    std::string nlo_s = "b2(b2(in0," + inv_s + "),in2)", nhi_s = "b2(b2(in1," + inv_s + "),in3)";
    std::string expect = "b0(b2(" + nlo_s + ",u6(" + angle_s + ")),b2(" + nhi_s + ",u7(" + angle_s + ")))";
    if (second == expect) {
      result.kind = kProgramQkNormRope;
      result.axis = axis;
      result.c[0] = head_dim;
      result.c[1] = eps;
      result.c[2] = theta;
      result.c[3] = exponent_scale;
    }
  }
  return result;
}

bool try_fast_program(hipStream_t stream, const ProgramClass &cls, const ProgramArgs &p,
                      uint64_t elements) {
  if (cls.kind == kProgramGeneric || elements == 0) return false;
  const uint32_t rank = p.rank;
  auto ptr = [](const View &v) { return (uint16_t *)v.base + v.offset; };
  auto aligned = [&](const View &v) {
    if (v.offset % 8) return false;
    for (uint32_t axis = 0; axis + 1 < rank; ++axis)
      if (v.stride[axis] % 8) return false;
    return true;
  };
  if (cls.kind == kProgramSiluMul || cls.kind == kProgramAdd) {
    if (rank != 2 || p.n_inputs != 2 || p.shape[1] % 8 != 0) return false;
    for (const View *v : {&p.inputs[0], &p.inputs[1], &p.outputs[0]})
      if (!bf16_rows(*v, 2) || !aligned(*v)) return false;
    PairArgs a{ptr(p.inputs[0]), ptr(p.inputs[1]), ptr(p.outputs[0]), p.inputs[0].stride[0],
               p.inputs[1].stride[0], p.outputs[0].stride[0], p.shape[0], p.shape[1] / 8};
    const uint64_t pieces = (uint64_t)a.rows * a.pieces_per_row;
    const uint32_t blocks = (uint32_t)std::min<uint64_t>((pieces + 255) / 256, 256 * 16);
    if (cls.kind == kProgramSiluMul)
      map_pair_kernel<true><<<blocks, 256, 0, stream>>>(a);
    else
      map_pair_kernel<false><<<blocks, 256, 0, stream>>>(a);
    return true;
  }
  if (cls.axis != rank - 1) return false;
  if (cls.kind == kProgramRmsNorm || cls.kind == kProgramResidualNorm) {
    const bool residual = cls.kind == kProgramResidualNorm;
    if (rank != 2 || p.n_inputs != (residual ? 3u : 2u)) return false;
    const uint32_t n_out = residual ? 2 : 1;
    const uint32_t dtype = p.inputs[0].dtype;
    if (dtype != FH_BF16 && dtype != FH_F32) return false;
    const bool wide = dtype == FH_F32;
    auto ptr = [](const View &v) { return (void *)(v.base + v.offset * dtype_size(v.dtype)); };
    for (uint32_t i = 0; i < p.n_inputs; ++i)
      if (!typed_rows(p.inputs[i], 2, dtype) || !aligned(p.inputs[i])) return false;
    for (uint32_t i = 0; i < n_out; ++i)
      if (!typed_rows(p.outputs[i], 2, dtype) || !aligned(p.outputs[i])) return false;
    const uint32_t width = p.shape[1];
    if (width % 8 != 0) return false;
    RowArgs a{};
    a.x = ptr(p.inputs[0]);
    a.x_stride = p.inputs[0].stride[0];
    const View &w = p.inputs[residual ? 2 : 1];
    a.weight = ptr(w);
    a.weight_stride = w.stride[0];
    if (residual) {
      a.update = ptr(p.inputs[1]);
      a.update_stride = p.inputs[1].stride[0];
    }
    // out_slot maps pairs to output tensors; pairs are (slot, value) with slot = output index
    a.out0 = ptr(p.outputs[0]);
    a.out0_stride = p.outputs[0].stride[0];
    if (residual) {
      a.out1 = ptr(p.outputs[1]);
      a.out1_stride = p.outputs[1].stride[0];
    }
    a.width = width;
    a.eps = cls.c[0];
    auto *kernel = residual ? (wide ? norm_rows_kernel<true, true> : norm_rows_kernel<true, false>)
                            : (wide ? norm_rows_kernel<false, true> : norm_rows_kernel<false, false>);
    kernel<<<dim3(p.shape[0]), 256, 0, stream>>>(a);
    return true;
  }
  if (cls.kind == kProgramQkNormRope) {
    if (rank != 3 || p.n_inputs != 5 || p.shape[2] > 64) return false;
    const uint32_t dtype = p.inputs[0].dtype;
    if (dtype != FH_BF16 && dtype != FH_F32) return false;
    auto ptr = [](const View &v) { return (void *)(v.base + v.offset * dtype_size(v.dtype)); };
    for (uint32_t i = 0; i < 4; ++i)
      if (!typed_rows(p.inputs[i], 3, dtype)) return false;
    if (p.inputs[4].dtype != FH_F32 || p.inputs[4].rank != 3) return false;
    for (uint32_t i = 0; i < 2; ++i)
      if (!typed_rows(p.outputs[i], 3, dtype)) return false;
    QkArgs a{};
    auto set = [](uint64_t (&dst)[2], const View &v) {
      dst[0] = v.stride[0];
      dst[1] = v.stride[1];
    };
    a.lo = ptr(p.inputs[0]);
    a.hi = ptr(p.inputs[1]);
    a.w_lo = ptr(p.inputs[2]);
    a.w_hi = ptr(p.inputs[3]);
    a.positions = (const float *)p.inputs[4].base + p.inputs[4].offset;
    a.out_lo = ptr(p.outputs[0]);
    a.out_hi = ptr(p.outputs[1]);
    set(a.lo_s, p.inputs[0]);
    set(a.hi_s, p.inputs[1]);
    set(a.wlo_s, p.inputs[2]);
    set(a.whi_s, p.inputs[3]);
    for (int axis = 0; axis < 3; ++axis) a.pos_s[axis] = p.inputs[4].stride[axis];
    set(a.olo_s, p.outputs[0]);
    set(a.ohi_s, p.outputs[1]);
    a.rows = p.shape[0];
    a.heads = p.shape[1];
    a.width = p.shape[2];
    a.head_dim = cls.c[0];
    a.eps = cls.c[1];
    a.theta = cls.c[2];
    a.exponent_scale = cls.c[3];
    // enough workgroups to fill the device for small batches, one per row for long ones
    const uint32_t head_blocks = (a.heads + 3) / 4;
    uint32_t per_row = 4096 / a.rows;
    per_row = per_row < 1 ? 1 : (per_row > head_blocks ? head_blocks : per_row);
    if (dtype == FH_F32)
      qk_norm_rope_kernel<true><<<dim3(a.rows, per_row), 256, 0, stream>>>(a);
    else
      qk_norm_rope_kernel<false><<<dim3(a.rows, per_row), 256, 0, stream>>>(a);
    return true;
  }
  return false;
}

bool norm_tail_of(const ProgramClass &cls, const ProgramArgs &p, const View &produced, NormTail *tail) {
  if (cls.kind != kProgramRmsNorm || p.rank != 2 || cls.axis != 1 || p.n_inputs != 2) return false;
  const View &x = p.inputs[0], &w = p.inputs[1], &out = p.outputs[0];
  if (p.shape[1] % 8 != 0 || p.shape[1] > 2048 || p.shape[0] == 0) return false;
  const uint32_t dtype = x.dtype;
  if (dtype != FH_BF16 && dtype != FH_F32) return false;
  for (const View *v : {&x, &w, &out}) {
    if (!typed_rows(*v, 2, dtype) || v->offset % 8 || v->stride[0] % 8) return false;
  }
  // the rows it reads are the rows just produced, element for element
  if (x.base != produced.base || x.offset != produced.offset || produced.dtype != dtype ||
      produced.rank != 2 || produced.shape[0] != p.shape[0] || produced.shape[1] != p.shape[1] ||
      x.stride[0] != produced.stride[0] || x.stride[1] != produced.stride[1])
    return false;
  const uint64_t size = dtype_size(dtype);
  tail->weight = w.base + w.offset * size;
  tail->weight_stride = w.stride[0];
  tail->out = out.base + out.offset * size;
  tail->out_stride = out.stride[0];
  tail->eps = cls.c[0];
  tail->wide = dtype == FH_F32;
  return true;
}

void launch_combine_routes_norm(hipStream_t stream, const float *partial, const View &indices,
                                const View &weights, const void *residual,
                                uint64_t residual_row_stride, void *out, uint64_t out_row_stride,
                                uint32_t rows, uint32_t routes, uint32_t columns, uint32_t experts,
                                const NormTail &tail) {
  auto *kernel = tail.wide ? combine_routes_norm_kernel<true> : combine_routes_norm_kernel<false>;
  kernel<<<dim3(rows), 256, 0, stream>>>(partial, indices, weights, residual, residual_row_stride, out,
                                         out_row_stride, routes, columns, experts, tail);
}

}  // namespace fh
