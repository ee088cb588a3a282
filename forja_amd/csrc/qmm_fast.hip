// MLX-4bit affine group-quantised matmul on the gfx950 matrix cores, dense and routed (MoE).
//
// y[m,n] = sum_k x[m,k] * (scale[n,k/64] * q[n,k] + bias[n,k/64])      (affine_quant_dot,
// crates/forja-cpu/src/lib.rs:1277-1310), q = nibble k%8 of word k/8, low nibble first.
//
// The work is HBM-bound on the packed weights, so the kernel is built around reading each weight
// byte once, with 16-byte loads, and spending as few vector instructions per nibble as possible:
//   * a nibble becomes the bf16 value 16+q with two integer ops for two nibbles
//     ((w >> s) & 0x00780078 | 0x41804180: q lands in mantissa bits 3..6 of exponent 2^4); the
//     pairs come out in the order (0,4)(1,5)(2,6)(3,7), and the activation tile is staged in LDS
//     with the same permutation inside every 8 elements;
//   * v_mfma_f32_32x32x16_bf16 contracts one 64-element quantisation group in four steps (each
//     lane holds the four packed words = 32 values of "its" half of the group for one output
//     column), giving part[m,n] = sum x * (16+q) exactly in f32;
//   * the affine parameters are applied once per group: acc += scale*part + (bias-16*scale)*xsum,
//     with xsum[m,group] = sum of the group's activations computed while staging.
// The dequantised weight is never rounded to bf16, so results track the f32 reference closely.
// Activations: bf16; 32 rows per MFMA tile (padded); a workgroup is 4 waves x 32 columns.
#include "fast_kernels.hpp"

#include <algorithm>
#include <string>

namespace fh {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kWaves = 4;           // waves per workgroup
constexpr int kColsPerWave = 32;
constexpr int kGroup = 64;          // quantisation group handled by this path
constexpr uint32_t kNoBlock = 0xffffffffu;

enum Epilogue { kStore = 0, kSwiglu = 1 };

struct QmmArgs {
  const uint16_t *x;        // bf16 activations, innermost axis contiguous
  uint64_t x_row_stride;    // elements between input rows
  const uint32_t *packed[2];
  const uint16_t *scales[2], *biases[2];
  uint64_t expert_words;    // u32 words per expert matrix (N*K/8); 0 for dense
  uint64_t expert_groups;   // scale entries per expert matrix (N*K/64)
  void *out;                // bf16 or f32
  uint64_t out_row_stride;  // elements
  uint32_t out_f32;
  uint32_t rows, inner, columns;
  // routed form
  const uint32_t *sorted_routes, *blocks, *n_blocks;
  uint32_t route_div;       // input row = route / route_div
  // dense form only
  const uint32_t *run_if_set;   // when not null: do nothing unless this device word is non-zero
  const uint16_t *residual;     // optional bf16 rows added to the result before it is rounded
  uint64_t residual_row_stride;
  // routed whole-K tile kernel: K is split inside the workgroup when tiles x column blocks is at
  // most this (0: never)
  uint32_t split_below;
};

__device__ inline uint32_t pack2(float lo, float hi) {
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ inline float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// (x & mask) | magic in one instruction.  The compiler splits the expression in two when both
// constants are literals (a VOP3 instruction reads one scalar operand at most); with the mask in a
// scalar register and the other constant in a vector register it is a single v_and_or_b32.
__device__ inline uint32_t and_or(uint32_t x, uint32_t mask, uint32_t magic) {
  return (x & mask) | magic;
}

// Eight nibbles of `w` as bf16 (16+q), in slot order (0,4)(1,5)(2,6)(3,7): two instructions per
// pair of nibbles.
__device__ inline bf16x8 unpack_word(uint32_t w) {
  uint32_t mask = 0x00780078u, magic = 0x41804180u;
  asm("" : "+s"(mask), "+v"(magic));   // no instruction: keeps the two constants in registers
  uint4 r;
  r.x = and_or(w << 3, mask, magic);
  r.y = and_or(w >> 1, mask, magic);
  r.z = and_or(w >> 5, mask, magic);
  r.w = and_or(w >> 9, mask, magic);
  return __builtin_bit_cast(bf16x8, r);
}

// MT = 32-row tiles per workgroup, KC = activation columns staged per pass.  The four waves of a
// workgroup share the staged activations and own 32 output columns each.
template <int MT, bool kPair, bool kRouted>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void qmm_mfma_kernel(QmmArgs a) {
  if (!kRouted && a.run_if_set && a.run_if_set[0] == 0) return;
  constexpr int NW = kWaves;
  constexpr int kThreads = 64 * NW;
  constexpr int KC = 512 / MT;  // 33 KB of LDS either way: two workgroups per CU overlap staging
  constexpr int kRows = 32 * MT;
  constexpr int kPitch = 2 * KC + 16;  // bytes; +16 spreads consecutive rows over the banks
  __shared__ __attribute__((aligned(16))) unsigned char xs[kRows * kPitch];
  __shared__ __attribute__((aligned(16))) float xsum[(KC / kGroup) * kRows];
  __shared__ uint32_t row_ids[kRows];

  const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const uint32_t nl = lane & 31, h = lane >> 5;
  const uint32_t column = (blockIdx.x * NW + wave) * kColsPerWave + nl;
  const uint32_t column_c = min(column, a.columns - 1);  // clamped for loads

  uint32_t expert = 0, count = 0, first = 0;
  if (kRouted) {
    if (blockIdx.y >= a.n_blocks[0]) return;
    expert = a.blocks[3 * blockIdx.y];
    if (expert == kNoBlock) return;
    first = a.blocks[3 * blockIdx.y + 1];
    count = a.blocks[3 * blockIdx.y + 2];
    for (uint32_t r = tid; r < kRows; r += kThreads)
      row_ids[r] = r < count ? a.sorted_routes[first + r] : 0;
  } else {
    first = blockIdx.y * kRows;
    count = min((uint32_t)kRows, a.rows - first);
  }
  const uint32_t words_per_row = a.inner / 8, groups_per_row = a.inner / kGroup;
  const uint32_t *w_row[2];
  const uint16_t *s_row[2], *b_row[2];
  for (int pj = 0; pj < (kPair ? 2 : 1); ++pj) {
    w_row[pj] = a.packed[pj] + expert * a.expert_words + (uint64_t)column_c * words_per_row + 4 * h;
    s_row[pj] = a.scales[pj] + expert * a.expert_groups + (uint64_t)column_c * groups_per_row;
    b_row[pj] = a.biases[pj] + expert * a.expert_groups + (uint64_t)column_c * groups_per_row;
  }

  constexpr int kP = kPair ? 2 : 1;
  constexpr int kPieces = kRows * KC / 8 / kThreads;  // 16-byte activation pieces per thread per pass
  constexpr int kGroupsPerPass = KC / kGroup;
  f32x16 acc[kP][MT];
  for (int pj = 0; pj < kP; ++pj)
    for (int mt = 0; mt < MT; ++mt)
      for (int j = 0; j < 16; ++j) acc[pj][mt][j] = 0.0f;

  // Two independent software pipelines hide memory latency:
  //  * weights: a ring of two quads of groups.  A quad is four consecutive groups = one whole
  //    128-byte line of every weight row, requested with four back-to-back loads so that the
  //    line is fetched from L2 exactly once whatever the L1 does; a slot is reloaded two quads
  //    ahead as soon as it has been consumed - the weight stream does not care about staging
  //    passes;
  //  * activations: the next pass's pieces are fetched into registers while the current pass is
  //    consumed from LDS.
  const uint32_t total_quads = a.inner / (4 * kGroup);
  uint4 wq[kP][2][4];
  uint2 scale_q[kP][2], bias_q[kP][2];   // four bf16 each
  auto load_quad = [&](int slot, uint32_t quad) {
    const uint32_t qd = min(quad, total_quads - 1);  // unconditional: the tail reloads the last quad
    for (int pj = 0; pj < kP; ++pj) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        wq[pj][slot][i] = *(const uint4 *)(w_row[pj] + (uint64_t)(4 * qd + i) * 8);
      scale_q[pj][slot] = *(const uint2 *)(s_row[pj] + 4 * qd);
      bias_q[pj][slot] = *(const uint2 *)(b_row[pj] + 4 * qd);
    }
  };
  uint4 x_regs[kPieces];
  auto fetch_pass = [&](uint32_t kc0) {
    const uint32_t kc = min((uint32_t)KC, a.inner - kc0);
    const uint32_t pieces_per_row = kc / 8;
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const uint32_t piece = tid + i * kThreads;
      const uint32_t row = piece / pieces_per_row, pc = piece % pieces_per_row;
      x_regs[i] = make_uint4(0, 0, 0, 0);
      if (row < count) {  // rows beyond kRows only arise in a short last pass and are >= count
        const uint64_t in_row = kRouted ? row_ids[row] / a.route_div : first + row;
        x_regs[i] = *(const uint4 *)(a.x + in_row * a.x_row_stride + kc0 + 8 * pc);
      }
    }
  };
  // Pass switch: publish the fetched activations (permuted inside each 8, plus per-group sums),
  // then start fetching the pass after.
  auto pass_switch = [&](uint32_t pass) {
    const uint32_t kc0 = pass * KC;
    const uint32_t kc = min((uint32_t)KC, a.inner - kc0);
    const uint32_t pieces_per_row = kc / 8;
    __syncthreads();  // the previous pass is consumed
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const uint32_t piece = tid + i * kThreads;
      const uint32_t row = piece / pieces_per_row, pc = piece % pieces_per_row;
      const uint4 v = x_regs[i];
      float sum = bf16_bits_to_f32(v.x & 0xffffu) + bf16_bits_to_f32(v.x >> 16) +
                  bf16_bits_to_f32(v.y & 0xffffu) + bf16_bits_to_f32(v.y >> 16) +
                  bf16_bits_to_f32(v.z & 0xffffu) + bf16_bits_to_f32(v.z >> 16) +
                  bf16_bits_to_f32(v.w & 0xffffu) + bf16_bits_to_f32(v.w >> 16);
      // eight consecutive pieces (= lanes) make one quantisation group
      sum += __shfl_xor(sum, 1, 64);
      sum += __shfl_xor(sum, 2, 64);
      sum += __shfl_xor(sum, 4, 64);
      if (row < (uint32_t)kRows) {
        uint4 permuted;
        permuted.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (x0, x4)
        permuted.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (x1, x5)
        permuted.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (x2, x6)
        permuted.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (x3, x7)
        *(uint4 *)(xs + row * kPitch + pc * 16) = permuted;
        if ((pc & 7) == 0) xsum[(pc >> 3) * kRows + row] = sum;
      }
    }
    __syncthreads();
    if (kc0 + KC < a.inner) fetch_pass(kc0 + KC);
  };
  // Two consecutive quantisation groups (members i0, i0+1 of ring slot `slot`; `group` is the
  // first one's number): four MFMA steps per group and row tile on independent accumulation
  // chains, the scales applied per group, and the bias term
  // sum_g (bias_g - 16 scale_g) * xsum_g[row] as one f32 MFMA over the two groups (lane half h
  // supplies group + h of both operands).
  auto consume_pair = [&](int slot, int i0, uint32_t group) {
    const uint32_t gi = group % kGroupsPerPass;  // index of the first group inside the staged pass
    f32x16 part[2][kP][MT];
#pragma unroll
    for (int q = 0; q < 2; ++q)
      for (int pj = 0; pj < kP; ++pj)
        for (int mt = 0; mt < MT; ++mt)
          for (int j = 0; j < 16; ++j) part[q][pj][mt][j] = 0.0f;
#pragma unroll
    for (int step = 0; step < 4; ++step) {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        bf16x8 b_op[kP];
        for (int pj = 0; pj < kP; ++pj) {
          const uint4 w = wq[pj][slot][i0 + q];
          b_op[pj] = unpack_word(step == 0 ? w.x : (step == 1 ? w.y : (step == 2 ? w.z : w.w)));
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const uint4 a_raw = *(const uint4 *)(xs + (mt * 32 + nl) * kPitch +
                                               ((gi + q) * kGroup + 32 * h + 8 * step) * 2);
          const bf16x8 a_op = __builtin_bit_cast(bf16x8, a_raw);
          for (int pj = 0; pj < kP; ++pj)
            part[q][pj][mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_op, b_op[pj],
                                                                      part[q][pj][mt], 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int pj = 0; pj < kP; ++pj) {
      const uint32_t scale_bits = i0 == 0 ? scale_q[pj][slot].x : scale_q[pj][slot].y;
      const uint32_t bias_bits = i0 == 0 ? bias_q[pj][slot].x : bias_q[pj][slot].y;
      const float scale0 = bf16_bits_to_f32(scale_bits & 0xffffu);
      const float scale1 = bf16_bits_to_f32(scale_bits >> 16);
      const float shift0 = bf16_bits_to_f32(bias_bits & 0xffffu) - 16.0f * scale0;
      const float shift1 = bf16_bits_to_f32(bias_bits >> 16) - 16.0f * scale1;
      const float shift = h ? shift1 : shift0;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int j = 0; j < 16; ++j)
          acc[pj][mt][j] = __builtin_fmaf(scale1, part[1][pj][mt][j],
                                          __builtin_fmaf(scale0, part[0][pj][mt][j], acc[pj][mt][j]));
        acc[pj][mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(
            xsum[(gi + h) * kRows + mt * 32 + nl], shift, acc[pj][mt], 0, 0, 0);
      }
    }
  };
  if (kRouted) __syncthreads();  // row_ids visible
  fetch_pass(0);
  load_quad(0, 0);
  load_quad(1, 1);
  for (uint32_t q0 = 0; q0 < total_quads; q0 += 2) {
#pragma unroll
    for (int uq = 0; uq < 2; ++uq) {
      const uint32_t quad = q0 + uq;
      if (quad >= total_quads) break;
      if ((uq * 4) % kGroupsPerPass == 0) pass_switch(quad * 4 / kGroupsPerPass);
      consume_pair(uq, 0, 4 * quad);
      consume_pair(uq, 2, 4 * quad + 2);
      load_quad(uq, quad + 2);
    }
  }
  // ---- epilogue and store; lane (column nl, half h) holds rows 8*(j/4) + 4h + j%4 of each tile
  if (column >= a.columns) return;
  for (int mt = 0; mt < MT; ++mt)
    for (int j = 0; j < 16; ++j) {
      const uint32_t row = mt * 32 + 8 * (j / 4) + 4 * h + (j % 4);
      if (row >= count) continue;
      float value = acc[0][mt][j];
      if (kPair) {
        const float gate = value, up = acc[kPair ? 1 : 0][mt][j];
        value = gate * (1.0f / (1.0f + __expf(-gate))) * up;
      }
      const uint64_t out_row = kRouted ? row_ids[row] : first + row;
      const uint64_t at = out_row * a.out_row_stride + column;
      if (!kRouted && a.residual)
        value += bf16_bits_to_f32(a.residual[out_row * a.residual_row_stride + column]);
      if (a.out_f32)
        ((float *)a.out)[at] = value;
      else
        ((uint16_t *)a.out)[at] = (uint16_t)(pack2(value, 0.0f) & 0xffffu);
    }
}

// ---- routed tiles with the whole K resident in LDS ------------------------------------------
//
// A route tile is at most 32 rows, so for K up to 2048 its activations (32 x K bf16, at most
// 128 KB) fit the 160 KB of LDS whole.  A workgroup of eight waves stages the tile once (one
// memory round trip, one barrier) and then every wave streams the packed weights of its own 32
// output columns (both projections for the gate/up pair) with no further synchronisation, a quad
// of groups (one 128-byte line per weight row) at a time, two quads ahead.
// One (tile, column block) unit of qmm_routed_tile_kernel; kSplit: the column block is 4 x 32
// columns and K is split over the workgroup's two wave quartets.  The two forms are separate
// instantiations so that the common one keeps constant wave-to-column and K-range arithmetic.
template <bool kPair, bool kSplit>
__device__ __forceinline__ void routed_tile_unit_body(const QmmArgs &a, uint32_t tile, uint32_t column_block) {
  constexpr int kTileWaves = 8, kTileThreads = 64 * kTileWaves, kRows = 32;
  constexpr int kP = kPair ? 2 : 1;
  constexpr uint32_t waves_across = kSplit ? kTileWaves / 2 : kTileWaves;
  extern __shared__ __attribute__((aligned(16))) unsigned char tile_lds[];
  const uint32_t row_pitch = 2 * a.inner + 16;  // bytes per staged row
  unsigned char *xs = tile_lds;
  float *xsum = (float *)(tile_lds + kRows * row_pitch);      // [K/64][32]
  uint32_t *row_ids = (uint32_t *)(xsum + (a.inner / kGroup) * kRows);
  const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  uint32_t nl = lane & 31, h = lane >> 5;
  asm volatile("" : "+v"(nl), "+v"(h));   // per unit: see pieces_per_row below
  const uint32_t all_quads = a.inner / (4 * kGroup);
  const uint32_t k_half = kSplit ? wave / waves_across : 0;
  const uint32_t total_quads = kSplit ? all_quads / 2 : all_quads;   // this wave's share of K
  const uint32_t quad0 = k_half * total_quads;
  const uint32_t words_per_row = a.inner / 8, groups_per_row = a.inner / kGroup;
  {
    __syncthreads();   // the previous unit is done with row_ids and the staged tile
    const uint32_t expert = a.blocks[3 * tile];
    if (expert == kNoBlock) return;
    const uint32_t first = a.blocks[3 * tile + 1], count = a.blocks[3 * tile + 2];
    if (tid < kRows) row_ids[tid] = tid < count ? a.sorted_routes[first + tid] : 0;
    const uint32_t column = (column_block * waves_across + wave % waves_across) * kColsPerWave + nl;
    const uint32_t column_c = min(column, a.columns - 1);

    const uint32_t *w_row[kP];
    const uint16_t *s_row[kP], *b_row[kP];
    for (int pj = 0; pj < kP; ++pj) {
      w_row[pj] = a.packed[pj] + expert * a.expert_words + (uint64_t)column_c * words_per_row + 4 * h;
      s_row[pj] = a.scales[pj] + expert * a.expert_groups + (uint64_t)column_c * groups_per_row;
      b_row[pj] = a.biases[pj] + expert * a.expert_groups + (uint64_t)column_c * groups_per_row;
    }
    uint4 wq[kP][2][4];
    uint2 scale_q[kP][2], bias_q[kP][2];
    auto load_quad = [&](int slot, uint32_t quad) {
      // unconditional: the tail reloads the last quad
      const uint32_t qd = quad0 + min(quad, total_quads - 1);
      for (int pj = 0; pj < kP; ++pj) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          wq[pj][slot][i] = *(const uint4 *)(w_row[pj] + (uint64_t)(4 * qd + i) * 8);
        scale_q[pj][slot] = *(const uint2 *)(s_row[pj] + 4 * qd);
        bias_q[pj][slot] = *(const uint2 *)(b_row[pj] + 4 * qd);
      }
    };
    load_quad(0, 0);   // cold memory: request before anything else
    load_quad(1, 1);
    __syncthreads();   // row_ids visible
    // ---- stage the tile: permuted inside each 8, with per-group row sums
    // (a fresh value per unit: with a loop-invariant divisor the compiler computes every piece's
    // row and column once, before the loop over units, and carries some forty registers of them
    // through the matrix loop)
    uint32_t pieces_per_row = a.inner / 8, pitch = row_pitch;
    asm volatile("" : "+s"(pieces_per_row), "+s"(pitch));
    const uint32_t pieces = kRows * pieces_per_row;
    for (uint32_t base = 0; base < pieces; base += 8 * kTileThreads) {
      uint4 x_regs[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t piece = base + tid + i * kTileThreads;
        const uint32_t row = piece / pieces_per_row, pc = piece % pieces_per_row;
        x_regs[i] = make_uint4(0, 0, 0, 0);
        if (piece < pieces && row < count)
          x_regs[i] = *(const uint4 *)(a.x + (uint64_t)(row_ids[row] / a.route_div) * a.x_row_stride + 8 * pc);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t piece = base + tid + i * kTileThreads;
        const uint32_t row = piece / pieces_per_row, pc = piece % pieces_per_row;
        const uint4 v = x_regs[i];
        float sum = bf16_bits_to_f32(v.x & 0xffffu) + bf16_bits_to_f32(v.x >> 16) +
                    bf16_bits_to_f32(v.y & 0xffffu) + bf16_bits_to_f32(v.y >> 16) +
                    bf16_bits_to_f32(v.z & 0xffffu) + bf16_bits_to_f32(v.z >> 16) +
                    bf16_bits_to_f32(v.w & 0xffffu) + bf16_bits_to_f32(v.w >> 16);
        sum += __shfl_xor(sum, 1, 64);   // eight consecutive pieces (= lanes) make one group
        sum += __shfl_xor(sum, 2, 64);
        sum += __shfl_xor(sum, 4, 64);
        if (piece < pieces) {
          uint4 permuted;
          permuted.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (x0, x4)
          permuted.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (x1, x5)
          permuted.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (x2, x6)
          permuted.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (x3, x7)
          *(uint4 *)(xs + row * pitch + pc * 16) = permuted;
          if ((pc & 7) == 0) xsum[(pc >> 3) * kRows + row] = sum;
        }
      }
    }
    __syncthreads();

    f32x16 acc[kP];
    for (int pj = 0; pj < kP; ++pj)
      for (int j = 0; j < 16; ++j) acc[pj][j] = 0.0f;
    const unsigned char *my_row = xs + nl * pitch + 64 * h;
    // Two consecutive groups (members i0, i0+1 of ring slot `slot`): independent accumulation
    // chains per group and projection, scales applied per group, bias term as one f32 MFMA over
    // the two groups (lane half h supplies group + h of both operands).
    auto consume_pair = [&](int slot, int i0, uint32_t group) {
      f32x16 part[2][kP];
#pragma unroll
      for (int q = 0; q < 2; ++q)
        for (int pj = 0; pj < kP; ++pj)
          for (int j = 0; j < 16; ++j) part[q][pj][j] = 0.0f;
#pragma unroll
      for (int step = 0; step < 4; ++step)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const uint4 a_raw = *(const uint4 *)(my_row + (group + q) * (2 * kGroup) + 16 * step);
          const bf16x8 a_op = __builtin_bit_cast(bf16x8, a_raw);
#pragma unroll
          for (int pj = 0; pj < kP; ++pj) {
            const uint4 w = wq[pj][slot][i0 + q];
            const bf16x8 b_op =
                unpack_word(step == 0 ? w.x : (step == 1 ? w.y : (step == 2 ? w.z : w.w)));
            part[q][pj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_op, b_op, part[q][pj], 0, 0, 0);
          }
        }
#pragma unroll
      for (int pj = 0; pj < kP; ++pj) {
        const uint32_t scale_bits = i0 == 0 ? scale_q[pj][slot].x : scale_q[pj][slot].y;
        const uint32_t bias_bits = i0 == 0 ? bias_q[pj][slot].x : bias_q[pj][slot].y;
        const float scale0 = bf16_bits_to_f32(scale_bits & 0xffffu);
        const float scale1 = bf16_bits_to_f32(scale_bits >> 16);
        const float shift0 = bf16_bits_to_f32(bias_bits & 0xffffu) - 16.0f * scale0;
        const float shift1 = bf16_bits_to_f32(bias_bits >> 16) - 16.0f * scale1;
#pragma unroll
        for (int j = 0; j < 16; ++j)
          acc[pj][j] = __builtin_fmaf(scale1, part[1][pj][j], __builtin_fmaf(scale0, part[0][pj][j], acc[pj][j]));
        acc[pj] = __builtin_amdgcn_mfma_f32_32x32x2f32(xsum[(group + h) * kRows + nl],
                                                       h ? shift1 : shift0, acc[pj], 0, 0, 0);
      }
    };
    for (uint32_t q0 = 0; q0 < total_quads; q0 += 2) {
#pragma unroll
      for (int uq = 0; uq < 2; ++uq) {
        const uint32_t quad = q0 + uq;
        if (quad >= total_quads) break;
        consume_pair(uq, 0, 4 * (quad0 + quad));
        consume_pair(uq, 2, 4 * (quad0 + quad) + 2);
        load_quad(uq, quad + 2);
      }
    }
    if (kSplit) {
      // the upper K half hands its sums to the quartet that owns the same columns; the staged
      // activations are no longer needed, their LDS carries the hand-over
      float *handed = (float *)tile_lds;   // [4 column groups][kP][16][64]
      const uint32_t group_of_wave = wave % waves_across;
      __syncthreads();
      if (k_half == 1)
        for (int pj = 0; pj < kP; ++pj)
          for (int j = 0; j < 16; ++j) handed[((group_of_wave * kP + pj) * 16 + j) * 64 + lane] = acc[pj][j];
      __syncthreads();
      if (k_half == 0)
        for (int pj = 0; pj < kP; ++pj)
          for (int j = 0; j < 16; ++j) acc[pj][j] += handed[((group_of_wave * kP + pj) * 16 + j) * 64 + lane];
    }
    // ---- epilogue and store; lane (column nl, half h) holds rows 8*(j/4) + 4h + j%4
    if (k_half != 0 || column >= a.columns) return;
    for (int j = 0; j < 16; ++j) {
      const uint32_t row = 8 * (j / 4) + 4 * h + (j % 4);
      if (row >= count) continue;
      float value = acc[0][j];
      if (kPair) {
        const float gate = value, up = acc[kP - 1][j];
        value = gate * (1.0f / (1.0f + __expf(-gate))) * up;
      }
      const uint64_t at = (uint64_t)row_ids[row] * a.out_row_stride + column;
      if (a.out_f32)
        ((float *)a.out)[at] = value;
      else
        ((uint16_t *)a.out)[at] = (uint16_t)(pack2(value, 0.0f) & 0xffffu);
    }
  }
}

template <bool kPair>
__device__ __forceinline__ void routed_tile_unit(const QmmArgs &a, uint32_t tile, uint32_t column_block) {
  routed_tile_unit_body<kPair, false>(a, tile, column_block);
}
template <bool kPair>
__device__ __forceinline__ void routed_tile_unit_split(const QmmArgs &a, uint32_t tile,
                                                       uint32_t column_block) {
  routed_tile_unit_body<kPair, true>(a, tile, column_block);
}

template <bool kPair>
__global__ __launch_bounds__(512) void qmm_routed_tile_kernel(QmmArgs a) {
  constexpr int kTileWaves = 8;
  // Work units are (tile, column block) pairs; the launch has as many workgroups as are resident
  // at once (the staged tile fills most of a CU's LDS) and every workgroup walks the units
  // unit, unit + gridDim.x, ...: the number of tiles is only known on the device, and a grid
  // sized for the worst case would spend its time retiring workgroups that have nothing to do.
  // Usually a column block is the 8 x 32 columns of the eight waves.  When the routes fall on
  // few tiles (few experts hit, many rows each) that would leave most of the device idle behind
  // long per-wave chains; a column block is then 4 x 32 columns and K is split over the two
  // wave quartets, whose sums meet in LDS.
  const uint32_t tiles = a.n_blocks[0];
  const uint32_t wide_blocks = (a.columns + kTileWaves * kColsPerWave - 1) / (kTileWaves * kColsPerWave);
  const uint32_t all_quads = a.inner / (4 * kGroup);
  // (only the gate/up pair: its launches are the ones with few column blocks)
  const bool split_k = kPair && (uint64_t)tiles * wide_blocks <= a.split_below && all_quads % 2 == 0;
  const uint32_t waves_across = split_k ? kTileWaves / 2 : kTileWaves;
  const uint32_t column_blocks =
      (a.columns + waves_across * kColsPerWave - 1) / (waves_across * kColsPerWave);
  // unit -> (tile, column block) without a division per step
  const uint32_t tile_step = gridDim.x / column_blocks, block_step = gridDim.x % column_blocks;
  uint32_t tile = blockIdx.x / column_blocks, column_block = blockIdx.x % column_blocks;
  while (tile < tiles) {
    if (kPair && split_k)
      routed_tile_unit_split<true>(a, tile, column_block);
    else
      routed_tile_unit<kPair>(a, tile, column_block);
    tile += tile_step;
    column_block += block_step;
    if (column_block >= column_blocks) {
      column_block -= column_blocks;
      ++tile;
    }
  }
}

constexpr uint32_t kTileMaxInner = 2048;   // 32 x 2048 bf16 + sums = 133 KB of the 160 KB of LDS

inline uint32_t routed_tile_lds_bytes(uint32_t inner) {
  return 32 * (2 * inner + 16) + (inner / kGroup) * 32 * 4 + 32 * 4;
}

// ---- decode-sized dense products: at most 128 activation rows -------------------------------
//
// With so few rows the weights are a few megabytes, and what a compute unit can pull from L2
// (about 50 GB/s) bounds the launch long before HBM does.  So the product is cut into slabs that
// make every byte a CU fetches count: a workgroup of eight waves takes 256 output columns (32
// per wave) and 256 values of K for all rows, stages that activation slab in LDS once (64 KB for
// 128 rows), and every wave contracts it with its own four groups of packed weights, which were
// requested before anything else.  There is a single pass and a single barrier.  The K slabs of
// a column block leave f32 partial tiles in workspace and sum_slabs_kernel adds them in slab
// order (a fixed order: results do not depend on scheduling).
struct SlabArgs {
  const uint16_t *x;
  uint64_t x_row_stride;
  const uint32_t *packed;
  const uint16_t *scales, *biases;
  float *partials;      // [K/256][rows][columns]
  void *out;            // used directly when there is a single slab
  uint64_t out_row_stride;
  uint32_t out_f32;
  uint32_t rows, inner, columns;
};

constexpr int kSlabK = 256, kSlabWaves = 8, kSlabThreads = 64 * kSlabWaves;
constexpr int kSlabP = 1;                     // 32-column operands per wave
constexpr int kSlabColsPerWave = 32 * kSlabP;
constexpr int kSlabPitch = 2 * kSlabK + 16;   // bytes per staged row

template <int MT>
constexpr uint32_t slab_lds_bytes() {
  return 32 * MT * kSlabPitch + (kSlabK / kGroup) * 32 * MT * 4;
}

template <int MT>
__global__ __launch_bounds__(kSlabThreads) void qmm_slab_kernel(SlabArgs a) {
  constexpr int kP = kSlabP;
  constexpr int kRows = 32 * MT;
  constexpr int kGroups = kSlabK / kGroup;   // 4
  extern __shared__ __attribute__((aligned(16))) unsigned char slab_lds[];
  unsigned char *xs = slab_lds;
  float *xsum = (float *)(slab_lds + kRows * kSlabPitch);
  const uint32_t tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const uint32_t nl = lane & 31, h = lane >> 5;
  const uint32_t slab = blockIdx.y, k0 = slab * kSlabK;
  const uint32_t groups_per_row = a.inner / kGroup;
  uint32_t column[kP];
  for (int pj = 0; pj < kP; ++pj)
    column[pj] = (blockIdx.x * kSlabWaves + wave) * kSlabColsPerWave + 32 * pj + nl;

  // weights first: they come from cold memory
  uint4 wq[kP][kGroups];
  uint32_t scale_bits[kP][kGroups], bias_bits[kP][kGroups];
#pragma unroll
  for (int pj = 0; pj < kP; ++pj) {
    const uint32_t column_c = min(column[pj], a.columns - 1);
    const uint32_t *w_row = a.packed + (uint64_t)column_c * (a.inner / 8) + k0 / 8 + 4 * h;
    const uint16_t *s_row = a.scales + (uint64_t)column_c * groups_per_row + k0 / kGroup;
    const uint16_t *b_row = a.biases + (uint64_t)column_c * groups_per_row + k0 / kGroup;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) {
      wq[pj][g] = *(const uint4 *)(w_row + 8 * g);
      scale_bits[pj][g] = s_row[g];
      bias_bits[pj][g] = b_row[g];
    }
  }
  // stage the activation slab: permuted inside each 8, with per-group row sums
  constexpr int kPieces = kRows * (kSlabK / 8) / kSlabThreads;
#pragma unroll
  for (int i0 = 0; i0 < kPieces; i0 += 8) {
    uint4 x_regs[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i0 + i >= kPieces) break;
      const uint32_t piece = tid + (i0 + i) * kSlabThreads;
      const uint32_t row = piece / (kSlabK / 8), pc = piece % (kSlabK / 8);
      x_regs[i] = make_uint4(0, 0, 0, 0);
      if (row < a.rows)
        x_regs[i] = *(const uint4 *)(a.x + (uint64_t)row * a.x_row_stride + k0 + 8 * pc);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (i0 + i >= kPieces) break;
      const uint32_t piece = tid + (i0 + i) * kSlabThreads;
      const uint32_t row = piece / (kSlabK / 8), pc = piece % (kSlabK / 8);
      const uint4 v = x_regs[i];
      float sum = bf16_bits_to_f32(v.x & 0xffffu) + bf16_bits_to_f32(v.x >> 16) +
                  bf16_bits_to_f32(v.y & 0xffffu) + bf16_bits_to_f32(v.y >> 16) +
                  bf16_bits_to_f32(v.z & 0xffffu) + bf16_bits_to_f32(v.z >> 16) +
                  bf16_bits_to_f32(v.w & 0xffffu) + bf16_bits_to_f32(v.w >> 16);
      sum += __shfl_xor(sum, 1, 64);   // eight consecutive pieces (= lanes) make one group
      sum += __shfl_xor(sum, 2, 64);
      sum += __shfl_xor(sum, 4, 64);
      uint4 permuted;
      permuted.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (x0, x4)
      permuted.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (x1, x5)
      permuted.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (x2, x6)
      permuted.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (x3, x7)
      *(uint4 *)(xs + row * kSlabPitch + pc * 16) = permuted;
      if ((pc & 7) == 0) xsum[(pc >> 3) * kRows + row] = sum;
    }
  }
  __syncthreads();

  f32x16 acc[kP][MT];
  for (int pj = 0; pj < kP; ++pj)
    for (int mt = 0; mt < MT; ++mt)
      for (int j = 0; j < 16; ++j) acc[pj][mt][j] = 0.0f;
  // The bias term sum_g (bias_g - 16 scale_g) * xsum_g[row] is itself a small product over the
  // groups: an f32 MFMA (K = 2 groups per instruction; lane half h supplies group 2p + h of
  // both operands) adds it straight into the accumulators.
#pragma unroll
  for (int pair = 0; pair < kGroups / 2; ++pair)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const float sums = xsum[(2 * pair + h) * kRows + mt * 32 + nl];
#pragma unroll
      for (int pj = 0; pj < kP; ++pj) {
        const float shift_even = bf16_bits_to_f32(bias_bits[pj][2 * pair]) -
                                 16.0f * bf16_bits_to_f32(scale_bits[pj][2 * pair]);
        const float shift_odd = bf16_bits_to_f32(bias_bits[pj][2 * pair + 1]) -
                                16.0f * bf16_bits_to_f32(scale_bits[pj][2 * pair + 1]);
        acc[pj][mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(sums, h ? shift_odd : shift_even,
                                                           acc[pj][mt], 0, 0, 0);
      }
    }
  // The group loop is kept rolled (a compact body keeps the register count down); the weight
  // registers rotate so that slot 0 is always the current group.
#pragma unroll 1
  for (int g = 0; g < kGroups; ++g) {
    bf16x8 b_op[kP][4];
    float scale[kP];
#pragma unroll
    for (int pj = 0; pj < kP; ++pj) {
      scale[pj] = bf16_bits_to_f32(scale_bits[pj][0]);
      b_op[pj][0] = unpack_word(wq[pj][0].x);
      b_op[pj][1] = unpack_word(wq[pj][0].y);
      b_op[pj][2] = unpack_word(wq[pj][0].z);
      b_op[pj][3] = unpack_word(wq[pj][0].w);
    }
    // up to four independent accumulation chains at a time keep the matrix pipe busy
    constexpr int kChunk = (MT * kP >= 4) ? 4 / kP : MT;
#pragma unroll
    for (int mt0 = 0; mt0 < MT; mt0 += kChunk) {
      f32x16 part[kP][kChunk];
#pragma unroll
      for (int pj = 0; pj < kP; ++pj)
        for (int c = 0; c < kChunk; ++c)
          for (int j = 0; j < 16; ++j) part[pj][c][j] = 0.0f;
#pragma unroll
      for (int step = 0; step < 4; ++step)
#pragma unroll
        for (int c = 0; c < kChunk; ++c) {
          const uint4 a_raw = *(const uint4 *)(xs + ((mt0 + c) * 32 + nl) * kSlabPitch +
                                               (g * kGroup + 32 * h + 8 * step) * 2);
          const bf16x8 a_op = __builtin_bit_cast(bf16x8, a_raw);
#pragma unroll
          for (int pj = 0; pj < kP; ++pj)
            part[pj][c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_op, b_op[pj][step],
                                                                  part[pj][c], 0, 0, 0);
        }
#pragma unroll
      for (int pj = 0; pj < kP; ++pj)
#pragma unroll
        for (int c = 0; c < kChunk; ++c)
#pragma unroll
          for (int j = 0; j < 16; ++j) acc[pj][mt0 + c][j] += scale[pj] * part[pj][c][j];
    }
#pragma unroll
    for (int pj = 0; pj < kP; ++pj)
#pragma unroll
      for (int r = 0; r + 1 < kGroups; ++r) {
        wq[pj][r] = wq[pj][r + 1];
        scale_bits[pj][r] = scale_bits[pj][r + 1];
      }
  }
  const bool direct = gridDim.y == 1;
  float *mine = a.partials + (uint64_t)slab * a.rows * a.columns;
#pragma unroll
  for (int pj = 0; pj < kP; ++pj) {
    if (column[pj] >= a.columns) continue;
    for (int mt = 0; mt < MT; ++mt)
      for (int j = 0; j < 16; ++j) {
        const uint32_t row = mt * 32 + 8 * (j / 4) + 4 * h + (j % 4);
        if (row >= a.rows) continue;
        if (!direct) {
          mine[(uint64_t)row * a.columns + column[pj]] = acc[pj][mt][j];
        } else {
          const uint64_t at = (uint64_t)row * a.out_row_stride + column[pj];
          if (a.out_f32)
            ((float *)a.out)[at] = acc[pj][mt][j];
          else
            ((uint16_t *)a.out)[at] = (uint16_t)(pack2(acc[pj][mt][j], 0.0f) & 0xffffu);
        }
      }
  }
}

// out[row, column] = sum over slabs (ascending) of partials[slab][row][column]; a thread takes
// four consecutive columns (the host guarantees columns % 4 == 0 and aligned output rows).
__global__ void sum_slabs_kernel(const float *partials, uint32_t slabs, uint32_t rows,
                                 uint32_t columns, void *out, uint64_t out_row_stride,
                                 uint32_t out_f32, const uint16_t *residual,
                                 uint64_t residual_row_stride) {
  const uint64_t flat = 4 * ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x);
  const uint64_t plane = (uint64_t)rows * columns;
  if (flat >= plane) return;
  float4 total = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  for (uint32_t s = 0; s < slabs; ++s) {
    const float4 v = *(const float4 *)(partials + s * plane + flat);
    total.x += v.x;
    total.y += v.y;
    total.z += v.z;
    total.w += v.w;
  }
  const uint64_t at = (flat / columns) * out_row_stride + flat % columns;
  if (residual) {   // four bf16 values, added before the result is rounded
    const uint2 r = *(const uint2 *)(residual + (flat / columns) * residual_row_stride + flat % columns);
    total.x += __uint_as_float(r.x << 16);
    total.y += __uint_as_float(r.x & 0xffff0000u);
    total.z += __uint_as_float(r.y << 16);
    total.w += __uint_as_float(r.y & 0xffff0000u);
  }
  if (out_f32) {
    *(float4 *)((float *)out + at) = total;
  } else {
    uint2 packed;
    packed.x = pack2(total.x, total.y);
    packed.y = pack2(total.z, total.w);
    *(uint2 *)((uint16_t *)out + at) = packed;
  }
}

// out[r, :] = residual[r, :] + sum_s weights[r, s] * partial[r*k + s, :], slots in ascending
// order (execute_gather_quant_weighted_sum, crates/forja-cpu/src/lib.rs:1153-1199); routes that
// name no valid expert contribute nothing.
__global__ void combine_routes_kernel(const float *partial, View indices, View weights,
                                      View residual, int has_residual, View out, uint32_t rows,
                                      uint32_t routes, uint32_t columns, uint32_t experts) {
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)rows * columns) return;
  uint32_t row = (uint32_t)(flat / columns), column = (uint32_t)(flat % columns);
  float value = 0.0f;
  for (uint32_t slot = 0; slot < routes; ++slot) {
    uint32_t expert = load_u32_at(indices, indices.offset + row * indices.stride[0] +
                                               slot * indices.stride[1]);
    if (expert >= experts) continue;
    float weight = load_float_at(weights, weights.offset + row * weights.stride[0] +
                                              slot * weights.stride[1]);
    value += weight * partial[((uint64_t)row * routes + slot) * columns + column];
  }
  if (has_residual)
    value += load_float_at(residual, residual.offset + row * residual.stride[0] +
                                         column * residual.stride[1]);
  store_float_at(out, out.offset + row * out.stride[0] + column * out.stride[1], value);
}

// The same sum for bf16 rows with 8-byte aligned columns: a thread owns four consecutive columns
// of a row, fetches the row's (expert, weight) pairs first and then all its partial rows at once
// (at most kMax routes), and adds them in ascending slot order.
template <int kMax>
__global__ __launch_bounds__(256) void combine_routes_rows_kernel(
    const float *partial, View indices, View weights, const uint16_t *residual,
    uint64_t residual_row_stride, uint16_t *out, uint64_t out_row_stride, uint32_t rows,
    uint32_t routes, uint32_t columns, uint32_t experts) {
  const uint64_t flat = 4 * ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x);
  if (flat >= (uint64_t)rows * columns) return;
  const uint32_t row = (uint32_t)(flat / columns), column = (uint32_t)(flat % columns);
  float weight[kMax];
  float4 part[kMax];
#pragma unroll
  for (int slot = 0; slot < kMax; ++slot) {
    weight[slot] = 0.0f;
    part[slot] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if ((uint32_t)slot < routes) {
      const uint32_t expert = load_u32_at(indices, indices.offset + row * indices.stride[0] +
                                                       slot * indices.stride[1]);
      if (expert < experts) {
        weight[slot] = load_float_at(weights, weights.offset + row * weights.stride[0] +
                                                  slot * weights.stride[1]);
        part[slot] = *(const float4 *)(partial + ((uint64_t)row * routes + slot) * columns + column);
      }
    }
  }
  float4 value = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
  for (int slot = 0; slot < kMax; ++slot) {   // a skipped route adds +0 * 0: no effect
    value.x += weight[slot] * part[slot].x;
    value.y += weight[slot] * part[slot].y;
    value.z += weight[slot] * part[slot].z;
    value.w += weight[slot] * part[slot].w;
  }
  if (residual) {
    const uint2 r = *(const uint2 *)(residual + (uint64_t)row * residual_row_stride + column);
    value.x += bf16_bits_to_f32(r.x & 0xffffu);
    value.y += bf16_bits_to_f32(r.x >> 16);
    value.z += bf16_bits_to_f32(r.y & 0xffffu);
    value.w += bf16_bits_to_f32(r.y >> 16);
  }
  *(uint2 *)(out + (uint64_t)row * out_row_stride + column) =
      make_uint2(pack2(value.x, value.y), pack2(value.z, value.w));
}

bool rows_contiguous(const View &v, uint32_t rank) {
  // innermost axis contiguous and every outer stride the dense product (weights, scales)
  uint64_t expected = 1;
  for (int axis = (int)rank - 1; axis >= 0; --axis) {
    if (v.shape[axis] != 1 && v.stride[axis] != expected) return false;
    expected *= v.shape[axis];
  }
  return true;
}

bool weights_eligible(const View &packed, const View &scales, const View &biases, uint32_t rank,
                      uint32_t inner, uint32_t bits, uint32_t group) {
  if (bits != 4 || group != kGroup || inner % 256 != 0) return false;
  if (scales.dtype != FH_BF16 || biases.dtype != FH_BF16) return false;
  if (!rows_contiguous(packed, rank) || !rows_contiguous(scales, rank) ||
      !rows_contiguous(biases, rank))
    return false;
  if (packed.offset % 4 != 0) return false;  // 16-byte aligned rows (K/8 words is a multiple of 32)
  if (scales.offset % 4 != 0 || biases.offset % 4 != 0) return false;  // 8-byte aligned quads
  return true;
}

template <bool kPair, bool kRouted>
void launch_qmm(hipStream_t stream, const QmmArgs &a, uint32_t row_blocks, int mt) {
  uint32_t wide_blocks = (a.columns + kWaves * kColsPerWave - 1) / (kWaves * kColsPerWave);
  dim3 grid(wide_blocks, row_blocks);
  if (mt == 1)
    qmm_mfma_kernel<1, kPair, kRouted><<<grid, 256, 0, stream>>>(a);
  else
    qmm_mfma_kernel<2, kPair, kRouted><<<grid, 256, 0, stream>>>(a);
}

// ---- decode-sized dense products, one kernel, no partial tiles in memory ----------------------
//
// A workgroup owns one 32 x 32 output tile (32 rows, 32 columns) for the whole of K and splits K
// over its waves in 256-value pieces (one 128-byte line of every packed weight row, so each line
// is fetched once).  Nothing is staged: a lane loads the 16-byte activation pieces of "its" row
// and K half straight into MFMA operand registers (permuted in registers to the order in which
// nibbles unpack) and sums them per group for the bias term.  The waves' 32 x 32 sums meet in LDS
// and wave 0 adds them in wave order (fixed: results do not depend on scheduling), adds the
// optional residual and stores.  Activations are re-read from L2 by every column tile and
// weights by every row tile; at decode sizes that is cheaper than writing f32 partial tiles to
// memory and summing them in a second launch.
struct TileProductArgs {
  const uint16_t *x;
  uint64_t x_row_stride;
  const uint32_t *packed;
  const uint16_t *scales, *biases;
  void *out;
  uint64_t out_row_stride;
  uint32_t out_f32;
  const uint16_t *residual;
  uint64_t residual_row_stride;
  uint32_t rows, inner, columns;
};

constexpr int kTileProductWaves = 8;

template <int kCols>   // 32-column tiles per wave: they share the wave's activation registers
__global__ __launch_bounds__(64 * kTileProductWaves) void qmm_tile_product_kernel(TileProductArgs a) {
  __shared__ float handed[kTileProductWaves - 1][kCols][16][64];
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
  const uint32_t nl = lane & 31, h = lane >> 5;
  const uint32_t row = blockIdx.y * 32 + nl;
  const bool row_live = row < a.rows;
  const uint32_t quads = a.inner / 256, groups_per_row = a.inner / kGroup;
  uint32_t column[kCols];
  const uint32_t *w_row[kCols];
  const uint16_t *s_row[kCols], *b_row[kCols];
#pragma unroll
  for (int c = 0; c < kCols; ++c) {
    column[c] = (blockIdx.x * kCols + c) * 32 + nl;
    const uint32_t column_c = min(column[c], a.columns - 1);
    w_row[c] = a.packed + (uint64_t)column_c * (a.inner / 8) + 4 * h;
    s_row[c] = a.scales + (uint64_t)column_c * groups_per_row;
    b_row[c] = a.biases + (uint64_t)column_c * groups_per_row;
  }
  const uint16_t *x_row = a.x + (uint64_t)min(row, a.rows - 1) * a.x_row_stride + 32 * h;
  f32x16 acc[kCols];
  for (int c = 0; c < kCols; ++c)
    for (int j = 0; j < 16; ++j) acc[c][j] = 0.0f;
  for (uint32_t quad = wave; quad < quads; quad += waves) {
    uint4 wq[kCols][4], xq[4][4];
    uint2 scale4[kCols], bias4[kCols];
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
#pragma unroll
      for (int i = 0; i < 4; ++i) wq[c][i] = *(const uint4 *)(w_row[c] + (uint64_t)(4 * quad + i) * 8);
      scale4[c] = *(const uint2 *)(s_row[c] + 4 * quad);
      bias4[c] = *(const uint2 *)(b_row[c] + 4 * quad);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int step = 0; step < 4; ++step) {
        xq[i][step] = make_uint4(0, 0, 0, 0);
        if (row_live) xq[i][step] = *(const uint4 *)(x_row + 256 * quad + 64 * i + 8 * step);
      }
    float group_sum[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float half_sum = 0.0f;
#pragma unroll
      for (int step = 0; step < 4; ++step) {
        const uint4 v = xq[i][step];
        half_sum += bf16_bits_to_f32(v.x & 0xffffu) + bf16_bits_to_f32(v.x >> 16) +
                    bf16_bits_to_f32(v.y & 0xffffu) + bf16_bits_to_f32(v.y >> 16) +
                    bf16_bits_to_f32(v.z & 0xffffu) + bf16_bits_to_f32(v.z >> 16) +
                    bf16_bits_to_f32(v.w & 0xffffu) + bf16_bits_to_f32(v.w >> 16);
        // the operand order in which nibbles unpack: (x0,x4)(x1,x5)(x2,x6)(x3,x7)
        uint4 permuted;
        permuted.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
        permuted.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
        permuted.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
        permuted.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
        xq[i][step] = permuted;
      }
      group_sum[i] = half_sum + __shfl_xor(half_sum, 32, 64);   // both K halves of the group
    }
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
      float shift[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t s_bits = (i < 2 ? scale4[c].x : scale4[c].y) >> (16 * (i & 1)) & 0xffffu;
        const uint32_t b_bits = (i < 2 ? bias4[c].x : bias4[c].y) >> (16 * (i & 1)) & 0xffffu;
        const float scale = bf16_bits_to_f32(s_bits);
        shift[i] = bf16_bits_to_f32(b_bits) - 16.0f * scale;
        f32x16 part;
        for (int j = 0; j < 16; ++j) part[j] = 0.0f;
#pragma unroll
        for (int step = 0; step < 4; ++step) {
          const uint4 w = wq[c][i];
          const uint32_t word = step == 0 ? w.x : (step == 1 ? w.y : (step == 2 ? w.z : w.w));
          part = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, xq[i][step]),
                                                         unpack_word(word), part, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[c][j] += scale * part[j];
      }
      // bias term of the four groups: two f32 MFMAs, lane half h supplying group 2p + h
#pragma unroll
      for (int p2 = 0; p2 < 2; ++p2)
        acc[c] = __builtin_amdgcn_mfma_f32_32x32x2f32(h ? group_sum[2 * p2 + 1] : group_sum[2 * p2],
                                                      h ? shift[2 * p2 + 1] : shift[2 * p2], acc[c], 0, 0, 0);
    }
  }
  if (wave != 0)
    for (int c = 0; c < kCols; ++c)
      for (int j = 0; j < 16; ++j) handed[wave - 1][c][j][lane] = acc[c][j];
  __syncthreads();
  if (wave != 0) return;
  for (int c = 0; c < kCols; ++c) {
    if (column[c] >= a.columns) continue;
    for (uint32_t other = 0; other + 1 < waves; ++other)
      for (int j = 0; j < 16; ++j) acc[c][j] += handed[other][c][j][lane];
    for (int j = 0; j < 16; ++j) {
      const uint32_t out_row = blockIdx.y * 32 + 8 * (j / 4) + 4 * h + (j % 4);
      if (out_row >= a.rows) continue;
      float value = acc[c][j];
      if (a.residual)
        value += bf16_bits_to_f32(a.residual[(uint64_t)out_row * a.residual_row_stride + column[c]]);
      const uint64_t at = (uint64_t)out_row * a.out_row_stride + column[c];
      if (a.out_f32)
        ((float *)a.out)[at] = value;
      else
        ((uint16_t *)a.out)[at] = (uint16_t)(pack2(value, 0.0f) & 0xffffu);
    }
  }
}

void launch_tile_product(fh_backend *backend, const QmmArgs &q, const uint16_t *residual,
                         uint64_t residual_row_stride) {
  TileProductArgs t{};
  t.x = q.x;
  t.x_row_stride = q.x_row_stride;
  t.packed = q.packed[0];
  t.scales = q.scales[0];
  t.biases = q.biases[0];
  t.out = q.out;
  t.out_row_stride = q.out_row_stride;
  t.out_f32 = q.out_f32;
  t.residual = residual;
  t.residual_row_stride = residual_row_stride;
  t.rows = q.rows;
  t.inner = q.inner;
  t.columns = q.columns;
  const uint32_t quads = q.inner / 256, column_tiles = (q.columns + 31) / 32, row_tiles = (q.rows + 31) / 32;
  const uint32_t waves = quads < (uint32_t)kTileProductWaves ? quads : (uint32_t)kTileProductWaves;
  KernelTimer timer(backend, FH_KC_QMM_KERNEL);
  qmm_tile_product_kernel<1><<<dim3(column_tiles, row_tiles), 64 * waves, 0, backend_stream(backend)>>>(t);
}

// Decode-sized dense product through the slab kernels; false when workspace is short.
template <int MT>
void launch_slab(hipStream_t stream, const SlabArgs &s, dim3 grid) {
  static bool configured = false;   // raise the dynamic LDS limit once per process
  if (!configured) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&qmm_slab_kernel<MT>),
                              hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)slab_lds_bytes<MT>());
    configured = true;
  }
  qmm_slab_kernel<MT><<<grid, kSlabThreads, slab_lds_bytes<MT>(), stream>>>(s);
}

bool launch_skinny(fh_backend *backend, const QmmArgs &q, const uint16_t *residual,
                   uint64_t residual_row_stride) {
  hipStream_t stream = backend_stream(backend);
  const uint32_t slabs = q.inner / kSlabK;
  const uint64_t plane = (uint64_t)q.rows * q.columns;
  SlabArgs s{};
  if (slabs > 1) {
    s.partials = (float *)backend_workspace(backend, slabs * plane * sizeof(float));
    if (!s.partials) return false;
  }
  s.x = q.x;
  s.x_row_stride = q.x_row_stride;
  s.packed = q.packed[0];
  s.scales = q.scales[0];
  s.biases = q.biases[0];
  s.out = q.out;
  s.out_row_stride = q.out_row_stride;
  s.out_f32 = q.out_f32;
  s.rows = q.rows;
  s.inner = q.inner;
  s.columns = q.columns;
  KernelTimer timer(backend, FH_KC_QMM_KERNEL);
  dim3 grid((q.columns + kSlabWaves * kSlabColsPerWave - 1) / (kSlabWaves * kSlabColsPerWave), slabs);
  if (q.rows <= 32)
    launch_slab<1>(stream, s, grid);
  else if (q.rows <= 64)
    launch_slab<2>(stream, s, grid);
  else
    launch_slab<4>(stream, s, grid);
  if (slabs > 1)
    sum_slabs_kernel<<<(uint32_t)((plane / 4 + 255) / 256), 256, 0, stream>>>(
        s.partials, slabs, q.rows, q.columns, q.out, q.out_row_stride, q.out_f32, residual,
        residual_row_stride);
  return true;
}

const uint32_t *u32_ptr(const View &v) { return (const uint32_t *)v.base + v.offset; }
const uint16_t *u16_ptr(const View &v) { return (const uint16_t *)v.base + v.offset; }

}  // namespace

namespace {

// f32 activations (the engines' own activation dtype) on the matrix cores: each value goes in as
// three bf16 pieces that add up to it exactly, so nothing of it is rounded away before the f32
// accumulation.  Decode batches of at most 32 rows, f32 results.
bool try_wide_quant_matmul(fh_backend *backend, const QmmProblem &p) {
  if (p.out.dtype != FH_F32 || p.out.stride[1] != 1) return false;
  if (!weights_eligible(p.packed, p.scales, p.biases, 2, p.inner, p.bits, p.group)) return false;
  if (p.x.stride[1] != 1 || p.x.stride[0] % 4 != 0 || p.x.offset % 4 != 0) return false;
  // K = 4096 (three pieces of so long a slice do not fit the registers): two launches over half
  // the K each, the second adding to what the first stored
  const uint32_t ranges = p.inner == 4096 ? 2 : 1, range = p.inner / ranges;
  if (!ksplit_dense_supports(p.rows, range, p.columns, true)) return false;
  const float *residual = nullptr;
  uint64_t residual_row_stride = 0;
  if (p.residual) {
    const View &r = *p.residual;
    if (r.dtype != FH_F32 || r.stride[1] != 1) return false;
    residual = (const float *)r.base + r.offset;
    residual_row_stride = r.stride[0];
  }
  float *out = (float *)p.out.base + p.out.offset;
  for (uint32_t i = 0; i < ranges; ++i) {
    const uint32_t first = i * range;
    KsplitDense d{(const float *)p.x.base + p.x.offset + first, p.x.stride[0], u32_ptr(p.packed) + first / 8,
                  u16_ptr(p.scales) + first / kGroup, u16_ptr(p.biases) + first / kGroup, out, p.out.stride[0], 1,
                  i == 0 ? (const void *)residual : (const void *)out,
                  i == 0 ? residual_row_stride : p.out.stride[0], p.rows, range, p.columns, true, p.inner};
    if (!launch_ksplit_dense(backend, d)) return false;   // (refused before anything ran: same answer for every range)
  }
  return true;
}

}  // namespace

bool try_fast_quant_matmul(fh_backend *backend, const QmmProblem &p) {
  hipStream_t stream = backend_stream(backend);
  if (p.x.dtype == FH_F32) return try_wide_quant_matmul(backend, p);
  if (p.x.dtype != FH_BF16) return false;
  if (p.out.dtype != FH_BF16 && p.out.dtype != FH_F32) return false;
  if (!weights_eligible(p.packed, p.scales, p.biases, 2, p.inner, p.bits, p.group)) return false;
  if (p.x.stride[1] != 1 || p.x.stride[0] % 8 != 0 || p.x.offset % 8 != 0) return false;
  if (p.out.stride[1] != 1) return false;
  QmmArgs a{};
  a.x = u16_ptr(p.x);
  a.x_row_stride = p.x.stride[0];
  a.packed[0] = u32_ptr(p.packed);
  a.scales[0] = u16_ptr(p.scales);
  a.biases[0] = u16_ptr(p.biases);
  a.out = p.out.dtype == FH_F32 ? (void *)((float *)p.out.base + p.out.offset)
                                : (void *)((uint16_t *)p.out.base + p.out.offset);
  a.out_row_stride = p.out.stride[0];
  a.out_f32 = p.out.dtype == FH_F32;
  a.rows = p.rows;
  a.inner = p.inner;
  a.columns = p.columns;
  const uint16_t *residual = nullptr;
  uint64_t residual_row_stride = 0;
  if (p.residual) {
    const View &r = *p.residual;
    if (r.dtype != FH_BF16 || p.out.dtype != FH_BF16 || r.stride[1] != 1 || r.stride[0] % 4 != 0 ||
        r.offset % 4 != 0)
      return false;
    residual = u16_ptr(r);
    residual_row_stride = r.stride[0];
  }
  // Decode rows whose weights stay cached between row tiles: K split over the waves of a
  // workgroup, the rows stationary in registers.
  if (ksplit_dense_supports(p.rows, p.inner, p.columns)) {
    KsplitDense d{a.x, a.x_row_stride, a.packed[0], a.scales[0], a.biases[0], a.out, a.out_row_stride,
                  a.out_f32, residual, residual_row_stride, p.rows, p.inner, p.columns};
    if (launch_ksplit_dense(backend, d)) return true;
  }
  // Decode rows.  When one workgroup per compute unit covers the output, the single-kernel tile
  // product; wider outputs go through the K slabs.
  if (p.rows <= 128 &&
      (uint64_t)((p.columns + 31) / 32) * ((p.rows + 31) / 32) <= 3 * backend_compute_units(backend)) {
    launch_tile_product(backend, a, residual, residual_row_stride);
    return true;
  }
  if (p.rows <= 128 && p.columns <= 16384 && p.columns % 4 == 0 && p.out.stride[0] % 4 == 0 &&
      p.out.offset % 4 == 0 && (!residual || p.inner > kSlabK)) {
    if (!launch_skinny(backend, a, residual, residual_row_stride)) return false;
    return true;
  }
  a.residual = residual;
  a.residual_row_stride = residual_row_stride;
  KernelTimer timer(backend, FH_KC_QMM_KERNEL);
  // (also a full decode batch against a vocabulary-sized matrix: 128 x 151936 x 2048 takes 132 us
  // through the GEMM's 128 x 128 tiles and 224 us through the streaming kernel, which reads the
  // weights once per 64 rows)
  if (p.rows > 128 || (p.rows > 64 && p.columns >= 32768)) {
    // the tiled GEMM, followed by the any-range kernel conditioned on the GEMM's refusal
    const uint32_t *refused = nullptr;
    if (launch_quant_gemm(backend, p, &refused)) {
      if (!refused) return true;   // weights known to be in range: the GEMM has done the product
      a.run_if_set = refused;
    }
  }
  int mt = p.rows <= 32 ? 1 : 2;
  uint32_t row_blocks = (p.rows + 32 * mt - 1) / (32 * mt);
  launch_qmm<false, false>(stream, a, row_blocks, mt);
  return true;
}

namespace {

constexpr uint32_t kRouteTile = 32;

struct RoutePlan {
  uint32_t *counts, *offsets, *sorted_routes, *blocks, *n_blocks;
  uint32_t max_blocks;
  char *rest;  // workspace after the plan
  bool reused; // nothing was packed for this call
};

// Packs the routes on the device (or reuses the plan the previous routed projection packed from
// the same indices); `extra` bytes of ordinary workspace are returned in plan->rest.
bool plan_routes(fh_backend *backend, const GatherProblem &p, uint64_t extra, ErrorSlot *error,
                 RoutePlan *plan, uint32_t *zero_rows = nullptr, uint32_t zero_row_words = 0,
                 uint32_t tile = kRouteTile) {
  uint64_t routes = (uint64_t)p.rows * p.k;
  plan->max_blocks = p.experts + (uint32_t)(routes / tile) + 1;
  auto round = [](uint64_t bytes) { return (bytes + 255) / 256 * 256; };
  uint64_t counts_b = round(p.experts * 4ull), offsets_b = round((p.experts + 1) * 4ull),
           sorted_b = round(routes * 4), blocks_b = round(plan->max_blocks * 12ull), nb_b = 256;
  RoutePlanKey key{p.indices_buffer, p.indices.offset, p.indices.stride[0], p.indices.stride[1],
                   p.rows, p.k, p.experts, tile};
  bool reuse = false;
  char *ws = backend_route_plan(backend, key, counts_b + offsets_b + sorted_b + blocks_b + nb_b, &reuse);
  if (!ws) return false;
  plan->rest = nullptr;
  if (extra) {
    plan->rest = backend_workspace(backend, extra);
    if (!plan->rest) return false;
  }
  plan->counts = (uint32_t *)ws;
  ws += counts_b;
  plan->offsets = (uint32_t *)ws;
  ws += offsets_b;
  plan->sorted_routes = (uint32_t *)ws;
  ws += sorted_b;
  plan->blocks = (uint32_t *)ws;
  ws += blocks_b;
  plan->n_blocks = (uint32_t *)ws;
  plan->reused = reuse;
  if (!reuse)
    launch_route_pack(backend_stream(backend), p.indices, p.rows, p.k, p.experts, tile,
                      plan->counts, plan->offsets, plan->sorted_routes, plan->blocks,
                      plan->max_blocks, plan->n_blocks, error, zero_rows, zero_row_words);
  return true;
}

// Routed product over the packed tiles: whole-K tile kernel when the tile fits LDS, else the
// multi-pass kernel.
template <bool kPair>
void launch_routed(hipStream_t stream, const QmmArgs &a, uint32_t max_blocks, uint32_t resident /* CUs */) {
  if (a.inner <= kTileMaxInner) {
    static bool configured = false;   // raise the dynamic LDS limit once per process
    if (!configured) {
      (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&qmm_routed_tile_kernel<kPair>),
                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)routed_tile_lds_bytes(kTileMaxInner));
      configured = true;
    }
    // as many workgroups as are resident at once (LDS and the 2048 threads of a CU decide how
    // many per compute unit) walk the (tile, column block) units
    const uint64_t most_units = (uint64_t)max_blocks * 2 * ((a.columns + 8 * kColsPerWave - 1) / (8 * kColsPerWave));
    const uint32_t per_unit = std::max<uint32_t>(1, std::min<uint32_t>(4, (160u * 1024u) / routed_tile_lds_bytes(a.inner)));
    const uint32_t grid = (uint32_t)std::min<uint64_t>(most_units, (uint64_t)resident * per_unit);
    qmm_routed_tile_kernel<kPair><<<dim3(grid), 512, routed_tile_lds_bytes(a.inner), stream>>>(a);
    return;
  }
  launch_qmm<kPair, true>(stream, a, max_blocks, 1);
}

// Route tile of the K-split kernels: 16 rows while an expert sees few routes on average (an
// expert with more gets a second tile and its weights are read again), else 32; 0 when the
// kernels do not take this K.
uint32_t ksplit_route_tile(const GatherProblem &p, bool pair) {
  if (!ksplit_supports(p.inner, p.columns, pair, true)) return 0;
  return (uint64_t)p.rows * p.k <= 10ull * p.experts ? 16 : 32;
}

bool launch_routed_ksplit(fh_backend *backend, const QmmArgs &a, bool pair, uint32_t max_blocks, uint32_t tile) {
  KsplitRouted r{};
  r.x = a.x;
  r.x_row_stride = a.x_row_stride;
  for (int pj = 0; pj < (pair ? 2 : 1); ++pj) {
    r.packed[pj] = a.packed[pj];
    r.scales[pj] = a.scales[pj];
    r.biases[pj] = a.biases[pj];
  }
  r.pair = pair;
  r.out = a.out;
  r.out_f32 = a.out_f32;
  r.inner = a.inner;
  r.columns = a.columns;
  r.sorted_routes = a.sorted_routes;
  r.blocks = a.blocks;
  r.n_blocks = a.n_blocks;
  r.max_blocks = max_blocks;
  r.tile_rows = tile;
  r.route_div = a.route_div;
  return launch_ksplit_routed(backend, r);
}

bool gather_eligible(const GatherProblem &p, int projections) {
  if (p.x.dtype != FH_BF16) return false;
  for (int pj = 0; pj < projections; ++pj)
    if (!weights_eligible(p.packed[pj], p.scales[pj], p.biases[pj], 3, p.inner, p.bits, p.group))
      return false;
  if ((uint64_t)p.rows * p.k > (1u << 24) || p.experts > 512) return false;
  return true;
}

}  // namespace

bool pack_routes(fh_backend *backend, const GatherProblem &p, uint64_t extra, ErrorSlot *error,
                 PackedRoutes *packed) {
  if ((uint64_t)p.rows * p.k > (1u << 24) || p.experts > 512) return false;
  RoutePlan plan;
  if (!plan_routes(backend, p, extra, error, &plan)) return false;
  packed->sorted_routes = plan.sorted_routes;
  packed->blocks = plan.blocks;
  packed->n_blocks = plan.n_blocks;
  packed->max_blocks = plan.max_blocks;
  packed->tile = kRouteTile;
  packed->rest = plan.rest;
  return true;
}

void launch_combine_routes(hipStream_t stream, const float *partial, const GatherProblem &p,
                           const View *residual) {
  View none{};
  none.base = nullptr;
  const uint64_t work = (uint64_t)p.rows * p.columns;
  combine_routes_kernel<<<dim3((unsigned)((work + 255) / 256)), 256, 0, stream>>>(
      partial, p.indices, p.weights, residual ? *residual : none, residual ? 1 : 0, p.out, p.rows,
      p.k, p.columns, p.experts);
}

namespace {

// The routed products on f32 activations (three bf16 pieces a value, see try_wide_quant_matmul):
// tiles of 16 routes, so only while an expert sees few routes on average -- the decode batches of
// a few lanes the engines run.  `x_rows` input rows of `x_row_stride` elements, `route_div` routes
// per input row; results are f32 rows of `p.columns`.
bool launch_wide_routed(fh_backend *backend, const GatherProblem &p, int projections, const float *x,
                        uint64_t x_row_stride, uint32_t route_div, float *out, const RoutePlan &plan) {
  KsplitRouted r{};
  r.x = x;
  r.x_row_stride = x_row_stride;
  for (int pj = 0; pj < projections; ++pj) {
    r.packed[pj] = u32_ptr(p.packed[pj]);
    r.scales[pj] = u16_ptr(p.scales[pj]);
    r.biases[pj] = u16_ptr(p.biases[pj]);
  }
  r.pair = projections == 2;
  r.out = out;
  r.out_f32 = 1;
  r.inner = p.inner;
  r.columns = p.columns;
  r.sorted_routes = plan.sorted_routes;
  r.blocks = plan.blocks;
  r.n_blocks = plan.n_blocks;
  r.max_blocks = plan.max_blocks;
  r.tile_rows = 16;
  r.route_div = route_div;
  r.wide = true;
  KernelTimer timer(backend, FH_KC_MOE_KERNEL);
  return launch_ksplit_routed(backend, r);
}

bool wide_gather_eligible(const GatherProblem &p, int projections) {
  if (p.x.dtype != FH_F32) return false;
  for (int pj = 0; pj < projections; ++pj)
    if (!weights_eligible(p.packed[pj], p.scales[pj], p.biases[pj], 3, p.inner, p.bits, p.group))
      return false;
  if ((uint64_t)p.rows * p.k > (1u << 24) || p.experts > 512) return false;
  return ksplit_route_tile(p, projections == 2) == 16;
}

bool try_wide_gather_projection(fh_backend *backend, const GatherProblem &p, int projections,
                                bool swiglu, ErrorSlot *error) {
  if (!wide_gather_eligible(p, projections) || (projections == 2 && !swiglu)) return false;
  if (p.out.dtype != FH_F32) return false;
  if (p.x.stride[1] != 1 || p.x.stride[0] % 4 != 0 || p.x.offset % 4 != 0) return false;
  if (p.out.stride[2] != 1 || p.out.stride[1] != p.columns ||
      p.out.stride[0] != (uint64_t)p.k * p.columns)
    return false;
  // rows of bad routes read zero: cleared by the packing kernel as it meets them, or all rows
  // first when an earlier plan is reused (see try_fast_gather_projection)
  RoutePlan plan;
  float *out = (float *)p.out.base + p.out.offset;
  if (!plan_routes(backend, p, 0, error, &plan, (uint32_t *)out, p.columns, 16)) return false;
  if (plan.reused)
    launch_fill_u32(backend_stream(backend), (uint32_t *)out, (uint64_t)p.rows * p.k * p.columns, 0);
  return launch_wide_routed(backend, p, projections, (const float *)p.x.base + p.x.offset, p.x.stride[0],
                            p.k, out, plan);
}

bool try_wide_gather_weighted(fh_backend *backend, const GatherProblem &p, const View *residual,
                              ErrorSlot *error) {
  if (!wide_gather_eligible(p, 1)) return false;
  if (p.x.stride[2] != 1 || p.x.stride[1] % 4 != 0 || p.x.offset % 4 != 0 ||
      p.x.stride[0] != (uint64_t)p.k * p.x.stride[1])
    return false;
  const uint64_t partial_bytes = (uint64_t)p.rows * p.k * p.columns * sizeof(float);
  RoutePlan plan;
  if (!plan_routes(backend, p, partial_bytes, error, &plan, nullptr, 0, 16)) return false;
  float *partial = (float *)plan.rest;
  if (!launch_wide_routed(backend, p, 1, (const float *)p.x.base + p.x.offset, p.x.stride[1], 1, partial,
                          plan))
    return false;
  auto rows_of_eight = [](const View &v) {   // f32 [rows, columns] in 16-byte aligned pieces of 8
    return v.dtype == FH_F32 && v.stride[1] == 1 && v.stride[0] % 8 == 0 && v.offset % 8 == 0;
  };
  if (p.norm_tail && p.norm_tail->wide && p.k <= 8 && p.columns % 8 == 0 && p.columns <= 2048 &&
      rows_of_eight(p.out) && (!residual || rows_of_eight(*residual))) {
    launch_combine_routes_norm(backend_stream(backend), partial, p.indices, p.weights,
                               residual ? (const float *)residual->base + residual->offset : nullptr,
                               residual ? residual->stride[0] : 0, (float *)p.out.base + p.out.offset,
                               p.out.stride[0], p.rows, p.k, p.columns, p.experts, *p.norm_tail);
    *p.norm_tail_taken = true;
    return true;
  }
  launch_combine_routes(backend_stream(backend), partial, p, residual);
  return true;
}

}  // namespace

bool try_fast_gather_projection(fh_backend *backend, const GatherProblem &p, int projections,
                                bool swiglu, ErrorSlot *error) {
  if (p.x.dtype == FH_F32) return try_wide_gather_projection(backend, p, projections, swiglu, error);
  if (!gather_eligible(p, projections)) return false;
  if (projections == 2 && !swiglu) return false;
  if (p.out.dtype != FH_BF16 || ((uint64_t)p.rows * p.k * p.columns) % 2 != 0) return false;
  // x [R,K] rows; out [R,k,N] must be dense so that route r*k+s is row r*k+s of [R*k, N]
  if (p.x.stride[1] != 1 || p.x.stride[0] % 8 != 0 || p.x.offset % 8 != 0) return false;
  if (p.out.stride[2] != 1 || p.out.stride[1] != p.columns ||
      p.out.stride[0] != (uint64_t)p.k * p.columns)
    return false;
  // Rows of bad routes must read zero and bad routes are never packed: the packing kernel clears
  // them as it meets them (a row = `columns` bf16); when the plan is reused instead, nothing
  // packs, and the whole output is cleared first.
  RoutePlan plan;
  const bool row_words = p.columns % 2 == 0 && p.out.offset % 2 == 0;
  const uint32_t ksplit_tile = ksplit_route_tile(p, projections == 2);
  if (!plan_routes(backend, p, 0, error, &plan,
                   row_words ? (uint32_t *)((uint16_t *)p.out.base + p.out.offset) : nullptr,
                   p.columns / 2, ksplit_tile ? ksplit_tile : kRouteTile))
    return false;
  hipStream_t stream = backend_stream(backend);
  if (plan.reused || !row_words)
    launch_fill_u32(stream, (uint32_t *)((uint16_t *)p.out.base + p.out.offset),
                    (uint64_t)p.rows * p.k * p.columns / 2, 0);
  QmmArgs a{};
  a.x = u16_ptr(p.x);
  a.x_row_stride = p.x.stride[0];
  for (int pj = 0; pj < projections; ++pj) {
    a.packed[pj] = u32_ptr(p.packed[pj]);
    a.scales[pj] = u16_ptr(p.scales[pj]);
    a.biases[pj] = u16_ptr(p.biases[pj]);
  }
  a.expert_words = (uint64_t)p.columns * p.inner / 8;
  a.expert_groups = (uint64_t)p.columns * p.inner / kGroup;
  a.out = (uint16_t *)p.out.base + p.out.offset;
  a.out_row_stride = p.columns;
  a.out_f32 = 0;
  a.rows = p.rows * p.k;
  a.inner = p.inner;
  a.columns = p.columns;
  a.sorted_routes = plan.sorted_routes;
  a.blocks = plan.blocks;
  a.n_blocks = plan.n_blocks;
  a.route_div = p.k;
  a.split_below = backend_compute_units(backend) / 2;
  KernelTimer timer(backend, FH_KC_MOE_KERNEL);
  if (ksplit_tile && launch_routed_ksplit(backend, a, projections == 2, plan.max_blocks, ksplit_tile)) return true;
  if (projections == 2)
    launch_routed<true>(stream, a, plan.max_blocks, backend_compute_units(backend));
  else
    launch_routed<false>(stream, a, plan.max_blocks, backend_compute_units(backend));
  return true;
}

bool try_fast_gather_weighted(fh_backend *backend, const GatherProblem &p, const View *residual,
                              ErrorSlot *error) {
  if (p.x.dtype == FH_F32) return try_wide_gather_weighted(backend, p, residual, error);
  if (!gather_eligible(p, 1)) return false;
  // x [R,k,K] dense rows so that route r*k+s is row r*k+s of [R*k, K]
  if (p.x.stride[2] != 1 || p.x.stride[1] % 8 != 0 || p.x.offset % 8 != 0 ||
      p.x.stride[0] != (uint64_t)p.k * p.x.stride[1])
    return false;
  uint64_t partial_bytes = (uint64_t)p.rows * p.k * p.columns * sizeof(float);
  RoutePlan plan;
  const uint32_t ksplit_tile = ksplit_route_tile(p, false);
  if (!plan_routes(backend, p, partial_bytes, error, &plan, nullptr, 0, ksplit_tile ? ksplit_tile : kRouteTile))
    return false;
  hipStream_t stream = backend_stream(backend);
  float *partial = (float *)plan.rest;
  QmmArgs a{};
  a.x = u16_ptr(p.x);
  a.x_row_stride = p.x.stride[1];
  a.packed[0] = u32_ptr(p.packed[0]);
  a.scales[0] = u16_ptr(p.scales[0]);
  a.biases[0] = u16_ptr(p.biases[0]);
  a.expert_words = (uint64_t)p.columns * p.inner / 8;
  a.expert_groups = (uint64_t)p.columns * p.inner / kGroup;
  a.out = partial;
  a.out_row_stride = p.columns;
  a.out_f32 = 1;
  a.rows = p.rows * p.k;
  a.inner = p.inner;
  a.columns = p.columns;
  a.sorted_routes = plan.sorted_routes;
  a.blocks = plan.blocks;
  a.n_blocks = plan.n_blocks;
  a.route_div = 1;
  a.split_below = backend_compute_units(backend) / 2;
  {
    KernelTimer timer(backend, FH_KC_MOE_KERNEL);
    if (!(ksplit_tile && launch_routed_ksplit(backend, a, false, plan.max_blocks, ksplit_tile)))
      launch_routed<false>(stream, a, plan.max_blocks, backend_compute_units(backend));
  }
  uint64_t work = (uint64_t)p.rows * p.columns;
  auto row_view = [&](const View &v) {   // bf16 [rows, columns], 8-byte aligned row pieces
    return v.dtype == FH_BF16 && v.stride[1] == 1 && v.stride[0] % 4 == 0 && v.offset % 4 == 0;
  };
  if (p.columns % 4 == 0 && p.k <= 16 && row_view(p.out) && (!residual || row_view(*residual))) {
    const uint16_t *res = residual ? (const uint16_t *)residual->base + residual->offset : nullptr;
    const uint64_t res_stride = residual ? residual->stride[0] : 0;
    uint16_t *out = (uint16_t *)p.out.base + p.out.offset;
    if (p.norm_tail && !p.norm_tail->wide && p.k <= 8 && p.columns % 8 == 0 && p.columns <= 2048 && p.out.stride[0] % 8 == 0 &&
        p.out.offset % 8 == 0 && (!residual || (residual->stride[0] % 8 == 0 && residual->offset % 8 == 0))) {
      launch_combine_routes_norm(stream, partial, p.indices, p.weights, res, res_stride, out,
                                 p.out.stride[0], p.rows, p.k, p.columns, p.experts, *p.norm_tail);
      *p.norm_tail_taken = true;
      return true;
    }
    const dim3 grid((unsigned)((work / 4 + 255) / 256));
    if (p.k <= 8)
      combine_routes_rows_kernel<8><<<grid, 256, 0, stream>>>(partial, p.indices, p.weights, res, res_stride,
                                                             out, p.out.stride[0], p.rows, p.k,
                                                             p.columns, p.experts);
    else
      combine_routes_rows_kernel<16><<<grid, 256, 0, stream>>>(partial, p.indices, p.weights, res, res_stride,
                                                              out, p.out.stride[0], p.rows, p.k,
                                                              p.columns, p.experts);
    return true;
  }
  View none{};
  none.base = nullptr;
  combine_routes_kernel<<<dim3((unsigned)((work + 255) / 256)), 256, 0, stream>>>(
      partial, p.indices, p.weights, residual ? *residual : none, residual ? 1 : 0, p.out, p.rows,
      p.k, p.columns, p.experts);
  return true;
}

namespace {

// Canonical expression string of value `v`: commutative operands are sorted so that equivalent
// instruction orders compare equal.
std::string canonical(const std::vector<fh_inst> &insts, uint32_t v, int depth = 0) {
  if (v >= insts.size() || depth > 16) return "?";
  const fh_inst &inst = insts[v];
  switch (inst.kind) {
  case 0: return "in" + std::to_string(inst.a);
  case 1: return "c" + std::to_string(inst.a);
  case 4: return "u" + std::to_string(inst.op) + "(" + canonical(insts, inst.a, depth + 1) + ")";
  case 5: {
    std::string l = canonical(insts, inst.a, depth + 1), r = canonical(insts, inst.b, depth + 1);
    if ((inst.op == 0 || inst.op == 2) && r < l) std::swap(l, r);
    return "b" + std::to_string(inst.op) + "(" + l + "," + r + ")";
  }
  default: return "?";
  }
}

}  // namespace

bool is_add_epilogue(const std::vector<fh_inst> &insts, const std::vector<uint32_t> &pairs) {
  if (pairs.size() != 2 || pairs[0] != 0) return false;
  return canonical(insts, pairs[1]) == "b0(in0,in1)";
}

bool is_swiglu_epilogue(const std::vector<fh_inst> &insts, const std::vector<uint32_t> &pairs) {
  if (pairs.size() != 2 || pairs[0] != 0) return false;
  std::string e = canonical(insts, pairs[1]);
  // gate * sigmoid(gate) * up, in any association
  return e == "b2(b2(in0,u9(in0)),in1)" || e == "b2(in1,b2(in0,u9(in0)))" ||
         e == "b2(in0,b2(in1,u9(in0)))" || e == "b2(b2(in0,in1),u9(in0))" ||
         e == "b2(u9(in0),b2(in0,in1))" || e == "b2(b2(in1,u9(in0)),in0)";
}

}  // namespace fh
