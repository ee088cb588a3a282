// MLX-4bit affine quantised products over few activation rows: the wave-reduced GEMV of decode
// batches (dense, at most 32 rows) and the routed products of a decode-sized MoE block (route
// tiles of at most 32 rows per expert).  Same arithmetic as qmm_fast.hip:
//   y[m,n] = sum_k x[m,k] * (scale[n,k/64] * q[n,k] + bias[n,k/64])      (affine_quant_dot,
//   crates/forja-cpu/src/lib.rs:1277-1310), q = nibble k%8 of word k/8, low nibble first;
// a nibble becomes the bf16 value 16+q, a 64-value group is contracted exactly in f32 on the
// matrix cores, and scale and (bias - 16 scale) * sum(x) are applied per group.
//
// The work is HBM-bound on the packed weights and every weight is used for one 16- or 32-row
// tile only, so the activations are the stationary operand: the waves of a workgroup split K
// between them, each wave keeps ITS K slice of the tile's rows in registers (64 values per group
// and row as two v_mfma_f32_16x16x32_bf16 A operands), loaded straight from memory in operand
// layout, and streams the matching K slice of every weight row the workgroup owns.  Lane (column
// n, quarter g) reads 16 bytes (half of one group, a quarter of a pair of groups) at a time, so a
// wave's load covers 64 contiguous bytes of 16 weight rows: the narrowest access that still
// reaches the read rate of a plain stream on this device (8-byte pieces stay 20 % below it).  Two
// half-wave swaps (v_permlane32_swap) then sort the words by group.  Nothing is staged through
// LDS and no barrier separates loading from computing; the waves' partial sums of a batch of
// columns meet in LDS once per batch (one barrier, double buffered) and the waves share the
// epilogue.
//
// What the instruction stream must not do, because it empties the ring of weight batches in
// flight (each was measured): wait on a vector load that is younger than the ring (table words
// are read as scalars; row ids are claimed where they are loaded), issue ring loads under a
// branch, or leave the loop body through an exit that rejoins it -- the wait-count pass then
// assumes the path with the fewest loads in flight and waits for all of them.
//
// Work units are (tile, batch of columns); a launch has as many workgroups as stay resident and
// workgroup w takes the contiguous units [w U / W, (w+1) U / W): every workgroup streams the same
// number of weight bytes to within one batch, whatever the number of tiles turns out to be on the
// device.
#include "fast_kernels.hpp"

namespace fh {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kGroup = 64;
constexpr uint32_t kNoBlock = 0xffffffffu;

struct KsplitArgs {
  const void *x;            // bf16 (or, in the three-piece form, f32) activations, innermost axis contiguous
  uint64_t x_row_stride;    // elements between input rows
  const uint32_t *packed[2];
  const uint16_t *scales[2], *biases[2];
  uint64_t expert_words;    // u32 words per expert matrix (N*K/8); 0 for dense
  uint64_t expert_groups;   // scale entries per expert matrix (N*K/64)
  void *out;                // bf16 or f32
  uint64_t out_row_stride;  // elements
  uint32_t out_f32;
  const void *residual;     // dense only: optional rows (of the activations' dtype) added before the result is rounded
  uint64_t residual_row_stride;
  uint32_t rows, inner, columns;
  uint32_t weight_inner;    // K of the weight matrix: the length of its rows (>= inner)
  // routed form: tiles (expert, first, count) over sorted_routes; input row = route / route_div
  const uint32_t *sorted_routes, *blocks, *n_blocks;
  uint32_t route_div;
  uint32_t batches_per_tile;
};

// A word the whole wave reads from a table no kernel writes while this one runs (the route plan):
// read through the constant address space it becomes a scalar load, which is waited for on its own
// counter.  As a vector load it would have to be waited for with vmcnt(0), i.e. together with every
// batch of weights still in flight.
__device__ inline uint32_t table_word(const uint32_t *table, uint32_t index) {
  typedef const __attribute__((address_space(4))) uint32_t *constant_words;
  return ((constant_words)(uintptr_t)table)[index];
}

__device__ inline uint32_t pack_bf16_pair(float lo, float hi) {
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ inline float bf16_bits(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// (x & mask) | magic: one v_and_or_b32 when neither constant is a literal (see unpack_word).
__device__ inline uint32_t and_or(uint32_t x, uint32_t mask, uint32_t magic) {
  return (x & mask) | magic;
}

// Eight nibbles of `w` as bf16 (16+q) in slot order (0,4)(1,5)(2,6)(3,7).
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

// The same slot order for eight consecutive activations.
__device__ inline uint4 permute_slots(const uint4 &v) {
  uint4 p;
  p.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (x0, x4)
  p.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (x1, x5)
  p.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (x2, x6)
  p.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (x3, x7)
  return p;
}

__device__ inline float sum8(const uint4 &v) {
  return bf16_bits(v.x & 0xffffu) + bf16_bits(v.x >> 16) + bf16_bits(v.y & 0xffffu) +
         bf16_bits(v.y >> 16) + bf16_bits(v.z & 0xffffu) + bf16_bits(v.z >> 16) +
         bf16_bits(v.w & 0xffffu) + bf16_bits(v.w >> 16);
}

// Element `index` (a per-lane value, 0..2*kWords-1) of bf16 values packed two to a word, as f32;
// 0 beyond the words.
template <int kWords>
__device__ inline float packed_bf16_at(const uint32_t (&words)[kWords], uint32_t index) {
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < kWords; ++i)
    if ((index >> 1) == (uint32_t)i) word = words[i];
  return __uint_as_float((index & 1u) ? (word & 0xffff0000u) : (word << 16));
}

// WAVES waves split K; G = quantisation groups per wave (K = 64 * G * WAVES, G even);
// RT = 16-row tiles of activations (the rows a weight is used for: 16 or 32).
// 16-column tiles per batch and projection: a batch is 4 KiB of weights per wave (two
// tile-projections of a four-group K slice, four of a two-group one), so that two batches fit
// the registers beside the stationary rows.
constexpr int batch_tiles(bool pair, int groups) { return (groups <= 2 ? 2 : 1) * (pair ? 1 : 2); }

// Batches of weights a wave keeps requested ahead of its arithmetic: two, and three where the
// stationary rows of a 32-row routed tile of a four-group K slice leave room for a single
// workgroup per compute unit, whose eight waves alone must keep that unit's share of HBM busy.
constexpr int ring_slots(int row_tiles, int groups, bool routed) { return row_tiles == 2 && groups > 2 && routed ? 3 : 2; }

typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

// Waves per SIMD the registers must leave room for: two workgroups per compute unit where the
// stationary rows are few (one contracts while the other waits at its exchange barrier).
constexpr int resident_waves(int waves, int row_tiles, int groups, bool routed, int pieces) {
  const bool two = pieces > 1 ? false : row_tiles == 1 ? groups <= 4 : groups <= 2 && waves <= 6 && routed;
  return two ? (2 * waves + 3) / 4 : (waves + 3) / 4;
}

// XP = bf16 pieces an activation is held in: 1 for bf16 rows; 3 for f32 rows, each value split
// exactly into the bf16 numbers of its high, middle and low eight significant bits, so that the
// three products with a weight operand (exact 16+q in bf16) add up, in the f32 accumulator, to
// the product with the f32 value itself.  The stationary rows then take three times the
// registers: one 16-row tile, one workgroup per compute unit.
template <int WAVES, int G, int RT, bool kPair, bool kRouted, int XP>
__global__ __launch_bounds__(64 * WAVES, resident_waves(WAVES, RT, G, kRouted, XP)) void qmm_ksplit_kernel(KsplitArgs a) {
  static_assert(XP == 1 || (XP == 3 && RT == 1), "f32 rows: one row tile");
  constexpr int P = kPair ? 2 : 1;
  constexpr int NS = ring_slots(RT, G, kRouted);
  constexpr int CT = batch_tiles(kPair, G);
  constexpr int kBatchCols = 16 * CT;
  constexpr int Q = (G + 3) / 4;             // f32 matrix steps of the bias term (4 groups each)
  constexpr int W2 = G / 2;                  // words of a lane's scales (or biases) of a column
  constexpr int kSlots = P * CT * RT;        // 16 x 16 accumulator blocks of a wave and batch
  constexpr int kQuads = CT * RT;            // blocks of results of a batch (both projections of a pair)
  constexpr int QPW = (kQuads + WAVES - 1) / WAVES;     // blocks a wave finishes per batch
  // With fewer blocks than waves the epilogue is dealt row by row instead (four times as many
  // pieces), so that every wave takes part in it.
  constexpr bool kWide = kQuads >= WAVES / 2;
  constexpr int kTriples = kQuads * 4;       // (column tile, row tile, row) triples of a batch
  constexpr int TPW = (kTriples + WAVES - 1) / WAVES;
  constexpr int kShare = kWide ? QPW * 4 : TPW;         // results per lane this wave finishes per batch
  // Scales and biases of a batch: kSub blocks of 16 columns x K/64 bf16 (each projection and
  // column tile, scales then biases), contiguous in memory.  A wave needs 2G bytes of each column
  // row; read directly, those 8-byte pieces of 64-byte sectors cost a quarter of the weight
  // bandwidth (measured).  So the workgroup reads each block once, coalesced -- a thread fetches
  // kShareWords words of every batch -- and passes it through LDS, two batches deep: written
  // before the exchange barrier of the batch before, read at the start of its own batch.
  // (Only where the memory requests bound the kernel: with two row tiles the instruction stream
  // does, and the direct loads, which cost no extra instructions, stay.)
  constexpr bool kStage = RT == 1;
  constexpr int kSub = P * CT * 2;
  constexpr int kPieces = kSub * 16 * WAVES;          // 2G-byte pieces of a batch (one per column and wave)
  constexpr int PT = kPieces / (64 * WAVES);          // pieces a thread fetches per batch (1 or 2)
  static_assert(PT * 64 * WAVES == kPieces, "whole pieces per thread");
  extern __shared__ __attribute__((aligned(16))) float exchange[];   // f32x4 [2][WAVES][kSlots][64]
  uint32_t *scale_lds = (uint32_t *)(exchange + 2 * WAVES * kSlots * 4 * 64);   // [2][kPieces][W2]
  const uint32_t lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // a weight row may be longer than the K this launch contracts (one of several K ranges)
  const uint32_t words_per_row = a.weight_inner / 8, groups_per_row = a.weight_inner / kGroup;
  const uint32_t tiles = kRouted ? table_word(a.n_blocks, 0) : (a.rows + 16 * RT - 1) / (16 * RT);
  const uint32_t units = tiles * a.batches_per_tile;
  const uint32_t first_unit = (uint32_t)((uint64_t)blockIdx.x * units / gridDim.x);
  const uint32_t last_unit = (uint32_t)((uint64_t)(blockIdx.x + 1) * units / gridDim.x);

  // ---- the stationary operand: this wave's K slice of the current tile's rows.
  // A lane reads 16 weight bytes (half a group) at a time, so that a wave's load covers 64
  // contiguous bytes of each of 16 weight rows; two half-wave swaps then leave the lane quarters
  // g = 0..3 holding words (0,4,2,6) and (1,5,3,7) of ONE group, and the activations are laid out
  // to match: quarter g holds the group's values [16 g', 16 g' + 16), g' = (0,2,1,3)[g].
  uint4 xa[XP][RT][G][2];  // A operands: [piece][row tile][group][half of the lane's 16 values]
  float xs[RT][Q];         // sum of the row's activations over group 4q + g (bias term operand)
  uint32_t out_rows[RT][4]; // output row of accumulator (row tile, i): tile row 16 rt + 4 g + i
  uint32_t tile_first = 0, tile_count = 0, current_tile = kNoBlock;
  const uint32_t g_perm = 2 * (g & 1) + (g >> 1);
  auto load_tile = [&](uint32_t tile) {
    current_tile = tile;
    if (kRouted) {
      const uint32_t expert = table_word(a.blocks, 3 * tile);
      tile_first = expert == kNoBlock ? 0 : table_word(a.blocks, 3 * tile + 1);
      tile_count = expert == kNoBlock ? 0 : table_word(a.blocks, 3 * tile + 2);
    } else {   // dense: row tile `tile` of the activation matrix
      tile_first = tile * (16 * RT);
      tile_count = min((uint32_t)(16 * RT), a.rows - tile_first);
    }
    // the rows this lane's accumulators belong to: fetched with the tile, not when a batch ends.
    // Rows past the tile's count read the tile's first row (or row 0): their products are
    // computed and never stored, which keeps this code free of branches.
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t row = 16 * rt + 4 * g + i;
        const uint32_t at = tile_first + (row < tile_count ? row : 0);
        out_rows[rt][i] = kRouted ? a.sorted_routes[at] : at;
      }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const uint32_t row = 16 * rt + n;
      const uint32_t safe = row < tile_count ? row : 0;
      const uint64_t in_row = kRouted ? a.sorted_routes[tile_first + safe] / a.route_div : tile_first + safe;
      const uint64_t x_at = in_row * a.x_row_stride + (uint64_t)wave * (G * kGroup) + 16 * g_perm;
      float sums[G];
#pragma unroll
      for (int j = 0; j < G; ++j) {
        float s;
        if constexpr (XP == 1) {
          const uint16_t *xp = (const uint16_t *)a.x + x_at;
          const uint4 lo = *(const uint4 *)(xp + kGroup * j), hi = *(const uint4 *)(xp + kGroup * j + 8);
          s = sum8(lo) + sum8(hi);
          xa[0][rt][j][0] = permute_slots(lo);
          xa[0][rt][j][1] = permute_slots(hi);
        } else {
          const float *xp = (const float *)a.x + x_at + kGroup * j;
          float value[16];
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const float4 four = *(const float4 *)(xp + 4 * v);
            value[4 * v] = four.x, value[4 * v + 1] = four.y, value[4 * v + 2] = four.z, value[4 * v + 3] = four.w;
          }
          s = 0.0f;
#pragma unroll
          for (int v = 0; v < 16; ++v) s += value[v];
          // piece 0 = low bits ... piece 2 = high bits: the small products are added first
#pragma unroll
          for (int piece = XP - 1; piece >= 0; --piece) {
            uint32_t top[16];   // the piece's bf16 bits in the upper half of a word
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              top[v] = __float_as_uint(value[v]) & 0xffff0000u;
              value[v] -= __uint_as_float(top[v]);   // exact: what the lower pieces hold
            }
#pragma unroll
            for (int half = 0; half < 2; ++half) {
              uint4 packed;   // eight consecutive values, two to a word, as bf16 rows hold them
              packed.x = __builtin_amdgcn_perm(top[8 * half + 1], top[8 * half + 0], 0x07060302u);
              packed.y = __builtin_amdgcn_perm(top[8 * half + 3], top[8 * half + 2], 0x07060302u);
              packed.z = __builtin_amdgcn_perm(top[8 * half + 5], top[8 * half + 4], 0x07060302u);
              packed.w = __builtin_amdgcn_perm(top[8 * half + 7], top[8 * half + 6], 0x07060302u);
              xa[piece][rt][j][half] = permute_slots(packed);
            }
          }
        }
        s += __shfl_xor(s, 16, 64);      // the four quarters of the group
        s += __shfl_xor(s, 32, 64);
        sums[j] = s;
      }
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        float mine = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (4 * q + i < G && g == (uint32_t)i) mine = sums[4 * q + i];
        xs[rt][q] = mine;
      }
      __builtin_amdgcn_sched_barrier(0);   // one row tile's loads in flight at a time (registers)
    }
    // The row ids are used when a batch ends; claim them here, so that the wait for them stands in
    // this (rare) path and not, as a wait for everything in flight, at the end of every batch.
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(out_rows[rt][i]));
  };

  // ---- the streamed operand: one batch of columns, this wave's K slice.  Every load is issued
  // unconditionally (addresses are clamped instead) so that the hardware counter a wave waits on
  // before it touches a batch counts exactly the younger batches still in flight.
  struct Batch {
    uint4 w[P][CT][W2];         // the lane's 32 nibbles of each pair of groups
    uint32_t s[P][CT][W2], b[P][CT][W2];   // direct form only: the column's G scales and biases, two to a word
    uint32_t residual[kShare];  // dense only: the values added to this wave's share of the results
  };
  // Where a stream of units stands: the loads run a ring ahead of the arithmetic, each with its own
  // cursor, advanced without divisions; the expert of a tile is read when the cursor enters it.
  struct Cursor {
    uint32_t unit, tile, batch, expert;
  };
  auto expert_of = [&](uint32_t tile) -> uint32_t {
    if (!kRouted) return 0;
    const uint32_t expert = table_word(a.blocks, 3 * tile);
    return expert == kNoBlock ? 0 : expert;
  };
  auto advance = [&](Cursor &c) {
    if (c.unit + 1 >= last_unit) return;     // the loads past the end repeat the last unit
    ++c.unit;
    if (++c.batch == a.batches_per_tile) {
      c.batch = 0;
      ++c.tile;
      c.expert = expert_of(c.tile);
    }
  };
  // Byte offsets of this lane inside a 16-column tile of one expert matrix: the rest of an address
  // is the same for the whole wave and stays in scalar registers.
  const uint32_t lane_weight_bytes = (n * words_per_row + wave * (G * 8) + 4 * g) * 4;
  const uint32_t lane_group_bytes = (n * groups_per_row + wave * G) * 2;
  // This thread's share of a batch's scales and biases: piece threadIdx.x + i * threads of the
  // kPieces, i.e. block piece / (16 WAVES), and inside the block (contiguous in memory and in
  // LDS alike) piece % (16 WAVES).  The part of the address that does not change is kept.
  struct Share {
    uint32_t words[PT][W2];
  };
  const uint16_t *share_from[PT];
#pragma unroll
  for (int i = 0; i < PT; ++i) {
    const uint32_t piece = threadIdx.x + i * (64 * WAVES);
    const uint32_t block = piece / (16 * WAVES), inside = piece % (16 * WAVES);
    const uint16_t *from = a.scales[0];
#pragma unroll
    for (int sub = 0; sub < kSub; ++sub) {
      const int tp = sub / 2, pj = tp / CT, ct = tp % CT;
      const uint16_t *base = (sub % 2 ? a.biases[pj] : a.scales[pj]) + (uint64_t)(16 * ct) * groups_per_row;
      if (block == (uint32_t)sub) from = base;
    }
    share_from[i] = from + (uint64_t)(inside / WAVES) * groups_per_row + (inside % WAVES) * G;
  }
  auto load_share = [&](Share &r, const Cursor &c) {
    if constexpr (!kStage) return;
    const uint64_t groups = c.expert * a.expert_groups + (uint64_t)c.batch * kBatchCols * groups_per_row;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const uint32_t *from = (const uint32_t *)(share_from[i] + groups);
#pragma unroll
      for (int k = 0; k < W2; ++k) r.words[i][k] = from[k];
    }
  };
  auto write_share = [&](const Share &r, uint32_t half) {
    if constexpr (!kStage) return;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      uint32_t *to = scale_lds + ((uint64_t)half * kPieces + threadIdx.x + i * (64 * WAVES)) * W2;
#pragma unroll
      for (int k = 0; k < W2; ++k) to[k] = r.words[i][k];
    }
  };
  // The value added to result (row, column), as the bits of its dtype (any readable word when
  // there is no residual: the load is unconditional).
  auto residual_at = [&](uint32_t row, uint32_t column) -> uint32_t {
    const uint64_t at = (uint64_t)row * a.residual_row_stride + column;
    if constexpr (XP == 1) return *(a.residual ? (const uint16_t *)a.residual + at : (const uint16_t *)a.x);
    return *(a.residual ? (const uint32_t *)a.residual + at : (const uint32_t *)a.x);
  };
  auto load_batch = [&](Batch &r, const Cursor &c) {
    const uint32_t batch = c.batch;
#pragma unroll
    for (int pj = 0; pj < P; ++pj)
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const uint64_t tile_column = batch * kBatchCols + 16 * ct;   // a multiple of 16 below a.columns
        const uint64_t words = c.expert * a.expert_words + tile_column * words_per_row;
        const char *wp = (const char *)(a.packed[pj] + words) + lane_weight_bytes;
#pragma unroll
        for (int k = 0; k < W2; ++k) r.w[pj][ct][k] = *(const uint4 *)(wp + 64 * k);
        if constexpr (!kStage) {
          const uint64_t groups = c.expert * a.expert_groups + tile_column * groups_per_row;
          const char *sp = (const char *)(a.scales[pj] + groups) + lane_group_bytes;
          const char *bp = (const char *)(a.biases[pj] + groups) + lane_group_bytes;
#pragma unroll
          for (int i = 0; i < W2; ++i) {
            r.s[pj][ct][i] = *(const uint32_t *)(sp + 4 * i);
            r.b[pj][ct][i] = *(const uint32_t *)(bp + 4 * i);
          }
        }
      }
    if (!kRouted) {
      if constexpr (kWide) {
#pragma unroll
        for (int qq = 0; qq < QPW; ++qq) {
          const uint32_t quad = wave + qq * WAVES;
          if (quad >= (uint32_t)kQuads) break;     // uniform: waves that finish no block load nothing
          const uint32_t ct = quad / RT, rt = quad % RT;
          const uint32_t column = min(batch * kBatchCols + 16 * ct + n, a.columns - 1);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const uint32_t row = min(c.tile * (16 * RT) + 16 * rt + 4 * g + i, a.rows - 1);
            r.residual[4 * qq + i] = residual_at(row, column);
          }
        }
      } else {
#pragma unroll
        for (int tt = 0; tt < TPW; ++tt) {
          const uint32_t t = min(wave + tt * WAVES, (uint32_t)kTriples - 1);
          const uint32_t ct = t / (RT * 4), rt = (t / 4) % RT, i = t % 4;
          const uint32_t row = min(c.tile * (16 * RT) + 16 * rt + 4 * g + i, a.rows - 1);
          const uint32_t column = min(batch * kBatchCols + 16 * ct + n, a.columns - 1);
          r.residual[tt] = residual_at(row, column);
        }
      }
    }
  };

  // Contracts the batch against the stationary rows, hands the partial sums to LDS buffer `buf`,
  // and takes this wave's share of the epilogue.
  // ... `pass_on` is this thread's share of the NEXT batch's scales and biases, written to the other
  // half of their LDS ring before the barrier; this batch's are read from half `buf` first.
  auto finish_batch = [&](const Batch &r, const Share &pass_on, uint32_t batch, uint32_t buf) {
    uint32_t scales[P * CT][W2], biases[P * CT][W2];
#pragma unroll
    for (int tp = 0; tp < P * CT; ++tp) {
      const uint32_t *at = scale_lds + ((uint64_t)buf * kPieces + (2 * tp) * (16 * WAVES) + n * WAVES + wave) * W2;
#pragma unroll
      for (int k = 0; k < W2; ++k) {
        scales[tp][k] = kStage ? at[k] : r.s[tp / CT][tp % CT][k];
        biases[tp][k] = kStage ? at[(16 * WAVES) * W2 + k] : r.b[tp / CT][tp % CT][k];
      }
    }
    f32x4 acc[P * CT][RT];
    // bias term sum_j (bias_j - 16 scale_j) * xsum_j[row] first: an f32 matrix step over four
    // groups, lane quarter g supplying group 4q + g of both operands
#pragma unroll
    for (int tp = 0; tp < P * CT; ++tp) {
      const int pj = tp / CT, ct = tp % CT;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) acc[tp][rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        const float shift = packed_bf16_at<W2>(biases[tp], 4 * q + g) -
                            16.0f * packed_bf16_at<W2>(scales[tp], 4 * q + g);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[tp][rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(xs[rt][q], shift, acc[tp][rt], 0, 0, 0);
      }
    }
    // the groups: each group's exact f32 sum is scaled into the accumulators one group late, so
    // that the matrix unit's result is not waited for
    f32x4 late[RT];
    float late_scale = 0.0f;
    u32x2 first_words = {0, 0}, second_words = {0, 0};
#pragma unroll
    for (int s = 0; s < P * CT * G; ++s) {
      const int tp = s / G, j = s % G, pj = tp / CT, ct = tp % CT;
      if (j % 2 == 0) {
        const uint4 w = r.w[pj][ct][j / 2];
        first_words = __builtin_amdgcn_permlane32_swap(w.x, w.z, false, false);
        second_words = __builtin_amdgcn_permlane32_swap(w.y, w.w, false, false);
      }
      const bf16x8 b0 = unpack_word(first_words[j % 2]), b1 = unpack_word(second_words[j % 2]);
      const uint32_t word = scales[tp][j / 2];
      const float scale = __uint_as_float((j & 1) ? (word & 0xffff0000u) : (word << 16));
      f32x4 part[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        part[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int piece = 0; piece < XP; ++piece) {
          part[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[piece][rt][j][0]), b0, part[rt], 0, 0, 0);
          part[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[piece][rt][j][1]), b1, part[rt], 0, 0, 0);
        }
      }
      if (s > 0) {
        const int before = (s - 1) / G;
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[before][rt][i] = __builtin_fmaf(late_scale, late[rt][i], acc[before][rt][i]);
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) late[rt] = part[rt];
      late_scale = scale;
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[P * CT - 1][rt][i] = __builtin_fmaf(late_scale, late[rt][i], acc[P * CT - 1][rt][i]);
    // One result: activation of a pair, residual of a dense product, rounding, store.
    auto store_result = [&](float value, float up, uint32_t out_row, uint32_t column, uint32_t residual_bits) {
      if (kPair) value = value * (1.0f / (1.0f + __expf(-value))) * up;
      if (!kRouted && a.residual) value += XP == 1 ? bf16_bits(residual_bits & 0xffffu) : __uint_as_float(residual_bits);
      const uint64_t at = (uint64_t)out_row * a.out_row_stride + column;
      if (a.out_f32)
        ((float *)a.out)[at] = value;
      else
        ((uint16_t *)a.out)[at] = (uint16_t)(pack_bf16_pair(value, 0.0f) & 0xffffu);
    };
    if constexpr (kWide) {
      f32x4 *mine = (f32x4 *)exchange + ((uint64_t)(buf * WAVES + wave) * kSlots) * 64 + lane;
#pragma unroll
      for (int tp = 0; tp < P * CT; ++tp)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) mine[(tp * RT + rt) * 64] = acc[tp][rt];
      write_share(pass_on, buf ^ 1u);
      __syncthreads();
      // (column tile, row tile) blocks of 16 x 16 results are dealt round-robin to the waves; the
      // owner adds the waves' sums in wave order (fixed: results do not depend on scheduling), four
      // rows of a column to a lane
#pragma unroll
      for (int qq = 0; qq < QPW; ++qq) {
        const int quad = (int)wave + qq * WAVES;
        if (quad >= kQuads) break;
        const int ct = quad / RT, rt = quad % RT;
        f32x4 total[P];
#pragma unroll
        for (int pj = 0; pj < P; ++pj) {
          const f32x4 *from = (const f32x4 *)exchange + ((uint64_t)(buf * WAVES) * kSlots + ((pj * CT + ct) * RT + rt)) * 64 + lane;
          total[pj] = from[0];
#pragma unroll
          for (int v = 1; v < WAVES; ++v) total[pj] += from[(uint64_t)v * kSlots * 64];
        }
        const uint32_t column = batch * kBatchCols + 16 * ct + n;
        if (column >= a.columns) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (16 * rt + 4 * g + i >= tile_count) continue;
          uint32_t out_row = out_rows[0][i];
#pragma unroll
          for (int r2 = 1; r2 < RT; ++r2)
            if (r2 == rt) out_row = out_rows[r2][i];
          store_result(total[0][i], total[P - 1][i], out_row, column, kRouted ? 0 : r.residual[4 * qq + i]);
        }
      }
    } else {
      float *mine = exchange + ((uint64_t)(buf * WAVES + wave) * kSlots * 4) * 64 + lane;
#pragma unroll
      for (int tp = 0; tp < P * CT; ++tp)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
#pragma unroll
          for (int i = 0; i < 4; ++i) mine[((tp * RT + rt) * 4 + i) * 64] = acc[tp][rt][i];
      write_share(pass_on, buf ^ 1u);
      __syncthreads();
      // (column tile, row tile, row) triples are dealt round-robin to the waves, one result to a lane
#pragma unroll
      for (int tt = 0; tt < TPW; ++tt) {
        const int t = (int)wave + tt * WAVES;
        if (t >= kTriples) break;
        const int ct = t / (RT * 4), rt = (t / 4) % RT, i = t % 4;
        float total[P];
#pragma unroll
        for (int pj = 0; pj < P; ++pj) {
          const float *from = exchange + ((uint64_t)(buf * WAVES) * kSlots * 4 + (((pj * CT + ct) * RT + rt) * 4 + i)) * 64 + lane;
          total[pj] = from[0];
#pragma unroll
          for (int v = 1; v < WAVES; ++v) total[pj] += from[(uint64_t)v * kSlots * 4 * 64];
        }
        const uint32_t row = 16 * rt + 4 * g + i, column = batch * kBatchCols + 16 * ct + n;
        if (row >= tile_count || column >= a.columns) continue;
        uint32_t out_row = 0;   // out_rows[rt][i], picked without indexing registers dynamically
#pragma unroll
        for (int r2 = 0; r2 < RT; ++r2)
#pragma unroll
          for (int i2 = 0; i2 < 4; ++i2)
            if (r2 == rt && i2 == i) out_row = out_rows[r2][i2];
        store_result(total[0], total[P - 1], out_row, column, kRouted ? 0 : r.residual[tt]);
      }
    }
  };

  if (first_unit >= last_unit) return;
  Cursor loading{first_unit, first_unit / a.batches_per_tile, first_unit % a.batches_per_tile, 0};
  loading.expert = expert_of(loading.tile);
  Cursor computing = loading, sharing = loading;
  // Scales and biases run one batch further ahead than the weights: the share of the first unit
  // goes to LDS at once, those of the next two are in flight when the loop starts.
  Share shares[NS], first_share;
  load_share(first_share, sharing);
  advance(sharing);
#pragma unroll
  for (int slot = 1; slot <= 2; ++slot) {
    load_share(shares[slot % NS], sharing);
    advance(sharing);
  }
  Batch ring[NS];
#pragma unroll
  for (int slot = 0; slot < NS; ++slot) {
    load_batch(ring[slot], loading);
    advance(loading);
  }
  write_share(first_share, 0);
  if (kStage) __syncthreads();   // the first unit's scales are in LDS
  // Whole rounds of the ring first, in a loop without exits in its body (an exit that rejoins the
  // loop would make every wait assume the shortest path, i.e. drain the ring); the last, partial
  // round is a copy of the body that requests nothing.  Unit number i of this workgroup uses ring
  // slot i % NS; share i + 1 is passed on while unit i is finished, share i + 3 requested after it.
  uint32_t base = first_unit, buf = 0;
  for (; base + NS <= last_unit; base += NS) {
#pragma unroll
    for (int slot = 0; slot < NS; ++slot) {
      if (computing.tile != current_tile) load_tile(computing.tile);
      finish_batch(ring[slot], shares[(slot + 1) % NS], computing.batch, buf);
      buf ^= 1u;
      load_share(shares[(slot + 3) % NS], sharing);
      load_batch(ring[slot], loading);
      advance(sharing);
      advance(loading);
      advance(computing);
    }
  }
#pragma unroll
  for (int slot = 0; slot < NS - 1; ++slot) {
    if (base + slot >= last_unit) break;
    if (computing.tile != current_tile) load_tile(computing.tile);
    finish_batch(ring[slot], shares[(slot + 1) % NS], computing.batch, buf);
    buf ^= 1u;
    advance(computing);
  }
}

// How K is split: waves and groups per wave; false when this K has no instantiation.
bool ksplit_shape(uint32_t inner, int *waves, int *groups) {
  switch (inner) {
  case 512: *waves = 4, *groups = 2; return true;
  case 768: *waves = 6, *groups = 2; return true;
  case 1024: *waves = 8, *groups = 2; return true;
  case 1536: *waves = 6, *groups = 4; return true;
  case 2048: *waves = 8, *groups = 4; return true;
  case 3072: *waves = 8, *groups = 6; return true;
  case 4096: *waves = 8, *groups = 8; return true;
  default: return false;
  }
}

// One launch: as many workgroups as stay resident at once (the runtime's own occupancy figure for
// this instantiation), never more than there are units of work.
template <int WAVES, int G, int RT, bool kPair, bool kRouted, int XP>
void launch_one(fh_backend *backend, const KsplitArgs &a, uint64_t most_units) {
  constexpr int P = kPair ? 2 : 1, CT = batch_tiles(kPair, G);
  constexpr uint32_t lds = 2u * WAVES * (CT * P * RT * 4) * 64 * sizeof(float) +   // partial sums
                           (RT == 1 ? 2u * (P * CT * 2 * 16 * WAVES) * (G / 2) * sizeof(uint32_t) : 0u);   // scales and biases
  const void *kernel = reinterpret_cast<const void *>(&qmm_ksplit_kernel<WAVES, G, RT, kPair, kRouted, XP>);
  static int per_unit = 0;   // set once per process: the dynamic LDS limit and the occupancy
  if (per_unit == 0) {
    (void)hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, kernel, 64 * WAVES, lds) != hipSuccess || blocks < 1)
      blocks = 1;
    per_unit = blocks > 2 ? 2 : blocks;
  }
  const uint64_t resident = (uint64_t)backend_compute_units(backend) * (uint32_t)per_unit;
  const uint32_t grid = (uint32_t)(most_units < resident ? most_units : resident);
  qmm_ksplit_kernel<WAVES, G, RT, kPair, kRouted, XP><<<dim3(grid), 64 * WAVES, lds, backend_stream(backend)>>>(a);
}

template <int RT, bool kPair, bool kRouted, int XP>
bool launch_shape(fh_backend *backend, const KsplitArgs &a, uint64_t most_units) {
  int waves = 0, groups = 0;
  if (!ksplit_shape(a.inner, &waves, &groups)) return false;
  switch (waves * 16 + groups) {
  case 4 * 16 + 2: launch_one<4, 2, RT, kPair, kRouted, XP>(backend, a, most_units); return true;
  case 6 * 16 + 2: launch_one<6, 2, RT, kPair, kRouted, XP>(backend, a, most_units); return true;
  case 8 * 16 + 2: launch_one<8, 2, RT, kPair, kRouted, XP>(backend, a, most_units); return true;
  case 6 * 16 + 4: launch_one<6, 4, RT, kPair, kRouted, XP>(backend, a, most_units); return true;
  case 8 * 16 + 4: launch_one<8, 4, RT, kPair, kRouted, XP>(backend, a, most_units); return true;
  default: break;
  }
  if constexpr (RT == 1 && !kRouted && XP == 1) {   // the long rows of dense decode products
    if (waves == 8 && groups == 6) {
      launch_one<8, 6, 1, false, false, 1>(backend, a, most_units);
      return true;
    }
    if (waves == 8 && groups == 8) {
      launch_one<8, 8, 1, false, false, 1>(backend, a, most_units);
      return true;
    }
  }
  return false;
}

}  // namespace

bool ksplit_supports(uint32_t inner, uint32_t columns, bool pair, bool routed) {
  int waves, groups;
  if (!ksplit_shape(inner, &waves, &groups) || (routed && groups > 4)) return false;
  return columns % (16u * batch_tiles(pair, groups)) == 0;   // whole batches of columns only
}

// Dense products of up to 128 rows: one row tile (16 rows, or 32 where the K slice of 32 rows fits
// the registers) per pass over the weights.  More than one pass only where the passes after the
// first find the weights in the caches in front of HBM.
constexpr uint64_t kCachedWeightBytes = 32ull << 20;

bool ksplit_dense_supports(uint32_t rows, uint32_t inner, uint32_t columns, bool wide) {
  int waves = 0, groups = 0;
  if (rows == 0 || rows > 128 || !ksplit_shape(inner, &waves, &groups)) return false;
  if (!ksplit_supports(inner, columns, false, false)) return false;
  // f32 rows: 16-row tiles of K slices of at most four groups, two passes at most
  if (wide) return groups <= 4 && rows <= 32 && (rows <= 16 || (uint64_t)columns * inner / 2 <= kCachedWeightBytes);
  const uint32_t tile_rows = rows > 16 && groups <= 4 ? 32 : 16;
  // (row tiles of 16, which the long K slices are held to, would take eight passes for 128 rows)
  return rows <= tile_rows || (groups <= 4 && (uint64_t)columns * inner / 2 <= kCachedWeightBytes);
}

bool launch_ksplit_dense(fh_backend *backend, const KsplitDense &d) {
  int waves = 0, groups = 0;
  if (!ksplit_dense_supports(d.rows, d.inner, d.columns, d.wide) || !ksplit_shape(d.inner, &waves, &groups)) return false;
  if (d.wide && !d.out_f32) return false;
  const bool wide_tiles = d.rows > 16 && groups <= 4 && !d.wide;
  KsplitArgs a{};
  a.x = d.x;
  a.x_row_stride = d.x_row_stride;
  a.packed[0] = d.packed;
  a.scales[0] = d.scales;
  a.biases[0] = d.biases;
  a.out = d.out;
  a.out_row_stride = d.out_row_stride;
  a.out_f32 = d.out_f32;
  a.residual = d.residual;
  a.residual_row_stride = d.residual_row_stride;
  a.rows = d.rows;
  a.inner = d.inner;
  a.weight_inner = d.weight_inner ? d.weight_inner : d.inner;
  a.columns = d.columns;
  const uint32_t batch_cols = 16 * batch_tiles(false, groups);
  a.batches_per_tile = (d.columns + batch_cols - 1) / batch_cols;
  const uint32_t tile_rows = wide_tiles ? 32 : 16;
  const uint64_t units = (uint64_t)((d.rows + tile_rows - 1) / tile_rows) * a.batches_per_tile;
  KernelTimer timer(backend, FH_KC_QMM_KERNEL);
  if (d.wide) return launch_shape<1, false, false, 3>(backend, a, units);
  return wide_tiles ? launch_shape<2, false, false, 1>(backend, a, units)
                    : launch_shape<1, false, false, 1>(backend, a, units);
}

bool launch_ksplit_routed(fh_backend *backend, const KsplitRouted &r) {
  int waves = 0, groups = 0;
  if ((r.tile_rows != 16 && r.tile_rows != 32) || !ksplit_shape(r.inner, &waves, &groups)) return false;
  if (!ksplit_supports(r.inner, r.columns, r.pair, true)) return false;
  if (groups > 4) return false;
  KsplitArgs a{};
  a.x = r.x;
  a.x_row_stride = r.x_row_stride;
  for (int pj = 0; pj < (r.pair ? 2 : 1); ++pj) {
    a.packed[pj] = r.packed[pj];
    a.scales[pj] = r.scales[pj];
    a.biases[pj] = r.biases[pj];
  }
  a.expert_words = (uint64_t)r.columns * r.inner / 8;
  a.expert_groups = (uint64_t)r.columns * r.inner / kGroup;
  a.out = r.out;
  a.out_row_stride = r.columns;
  a.out_f32 = r.out_f32;
  a.inner = r.inner;
  a.weight_inner = r.inner;
  a.columns = r.columns;
  a.sorted_routes = r.sorted_routes;
  a.blocks = r.blocks;
  a.n_blocks = r.n_blocks;
  a.route_div = r.route_div;
  const uint32_t batch_cols = 16 * batch_tiles(r.pair, groups);
  a.batches_per_tile = (r.columns + batch_cols - 1) / batch_cols;
  const uint64_t most = (uint64_t)r.max_blocks * a.batches_per_tile;
  if (r.wide) {   // f32 rows: 16-row tiles, f32 results
    if (r.tile_rows != 16 || !r.out_f32) return false;
    return r.pair ? launch_shape<1, true, true, 3>(backend, a, most) : launch_shape<1, false, true, 3>(backend, a, most);
  }
  if (r.pair)
    return r.tile_rows == 16 ? launch_shape<1, true, true, 1>(backend, a, most)
                             : launch_shape<2, true, true, 1>(backend, a, most);
  return r.tile_rows == 16 ? launch_shape<1, false, true, 1>(backend, a, most)
                           : launch_shape<2, false, true, 1>(backend, a, most);
}

}  // namespace fh
