// MLX-4bit quantised matmul for many activation rows (prefill chunks): a tiled f16 MFMA GEMM
// whose weight operand is dequantised on its way from LDS into the operand registers
// (gemm_q4_kernel: the packed words travel, 0.5 byte per weight), or, for the shapes that kernel
// does not take, read from an fp16 matrix written once per weight (gemm_f16_wide_kernel,
// gemm_f16_kernel).
//
// y[m,n] = sum_k x[m,k] * (scale[n,k/64] * q[n,k] + bias[n,k/64])   (affine_quant_dot,
// crates/forja-cpu/src/lib.rs:1277-1310).  With thousands of rows per weight the work is bound
// by the matrix cores, not by HBM.
//   * Operands are fp16, not bf16: a dequantised weight rounded to bf16 (8 significant bits) is
//     too coarse for the stated tolerance on outputs that cancel, fp16 (11 bits) is not, and the
//     matrix cores run both at the same rate.  bf16 activations convert to fp16 exactly once a row
//     is scaled by a power of two into the fp16 range (undone exactly when the result is stored).
//   * Weights are centred: w = scale * q - c with c = 7.5 * scale, which halves their magnitude
//     and so their rounding error; at the deepest contraction (K = 17408) the uncentred form does
//     not meet the tolerance.  What centring takes out, (bias + c) * sum of the group's
//     activations, is put back through the same GEMM: both operands get three more K columns per
//     quantisation group, holding S/64 and 64 * (bias + c) each split in an fp16 head and tail
//     (head*head + tail*head + head*tail, about 22 significant bits), so the kernel needs no
//     side channel for it.  The contraction grows by 3/64.
//   * prepare_rows_kernel writes the activation operand [rows, Kt], Kt = K + 3K/64 rounded up to
//     the K step, every 8 values in the order (0,4,1,5,2,6,3,7) in which nibbles unpack pairwise.
//     prepare_extras_kernel writes the weights' extra columns [N, Kt - K] (kept per weight matrix
//     by the backend: 3/64 of a value per weight), prepare_weights_kernel the whole fp16 operand
//     [N, Kt] for the kernels that read one.  Both raise a flag when some scale or bias does not
//     fit this scheme's fp16 range; the GEMM kernel then returns at once and the caller runs its
//     any-range kernel instead.
//   * GEMM: workgroup tile 256 rows x 256 columns, K step 64, eight waves in a 2 x 4 arrangement
//     (two per SIMD), each owning 128 x 64 outputs = 8 accumulator tiles of
//     v_mfma_f32_32x32x16_f16; 128 x 128 tiles of four waves where the large tiles would leave
//     compute units idle.  What comes from memory goes straight into LDS (no registers), double
//     buffered, 16-byte pieces XOR-swizzled inside each row so that operand reads are
//     bank-conflict free without padding; one barrier per step.  Operand registers are double
//     buffered too: the reads of a sub-step are issued before the previous sub-step's MFMAs.
//   * The workgroup -> tile map gives the 32 workgroups that run together on one XCD a patch of
//     about 4 row tiles x 8 column tiles, so that its L2 serves each activation tile to 8
//     workgroups and each weight tile to 4, instead of every workgroup streaming its own.
// Accumulation is f32.
#include <type_traits>

#include "fast_kernels.hpp"

namespace fh {

namespace {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kBM = 256, kBN = 256;
constexpr int kPadK = 64;   // operand rows are padded to a multiple of this (every K step divides it)
// K step and LDS stages of the GEMM.  Steps of 32 with three or four stages measured the same
// (the kernel is bound by what the matrix cores and the L2 -> LDS path sustain, not by latency).
constexpr int kGemmK = 64, kGemmStages = 2;
// A tile is 2 x 2 quadrants of kQ x kQ, one per wave: kQ = 128 (256 x 256 tiles) wherever that
// gives every compute unit work, kQ = 64 (128 x 128 tiles, four times as many) for the small
// products of small models, which would otherwise leave most of the device idle.
constexpr int out_pitch(int quadrant) { return 2 * quadrant + 16; }   // bytes per row of a wave's staged output quadrant
constexpr int gemm_lds_bytes(int quadrant) {
  const int pipeline = kGemmStages * 2 * (2 * quadrant) * 2 * kGemmK;   // both operand tiles of every stage
  const int output = 4 * (quadrant * out_pitch(quadrant) + 4 * quadrant);   // four quadrants of bf16 rows + row factors
  return pipeline > output ? pipeline : output;
}
constexpr int gemm_q4_lds_bytes(int side, int waves, int part_rows, int part_columns) {
  const int pipeline = 4 * side * 2 * kGemmK + 2 * side * 64;   // two tiles a side + packed words of two pairs of K steps
  const int output = waves * (part_rows * out_pitch(part_columns) + 4 * part_rows);
  return pipeline > output ? pipeline : output;
}
constexpr int kLargeLds = gemm_q4_lds_bytes(256, 8, 128, 64), kSmallLds = gemm_q4_lds_bytes(128, 4, 64, 64);
constexpr int kWideLds = 8 * (128 * out_pitch(64) + 4 * 128) > 4 * 256 * 2 * kGemmK ? 8 * (128 * out_pitch(64) + 4 * 128)
                                                                                      : 4 * 256 * 2 * kGemmK;
constexpr int kBand = 8;   // column tiles per band of the tile numbering
constexpr uint32_t kMaxGroups = 512;              // quantisation groups per row the row kernel holds

// Columns of the operand matrices: K values, then 3 per group, rounded up to the K step.
inline uint32_t padded_inner(uint32_t inner) {
  const uint32_t with_sums = inner + 3 * (inner / 64);
  return (with_sums + kPadK - 1) / kPadK * kPadK;
}

struct GemmArgs {
  const uint16_t *a, *b;    // fp16 operand matrices [rows, kt] and [columns, kt]
  // gemm_q4_kernel instead of b: the weights as they are, and the fp16 columns [columns, kt - inner]
  // that follow the inner values in a row of b
  const uint32_t *packed;
  const uint16_t *scales;
  const uint16_t *extras;
  uint32_t inner;
  const float *row_unscale; // per row: multiply the result by this
  uint32_t kt;
  void *out;
  uint64_t out_row_stride;
  uint32_t out_f32;
  uint32_t rows, columns;
  uint32_t row_tiles, column_tiles;
  const uint32_t *refused;     // non-zero: some scale or bias is out of range, do nothing
  const uint16_t *residual;    // optional bf16 rows added before rounding
  uint64_t residual_row_stride;
  uint32_t row_stores;         // bf16 output (and residual) rows are 16-byte aligned, columns % 8 == 0
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

__device__ inline uint16_t f16_bits(float v) {
  return __builtin_bit_cast(uint16_t, (_Float16)v);
}

// Head and tail of v in fp16: v ~ head + tail.
__device__ inline void split_f16(float v, float *head, float *tail) {
  *head = (float)(_Float16)v;
  *tail = (float)(_Float16)(v - *head);
}

// x bf16 [rows, inner] -> fp16 [rows, kt].  Each row is multiplied by the power of two that
// brings its largest magnitude into [2^14, 2^15) (unscale[row] is the inverse); every 8 values are
// stored in the order (0,4,1,5,2,6,3,7); after the inner values come, for every group g of 64,
// (head, tail, head) of S_g / 64 with S_g the f32 sum of the group's scaled values, then zeros.
// One wave per row.
__global__ __launch_bounds__(256) void prepare_rows_kernel(const uint16_t *x, uint64_t x_row_stride,
                                                           uint32_t rows, uint32_t inner, uint32_t kt,
                                                           uint16_t *out, float *unscale,
                                                           uint32_t *refused) {
  __shared__ float sums[4][kMaxGroups];
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t row = blockIdx.x * 4 + wave;
  // the refusal flag of this product starts clear (prepare_weights_kernel, launched next, sets it)
  if (blockIdx.x == 0 && threadIdx.x == 0) refused[0] = 0;
  if (row >= rows) return;   // no workgroup-wide barrier below
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
  int down = exponent - 14;                                      // scale by 2^-down
  if (down < -100) down = -100;                                  // rows of zeros and denormals
  const float scale = __uint_as_float((uint32_t)(127 - down) << 23);
  if (lane == 0) unscale[row] = __uint_as_float((uint32_t)(127 + down) << 23);
  uint16_t *out_row = out + (uint64_t)row * kt;
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
    if ((piece & 7) == 0) sums[wave][piece >> 3] = sum;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const uint32_t groups = inner / 64;
  for (uint32_t extra = lane; extra < kt - inner; extra += 64) {
    const uint32_t group = extra / 3, kind = extra % 3;
    float value = 0.0f;
    if (group < groups) {
      float head, tail;
      split_f16(sums[wave][group] * (1.0f / 64.0f), &head, &tail);
      value = kind == 1 ? tail : head;
    }
    out_row[inner + extra] = f16_bits(value);
  }
}

// Scales and biases this scheme can take: every centred weight and 64 * (bias + centre) must
// stay inside the fp16 range.  False for NaN too.
__device__ inline bool f16_safe(float scale, float bias) {
  return fabsf(scale) <= 4000.0f && fabsf(bias + 7.5f * scale) <= 900.0f;
}

// packed/scales/biases [columns, inner] -> fp16 [columns, kt]: scale * q - 7.5 * scale (one
// rounding, from f32) in the order (0,4,1,5,2,6,3,7) inside every 8, then per group (head, head,
// tail) of 64 * (bias + 7.5 * scale), then zeros.  Eight threads per 64-value chunk, one packed
// word each; refused[0] is set when a group is out of range.
__global__ __launch_bounds__(256) void prepare_weights_kernel(const uint32_t *packed,
                                                              const uint16_t *scales,
                                                              const uint16_t *biases, uint32_t columns,
                                                              uint32_t inner, uint32_t kt,
                                                              uint16_t *out, uint32_t *refused) {
  const uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t part = (uint32_t)(flat & 7);
  const uint32_t chunks = kt / 64, groups = inner / 64;
  const uint64_t chunk_flat = flat >> 3;
  if (chunk_flat >= (uint64_t)columns * chunks) return;
  const uint32_t column = (uint32_t)(chunk_flat / chunks), chunk = (uint32_t)(chunk_flat % chunks);
  uint16_t *to = out + (uint64_t)column * kt + 64 * chunk + 8 * part;
  const uint16_t *s_row = scales + (uint64_t)column * groups, *b_row = biases + (uint64_t)column * groups;
  if (chunk < groups) {
    const float scale = bf16_bits_to_f32(s_row[chunk]), bias = bf16_bits_to_f32(b_row[chunk]);
    if (part == 0 && !f16_safe(scale, bias)) refused[0] = 1;
    const uint32_t w = packed[(uint64_t)column * (inner / 8) + 8 * chunk + part];
    const float centre = 7.5f * scale;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = __builtin_fmaf(scale, (float)((w >> (4 * i)) & 15u), -centre);
    *(uint4 *)to = make_uint4(pack_f16(v[0], v[4]), pack_f16(v[1], v[5]), pack_f16(v[2], v[6]),
                              pack_f16(v[3], v[7]));
    return;
  }
  uint16_t values[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t extra = 64 * (chunk - groups) + 8 * part + i;
    const uint32_t group = extra / 3, kind = extra % 3;
    float value = 0.0f;
    if (group < groups) {
      const float scale = bf16_bits_to_f32(s_row[group]), bias = bf16_bits_to_f32(b_row[group]);
      float head, tail;
      split_f16(64.0f * (bias + 7.5f * scale), &head, &tail);
      value = kind == 2 ? tail : head;
    }
    values[i] = f16_bits(value);
  }
  *(uint4 *)to = make_uint4(values[0] | ((uint32_t)values[1] << 16), values[2] | ((uint32_t)values[3] << 16),
                            values[4] | ((uint32_t)values[5] << 16), values[6] | ((uint32_t)values[7] << 16));
}

constexpr uint32_t wait_vmcnt(uint32_t n) {   // s_waitcnt immediate: vmcnt(n) only
  return (n & 15u) | ((n >> 4) << 14) | 0x0f70u;
}

// Stores a workgroup's finished tile: acc[i][j] is the 32 x 32 block (i, j) of wave (wm, wn)'s
// quadrant, rows scaled back by row_unscale, the residual rows added, one rounding.
// A wave's part of the tile is kQM rows x kQN columns; the waves are arranged kWN to a row.
template <int kQM, int kQN, int kWN>
__device__ inline void store_tile(const GemmArgs &a, f32x16 (&acc)[kQM / 32][kQN / 32], unsigned char *gemm_lds,
                                  uint32_t row0, uint32_t col0) {
  constexpr int kMIR = kQM / 32, kMIC = kQN / 32;
  constexpr int kOutPitch = out_pitch(kQN);
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave / kWN, wn = wave % kWN;
  const uint32_t l32 = lane & 31, kh = lane >> 5;
  // Lane (column l32, half kh) holds rows 8*(r/4) + 4*kh + r%4 of each 32 x 32 tile: a column
  // per lane, the wrong way round for memory.  When the output rows allow 16-byte stores, every
  // wave turns its 128 x 128 quadrant round through its own piece of LDS: the residual rows (if
  // any) are staged there first, every lane then replaces "its" elements by the finished bf16
  // result (f32 sum, one rounding), and the rows leave with one 16-byte store per lane, 256
  // contiguous bytes per row.  Only wave-local ordering is needed: nobody else touches the piece.
  if (a.row_stores) {
    constexpr int kPieces = kQN / 8;           // 16-byte pieces of a quadrant's row
    constexpr int kRowsAtOnce = 64 / kPieces;  // rows one wave-wide 16-byte access covers
    unsigned char *mine = gemm_lds + wave * (kQM * kOutPitch + 4 * kQM);
    float *unscale_of = (float *)(mine + kQM * kOutPitch);   // the quadrant's row factors
    const uint32_t quad_row0 = row0 + kQM * wm, quad_col0 = col0 + kQN * wn;
    const uint32_t piece_row = lane / kPieces, piece_col = 8 * (lane % kPieces);
    unscale_of[lane] = a.row_unscale[min(quad_row0 + lane, a.rows - 1)];
    if (kQM > 64) unscale_of[64 + lane] = a.row_unscale[min(quad_row0 + 64 + lane, a.rows - 1)];
    if (a.residual) {
#pragma unroll 4
      for (int it = 0; it < kQM / kRowsAtOnce; ++it) {
        const uint32_t row = kRowsAtOnce * it + piece_row;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (quad_row0 + row < a.rows && quad_col0 + piece_col < a.columns)
          v = *(const uint4 *)(a.residual + (uint64_t)(quad_row0 + row) * a.residual_row_stride +
                               quad_col0 + piece_col);
        *(uint4 *)(mine + row * kOutPitch + 2 * piece_col) = v;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int i = 0; i < kMIR; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const uint32_t row = 32 * i + 8 * (r / 4) + 4 * kh + (r % 4);
        const float unscale = unscale_of[row];
#pragma unroll
        for (int j = 0; j < kMIC; ++j) {
          uint16_t *slot = (uint16_t *)(mine + row * kOutPitch) + 32 * j + l32;
          float value = acc[i][j][r] * unscale;
          if (a.residual) value += bf16_bits_to_f32(*slot);
          *slot = (uint16_t)(pack2(value, 0.0f) & 0xffffu);
        }
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    uint16_t *out = (uint16_t *)a.out;
#pragma unroll 4
    for (int it = 0; it < kQM / kRowsAtOnce; ++it) {
      const uint32_t row = kRowsAtOnce * it + piece_row;
      const uint4 v = *(const uint4 *)(mine + row * kOutPitch + 2 * piece_col);
      if (quad_row0 + row < a.rows && quad_col0 + piece_col < a.columns)
        *(uint4 *)(out + (uint64_t)(quad_row0 + row) * a.out_row_stride + quad_col0 + piece_col) = v;
    }
    return;
  }
  // store: lane (column l32, half kh) holds rows 8*(r/4) + 4*kh + r%4 of each 32 x 32 tile
#pragma unroll
  for (int i = 0; i < kMIR; ++i)
#pragma unroll
    for (int j = 0; j < kMIC; ++j) {
      const uint32_t column = col0 + kQN * wn + 32 * j + l32;
      if (column >= a.columns) continue;
      for (int r = 0; r < 16; ++r) {
        const uint32_t row = row0 + kQM * wm + 32 * i + 8 * (r / 4) + 4 * kh + (r % 4);
        if (row >= a.rows) continue;
        const uint64_t at_out = (uint64_t)row * a.out_row_stride + column;
        float value = acc[i][j][r] * a.row_unscale[row];
        if (a.residual)
          value += __uint_as_float((uint32_t)a.residual[(uint64_t)row * a.residual_row_stride + column] << 16);
        if (a.out_f32)
          ((float *)a.out)[at_out] = value;
        else
          ((uint16_t *)a.out)[at_out] = (uint16_t)(pack2(value, 0.0f) & 0xffffu);
      }
    }
}

template <int kBK, int kStages, int kQ>
__global__ __launch_bounds__(256) void gemm_f16_kernel(GemmArgs a) {
  if (a.refused[0] != 0) return;
  constexpr int kSide = 2 * kQ;                  // rows (and columns) of a tile
  constexpr int kMI = kQ / 32;                   // 32 x 32 blocks along a quadrant's side
  constexpr int kSub = kBK / 16;                 // MFMA sub-steps per K step
  constexpr int kRowBytes = 2 * kBK;             // one tile row in LDS
  constexpr int kTile = kSide * kRowBytes;       // one operand tile of one stage
  constexpr int kSlots = kRowBytes / 16;         // 16-byte pieces per row
  constexpr int kRowsPerLoad = 64 / kSlots;      // rows one wave-wide load instruction covers
  constexpr int kStaged = kSide / 4;             // rows of each operand tile a wave stages
  constexpr int kLoads = kStaged / kRowsPerLoad; // instructions per wave, operand and stage
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_lds[];
  unsigned char *a_tiles = gemm_lds;                      // [kStages][kBM][kRowBytes], pieces swizzled
  unsigned char *b_tiles = gemm_lds + kStages * kTile;    // [kStages][kBN][kRowBytes]
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: LDS bases stay scalar
  const uint32_t wm = wave >> 1, wn = wave & 1;
  const uint32_t l32 = lane & 31, kh = lane >> 5;
  // A row's piece p sits in slot p ^ swizzle(row), which spreads the 32 rows a wave reads at once
  // over all LDS banks.
  auto swizzle_of = [](uint32_t row) { return kBK == 64 ? (row >> 1) & 7u : (row >> 2) & 3u; };

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
  const uint32_t row0 = bm * kSide, col0 = bn * kSide;

  // Staging: a wave owns 64 rows of each operand tile; one instruction moves kRowsPerLoad rows
  // (lane -> row lane / kSlots, LDS slot lane % kSlots) and the piece a lane fetches is its slot
  // XOR the row's swizzle.  Rows past the end of a matrix reload its last row; what they produce
  // is never stored.  Addresses are a wave-uniform base that advances with the K step plus a
  // 32-bit per-lane offset that never changes (both matrices are far below 4 GiB).
  uint32_t a_off[kLoads], b_off[kLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const uint32_t in_tile = kStaged * wave + kRowsPerLoad * i + lane / kSlots;
    const uint32_t piece = (lane % kSlots) ^ swizzle_of(in_tile);
    a_off[i] = (min(row0 + in_tile, a.rows - 1) * a.kt + 8 * piece) * 2;
    b_off[i] = (min(col0 + in_tile, a.columns - 1) * a.kt + 8 * piece) * 2;
  }
  const uint32_t steps = a.kt / kBK;
  // one pair of load instructions (activation rows and weight rows) of stage `step`
  auto stage_pair = [&](uint32_t buffer, uint32_t step, int i) {
    const uint32_t st = min(step, steps - 1);   // past the end: reload the last step, never used
    const unsigned char *from_a = (const unsigned char *)a.a + (uint64_t)st * (kBK * 2);
    const unsigned char *from_b = (const unsigned char *)a.b + (uint64_t)st * (kBK * 2);
    unsigned char *to_a = a_tiles + buffer * kTile + (kStaged * wave + kRowsPerLoad * i) * kRowBytes;
    unsigned char *to_b = b_tiles + buffer * kTile + (kStaged * wave + kRowsPerLoad * i) * kRowBytes;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(from_a + a_off[i]),
                                     (__attribute__((address_space(3))) void *)to_a, 16, 0, 0);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(from_b + b_off[i]),
                                     (__attribute__((address_space(3))) void *)to_b, 16, 0, 0);
  };

  f32x16 acc[kMI][kMI];
#pragma unroll
  for (int i = 0; i < kMI; ++i)
#pragma unroll
    for (int j = 0; j < kMI; ++j)
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Operand registers, two sets: the set for the next sub-step is read from LDS while the matrix
  // pipe works on the current one.
  f16x8 a_op[2][kMI], b_op[2][kMI];
  const uint32_t swizzle = swizzle_of(l32);
  auto read_operands = [&](uint32_t buffer, int s, int set) {
    const unsigned char *at = a_tiles + buffer * kTile + (kQ * wm + l32) * kRowBytes;
    const unsigned char *bt = b_tiles + buffer * kTile + (kQ * wn + l32) * kRowBytes;
    const uint32_t piece = 16 * ((2 * s + kh) ^ swizzle);
#pragma unroll
    for (int i = 0; i < kMI; ++i) {
      a_op[set][i] = __builtin_bit_cast(f16x8, *(const uint4 *)(at + 32 * i * kRowBytes + piece));
      b_op[set][i] = __builtin_bit_cast(f16x8, *(const uint4 *)(bt + 32 * i * kRowBytes + piece));
    }
  };

  // K pipeline over kStages LDS buffers.  During step t the loads of step t + kStages - 1 are
  // issued into the buffer step t - 1 has just freed, one pair of instructions behind every
  // fourth MFMA so that they issue in the shadow of the matrix pipe; at the end of step t the
  // loads of step t + 1 must have landed.
#pragma unroll
  for (int p = 0; p < kStages - 1; ++p)
#pragma unroll
    for (int i = 0; i < kLoads; ++i) stage_pair(p, p, i);
  __builtin_amdgcn_s_waitcnt(wait_vmcnt((kStages - 2) * 2 * kLoads));   // step 0 has landed
  __syncthreads();
  uint32_t buffer = 0, refill = kStages - 1;
  for (uint32_t step = 0; step < steps; ++step) {
    read_operands(buffer, 0, 0);
    int issued = 0;
#pragma unroll
    for (int s = 0; s < kSub; ++s) {
      __builtin_amdgcn_sched_barrier(0);
      if (s + 1 < kSub) read_operands(buffer, s + 1, (s + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < kMI; ++i) {
#pragma unroll
        for (int j = 0; j < kMI; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_op[s & 1][i], b_op[s & 1][j], acc[i][j], 0, 0, 0);
        if (issued < kLoads) {
          __builtin_amdgcn_sched_barrier(0);
          stage_pair(refill, step + kStages - 1, issued);
          ++issued;
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    static_assert(kLoads <= kMI * kSub, "one load pair per MFMA row at most");
    __builtin_amdgcn_s_waitcnt(0xc07f);                                   // lgkmcnt(0): reads done
    __builtin_amdgcn_s_waitcnt(wait_vmcnt((kStages - 2) * 2 * kLoads));   // step + 1 has landed
    __syncthreads();
    refill = buffer;
    buffer = buffer + 1 == kStages ? 0 : buffer + 1;
  }
  __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));   // nothing is on its way into LDS any more
  __syncthreads();
  store_tile<kQ, kQ, 2>(a, acc, gemm_lds, row0, col0);
}


// 64 lanes x 16 bytes from memory straight into LDS at `lds_base` + 16 * lane, issued as an
// instruction the compiler does not see: while it knows of such a load in flight it waits for ALL
// outstanding LDS reads wherever it has to wait for one (it cannot tell the load's LDS write from
// the wave's own LDS traffic), i.e. also for the operand reads just issued for the next sub-step,
// and it drains every such load at a __syncthreads().  Callers order these loads by hand (vmcnt).
__device__ inline void load_to_lds_16(const void *from, unsigned char *lds_base) {
  // (uniform by construction; the intrinsic tells the compiler so)
  const uint32_t at = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds_base);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(from), "s"(at) : "memory");   // (m0 is the compiler's only for its own such loads: kernels that use this have none)
}

__device__ inline void lds_barrier() { asm volatile("s_barrier" ::: "memory"); }

// The same GEMM with eight waves to a 256 x 256 tile (two per SIMD), each owning 128 rows x 64
// columns (128 accumulator registers): while one wave of a SIMD waits for its operands or at the
// barrier the other one feeds the matrix pipe.
template <int kBK>
__global__ __launch_bounds__(512) void gemm_f16_wide_kernel(GemmArgs a) {
  if (a.refused[0] != 0) return;
  constexpr int kSide = 256, kQM = 128, kQN = 64, kWN = 4;
  constexpr int kMIR = kQM / 32, kMIC = kQN / 32;
  constexpr int kSub = kBK / 16;
  constexpr int kRowBytes = 2 * kBK;
  constexpr int kTile = kSide * kRowBytes;
  constexpr int kSlots = kRowBytes / 16;
  constexpr int kRowsPerLoad = 64 / kSlots;
  constexpr int kStaged = kSide / 8;             // rows of each operand tile a wave stages
  constexpr int kLoads = kStaged / kRowsPerLoad;
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_lds[];
  unsigned char *a_tiles = gemm_lds;
  unsigned char *b_tiles = gemm_lds + 2 * kTile;
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave / kWN, wn = wave % kWN;
  const uint32_t l32 = lane & 31, kh = lane >> 5;
  auto swizzle_of = [](uint32_t row) { return kBK == 64 ? (row >> 1) & 7u : (row >> 2) & 3u; };
  const uint32_t xcd = blockIdx.x % 8, nth = blockIdx.x / 8;
  const uint32_t tile = (nth / 32) * 256 + xcd * 32 + nth % 32;
  if (tile >= a.row_tiles * a.column_tiles) return;
  const uint32_t band = tile / (a.row_tiles * kBand);
  const uint32_t band_width = min((uint32_t)kBand, a.column_tiles - band * kBand);
  const uint32_t in_band = tile - band * a.row_tiles * kBand;
  const uint32_t bm = in_band / band_width, bn = band * kBand + in_band % band_width;
  const uint32_t row0 = bm * kSide, col0 = bn * kSide;
  uint32_t a_off[kLoads], b_off[kLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const uint32_t in_tile = kStaged * wave + kRowsPerLoad * i + lane / kSlots;
    const uint32_t piece = (lane % kSlots) ^ swizzle_of(in_tile);
    a_off[i] = (min(row0 + in_tile, a.rows - 1) * a.kt + 8 * piece) * 2;
    b_off[i] = (min(col0 + in_tile, a.columns - 1) * a.kt + 8 * piece) * 2;
  }
  const uint32_t steps = a.kt / kBK;
  auto stage_pair = [&](uint32_t buffer, uint32_t step, int i) {
    const uint32_t st = min(step, steps - 1);
    const unsigned char *from_a = (const unsigned char *)a.a + (uint64_t)st * (kBK * 2);
    const unsigned char *from_b = (const unsigned char *)a.b + (uint64_t)st * (kBK * 2);
    unsigned char *to_a = a_tiles + buffer * kTile + (kStaged * wave + kRowsPerLoad * i) * kRowBytes;
    unsigned char *to_b = b_tiles + buffer * kTile + (kStaged * wave + kRowsPerLoad * i) * kRowBytes;
    load_to_lds_16(from_a + a_off[i], to_a);
    load_to_lds_16(from_b + b_off[i], to_b);
  };
  f32x16 acc[kMIR][kMIC];
#pragma unroll
  for (int i = 0; i < kMIR; ++i)
#pragma unroll
    for (int j = 0; j < kMIC; ++j)
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  f16x8 a_op[2][kMIR], b_op[2][kMIC];
  const uint32_t swizzle = swizzle_of(l32);
  auto read_operands = [&](uint32_t buffer, int s, int set) {
    const unsigned char *at = a_tiles + buffer * kTile + (kQM * wm + l32) * kRowBytes;
    const unsigned char *bt = b_tiles + buffer * kTile + (kQN * wn + l32) * kRowBytes;
    const uint32_t piece = 16 * ((2 * s + kh) ^ swizzle);
#pragma unroll
    for (int i = 0; i < kMIR; ++i)
      a_op[set][i] = __builtin_bit_cast(f16x8, *(const uint4 *)(at + 32 * i * kRowBytes + piece));
#pragma unroll
    for (int j = 0; j < kMIC; ++j)
      b_op[set][j] = __builtin_bit_cast(f16x8, *(const uint4 *)(bt + 32 * j * kRowBytes + piece));
  };
#pragma unroll
  for (int i = 0; i < kLoads; ++i) stage_pair(0, 0, i);
  __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));
  lds_barrier();
  uint32_t buffer = 0;
  for (uint32_t step = 0; step < steps; ++step) {
    read_operands(buffer, 0, 0);
    int issued = 0;
#pragma unroll
    for (int s = 0; s < kSub; ++s) {
      __builtin_amdgcn_sched_barrier(0);
      if (s + 1 < kSub) read_operands(buffer, s + 1, (s + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < kMIR; ++i) {
#pragma unroll
        for (int j = 0; j < kMIC; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_op[s & 1][i], b_op[s & 1][j], acc[i][j], 0, 0, 0);
        if (issued < kLoads) {
          __builtin_amdgcn_sched_barrier(0);
          stage_pair(buffer ^ 1u, step + 1, issued);
          ++issued;
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));
    lds_barrier();
    buffer ^= 1u;
  }
  lds_barrier();
  store_tile<kQM, kQN, kWN>(a, acc, gemm_lds, row0, col0);
}

// packed/scales/biases [columns, inner] -> the columns an operand row holds after its inner
// values, fp16 [columns, kt - inner]: per group (head, head, tail) of 64 * (bias + 7.5 * scale),
// then zeros.  One thread per 8 values; refused[0] is set when a group is out of range.
__global__ __launch_bounds__(256) void prepare_extras_kernel(const uint16_t *scales, const uint16_t *biases,
                                                             uint32_t columns, uint32_t inner, uint32_t kt,
                                                             uint16_t *out, uint32_t *refused) {
  const uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t width = kt - inner, chunks = width / 8, groups = inner / 64;
  if (flat >= (uint64_t)columns * chunks) return;
  const uint32_t column = (uint32_t)(flat / chunks), chunk = (uint32_t)(flat % chunks);
  const uint16_t *s_row = scales + (uint64_t)column * groups, *b_row = biases + (uint64_t)column * groups;
  uint16_t values[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t extra = 8 * chunk + i;
    const uint32_t group = extra / 3, kind = extra % 3;
    float value = 0.0f;
    if (group < groups) {
      const float scale = bf16_bits_to_f32(s_row[group]), bias = bf16_bits_to_f32(b_row[group]);
      // the GEMM multiplies by the scale as an fp16 number: it must be one exactly
      if (kind == 0 && (!f16_safe(scale, bias) || (scale != 0.0f && fabsf(scale) < 6.103515625e-5f))) refused[0] = 1;
      float head, tail;
      split_f16(64.0f * (bias + 7.5f * scale), &head, &tail);
      value = kind == 2 ? tail : head;
    }
    values[i] = f16_bits(value);
  }
  *(uint4 *)(out + (uint64_t)column * width + 8 * chunk) =
      make_uint4(values[0] | ((uint32_t)values[1] << 16), values[2] | ((uint32_t)values[3] << 16),
                 values[4] | ((uint32_t)values[5] << 16), values[6] | ((uint32_t)values[7] << 16));
}

// Eight nibbles of `w` as the centred weights scale * (q - 7.5) in fp16, in the order
// (0,4)(1,5)(2,6)(3,7).  A nibble lands in mantissa bits 1..4 of 512.0 (whose unit in the last
// place is 0.5), giving 512 + q exactly; 519.5 is taken off exactly and the product with the
// scale is rounded once, like a weight formed in f32 and rounded.  scale2 = (scale, scale).
__device__ inline f16x8 dequantise_word(uint32_t w, f16x2 scale2, uint32_t mask, uint32_t magic) {
  const f16x2 centre = {(_Float16)519.5f, (_Float16)519.5f};
  uint32_t bits[4] = {((w << 1) & mask) | magic, ((w >> 3) & mask) | magic, ((w >> 7) & mask) | magic,
                      ((w >> 11) & mask) | magic};
  uint4 r;
  r.x = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(f16x2, bits[0]) - centre) * scale2);
  r.y = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(f16x2, bits[1]) - centre) * scale2);
  r.z = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(f16x2, bits[2]) - centre) * scale2);
  r.w = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(f16x2, bits[3]) - centre) * scale2);
  return __builtin_bit_cast(f16x8, r);
}

// The GEMM with the weights dequantised on their way into LDS.
//   * Waves: kWM x kWN of them share a square tile, each owning kQM rows x kQN columns of it:
//     2 x 4 waves of 128 x 64 for 256 x 256 tiles (two waves per SIMD: while one waits for its
//     operands or at the barrier the other feeds the matrix pipe; with one wave per SIMD owning
//     128 x 128 the pipe sat idle 45 % of the time), 2 x 2 waves of 64 x 64 for 128 x 128 tiles (two
//     workgroups per compute unit).
//   * Activations: the fp16 rows prepare_rows_kernel writes, from memory straight into LDS
//     (load_to_lds_16), double buffered.
//   * Weights: the packed words themselves go from memory into LDS the same way (64 bytes = two K
//     steps of a column per request, half a byte per weight instead of two), and from there into
//     the operand registers: a lane reads the 16 bytes that hold its 32 weights of a K step (a
//     column, half a group) and turns one word into one matrix operand per sub-step (per nibble
//     pair two integer and two packed fp16 instructions).  The dequantised weights never exist in
//     LDS: per K step a workgroup moves 40 KB from memory instead of 64 and reads 150 KB of LDS
//     instead of 190.
//   * The columns after the inner values (the bias term, see the head of this file) are plain fp16
//     on both sides: for the last few K steps the weights' tile is loaded from `extras`.
//   * Scales: a thread keeps the bf16 scales of eight groups of its column in registers (one
//     16-byte load per eight K steps).
//   * Every load into LDS is issued as inline assembly and ordered by the waits written here
//     (see load_to_lds_16, lds_barrier): what the compiler knows of are the operand reads, whose
//     waits it then counts exactly.
// LDS: activations [2][side][128 B], fp16 weights of the extra columns [2][side][128 B], packed words of two pairs of K
// steps [2][side][64 B].  A column's four 16-byte quarters of a pair sit in slots
// quarter ^ ((column >> 2) & 3), which spreads the 16 lanes a read serves at once over all banks.
template <int kWM, int kWN, int kQM, int kQN>
__global__ __launch_bounds__(64 * kWM * kWN) void gemm_q4_kernel(GemmArgs a) {
  if (a.refused[0] != 0) return;
  constexpr int kWaves = kWM * kWN, kThreads = 64 * kWaves;
  constexpr int kBK = 64;
  constexpr int kSide = kQM * kWM;
  static_assert(kSide == kQN * kWN, "square tiles");
  constexpr int kMIR = kQM / 32, kMIC = kQN / 32;
  constexpr int kSub = 4;
  constexpr int kRowBytes = 2 * kBK;
  constexpr int kTile = kSide * kRowBytes;       // one fp16 operand tile
  constexpr int kPair = kSide * 64;              // the packed words of two K steps of a tile's columns
  constexpr int kStaged = kSide / kWaves;        // rows of an fp16 tile a wave stages
  constexpr int kLoads = kStaged / 8;            // instructions per wave and fp16 tile (8 rows each)
  constexpr int kPairLoads = kSide / 16 / kWaves;   // instructions per wave and pair (16 columns each)
  extern __shared__ __attribute__((aligned(16))) unsigned char gemm_lds[];
  unsigned char *a_tiles = gemm_lds;                 // [2][kSide][128]
  unsigned char *b_tiles = gemm_lds + 2 * kTile;     // [2][kSide][128]
  unsigned char *pairs = gemm_lds + 4 * kTile;       // [2][kSide][64]
  const uint32_t tid = threadIdx.x, lane = tid & 63;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t wm = wave / kWN, wn = wave % kWN;
  const uint32_t l32 = lane & 31, kh = lane >> 5;
  auto swizzle_of = [](uint32_t row) { return (row >> 1) & 7u; };

  const uint32_t xcd = blockIdx.x % 8, nth = blockIdx.x / 8;
  const uint32_t tile = (nth / 32) * 256 + xcd * 32 + nth % 32;
  if (tile >= a.row_tiles * a.column_tiles) return;
  const uint32_t band = tile / (a.row_tiles * kBand);
  const uint32_t band_width = min((uint32_t)kBand, a.column_tiles - band * kBand);
  const uint32_t in_band = tile - band * a.row_tiles * kBand;
  const uint32_t bm = in_band / band_width, bn = band * kBand + in_band % band_width;
  const uint32_t row0 = bm * kSide, col0 = bn * kSide;

  const uint32_t main_steps = a.inner / kBK, steps = a.kt / kBK;   // main_steps is even
  const uint32_t extras_width = a.kt - a.inner;
  // ---- staging addresses: a wave-uniform base that advances with K plus a per-lane offset
  uint32_t a_off[kLoads], e_off[kLoads], p_off[kPairLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const uint32_t in_tile = kStaged * wave + 8 * i + lane / 8;
    const uint32_t piece = (lane % 8) ^ swizzle_of(in_tile);
    a_off[i] = (min(row0 + in_tile, a.rows - 1) * a.kt + 8 * piece) * 2;
    e_off[i] = (min(col0 + in_tile, a.columns - 1) * extras_width + 8 * piece) * 2;
  }
#pragma unroll
  for (int i = 0; i < kPairLoads; ++i) {
    const uint32_t column = 16 * (kPairLoads * wave + i) + lane / 4;
    const uint32_t quarter = (lane % 4) ^ ((column >> 2) & 3u);
    p_off[i] = min(col0 + column, a.columns - 1) * (a.inner / 2) + 16 * quarter;
  }
  auto stage_a = [&](uint32_t buffer, uint32_t step, int i) {
    const uint32_t st = min(step, steps - 1);   // past the end: the last tile again, never used
    const unsigned char *from = (const unsigned char *)a.a + (uint64_t)st * (kBK * 2);
    load_to_lds_16(from + a_off[i], a_tiles + buffer * kTile + (kStaged * wave + 8 * i) * kRowBytes);
  };
  // the weights' fp16 tile of step `step`, one of the steps after the inner ones
  auto stage_extras = [&](uint32_t buffer, uint32_t step, int i) {
    const uint32_t st = min(step, steps - 1) - main_steps;
    const unsigned char *from = (const unsigned char *)a.extras + (uint64_t)st * (kBK * 2);
    load_to_lds_16(from + e_off[i], b_tiles + buffer * kTile + (kStaged * wave + 8 * i) * kRowBytes);
  };
  auto stage_pair = [&](uint32_t pair, int i) {
    const uint32_t pr = min(pair, main_steps / 2 - 1);   // past the end: into the buffer nobody reads
    const unsigned char *from = (const unsigned char *)a.packed + (uint64_t)pr * 64;
    load_to_lds_16(from + p_off[i], pairs + (pair & 1u) * kPair + 16 * (kPairLoads * wave + i) * 64);
  };

  f32x16 acc[kMIR][kMIC];
#pragma unroll
  for (int i = 0; i < kMIR; ++i)
#pragma unroll
    for (int j = 0; j < kMIC; ++j)
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  f16x8 a_op[2][kMIR], b_op[2][kMIC];
  const uint32_t swizzle = swizzle_of(l32);
  // Lane half kh contracts K values [32 kh + 8 s, + 8) of a step in sub-step s (the order in which
  // its 16 bytes of packed words unpack), i.e. piece 4 kh + s of a tile row.
  auto read_a = [&](uint32_t buffer, int s, int set) {
    const unsigned char *at = a_tiles + buffer * kTile + (kQM * wm + l32) * kRowBytes;
    const uint32_t piece = 16 * ((4 * kh + s) ^ swizzle);
#pragma unroll
    for (int i = 0; i < kMIR; ++i)
      a_op[set][i] = __builtin_bit_cast(f16x8, *(const uint4 *)(at + 32 * i * kRowBytes + piece));
  };
  auto read_b = [&](uint32_t buffer, int s, int set) {
    const unsigned char *bt = b_tiles + buffer * kTile + (kQN * wn + l32) * kRowBytes;
    const uint32_t piece = 16 * ((4 * kh + s) ^ swizzle);
#pragma unroll
    for (int j = 0; j < kMIC; ++j)
      b_op[set][j] = __builtin_bit_cast(f16x8, *(const uint4 *)(bt + 32 * j * kRowBytes + piece));
  };
  // ---- the weights of this lane's columns kQN wn + 32 j + l32: 16 bytes of packed words per
  // column and K step (the half kh of the step's group), one word per sub-step, and the columns'
  // scales
  const uint32_t quarter_swizzle = (l32 >> 2) & 3u;
  uint4 words[kMIC], next_words[kMIC];
  auto read_words = [&](uint4 (&to)[kMIC], uint32_t step) {
    const unsigned char *from = pairs + ((step >> 1) & 1u) * kPair + (kQN * wn + l32) * 64 +
                                16 * ((2 * (step & 1u) + kh) ^ quarter_swizzle);
#pragma unroll
    for (int j = 0; j < kMIC; ++j) to[j] = *(const uint4 *)(from + 32 * j * 64);
  };
  const uint32_t groups = a.inner / 64;
  uint32_t scale_off[kMIC];
#pragma unroll
  for (int j = 0; j < kMIC; ++j) scale_off[j] = min(col0 + kQN * wn + 32 * j + l32, a.columns - 1) * groups * 2;
  uint4 scale_block[kMIC], next_block[kMIC];   // bf16 scales of eight groups per column
  auto load_scales = [&](uint4 (&to)[kMIC], uint32_t block) {
    const uint32_t bl = min(block, groups / 8 - 1);
    const unsigned char *from = (const unsigned char *)a.scales + (uint64_t)bl * 16;
#pragma unroll
    for (int j = 0; j < kMIC; ++j) to[j] = *(const uint4 *)(from + scale_off[j]);
  };
  f16x2 scale2[kMIC], next_scale2[kMIC];
  auto pick_scales = [&](f16x2 (&to)[kMIC], uint32_t step) {
    const uint32_t e = step & 7u;   // uniform
#pragma unroll
    for (int j = 0; j < kMIC; ++j) {
      const uint4 v = scale_block[j];
      const uint32_t word = e < 4 ? (e < 2 ? v.x : v.y) : (e < 6 ? v.z : v.w);
      const float scale = __uint_as_float((e & 1u) ? (word & 0xffff0000u) : (word << 16));
      const _Float16 h = (_Float16)scale;
      to[j] = f16x2{h, h};
    }
  };
  uint32_t mask = 0x001e001eu, magic = 0x60006000u;
  asm("" : "+s"(mask), "+v"(magic));   // no instruction: keeps the two constants in registers

  // ---- prologue: activations of step 0, packed words of steps 0..1, scales of groups 0..15;
  // then the operands of the first sub-step
#pragma unroll
  for (int i = 0; i < kLoads; ++i) stage_a(0, 0, i);
#pragma unroll
  for (int i = 0; i < kPairLoads; ++i) stage_pair(0, i);
  load_scales(scale_block, 0);
  load_scales(next_block, 1);
  __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));
  lds_barrier();
  read_words(words, 0);
  pick_scales(scale2, 0);
  read_a(0, 0, 0);
#pragma unroll
  for (int j = 0; j < kMIC; ++j) b_op[0][j] = dequantise_word(words[j].x, scale2[j], mask, magic);
  // One inner step.  On entry the operands of its first sub-step are in registers (set 0).  kOdd:
  // the step's parity (= the LDS buffer its activations are in); kLast: the last inner step, which
  // requests the first fp16 tile of the weights' side and prepares no weights for a next step.
  // Even steps request the packed words of the two steps after the next.  Every request of the
  // step is made at its start; behind the first rows of matrix instructions of a sub-step the
  // lane unpacks the word of the next sub-step of each of its columns (a wave's unpacking runs
  // beside the matrix instructions of the other wave on its SIMD); the matrix instructions of the
  // last sub-step run behind the barrier, covering the latency of the next step's first reads.
  auto inner_step = [&](auto odd_tag, auto last_tag, uint32_t step) {
    constexpr bool kOdd = decltype(odd_tag)::value, kLast = decltype(last_tag)::value;
    constexpr uint32_t buffer = kOdd ? 1u : 0u;
    if (!kLast) {
      if (kOdd && ((step + 1) & 7u) == 0) {   // the next step opens a block of eight groups
#pragma unroll
        for (int j = 0; j < kMIC; ++j) scale_block[j] = next_block[j];
        load_scales(next_block, (step + 1) / 8 + 1);
      }
      pick_scales(next_scale2, step + 1);
      read_words(next_words, step + 1);
    }
#pragma unroll
    for (int i = 0; i < kLoads; ++i) stage_a(buffer ^ 1u, step + 1, i);
    if (kLast) {
#pragma unroll
      for (int i = 0; i < kLoads; ++i) stage_extras(0, main_steps, i);
    } else if (!kOdd) {
#pragma unroll
      for (int i = 0; i < kPairLoads; ++i) stage_pair(step / 2 + 1, i);
    }
#pragma unroll
    for (int s = 0; s < kSub - 1; ++s) {
      __builtin_amdgcn_sched_barrier(0);
      read_a(buffer, s + 1, (s + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < kMIR; ++i) {
#pragma unroll
        for (int j = 0; j < kMIC; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_op[s & 1][i], b_op[s & 1][j], acc[i][j], 0, 0, 0);
        if (i < kMIC) {   // behind row i: the operand of column block i for the next sub-step
          const uint4 v = words[i];
          const uint32_t w = s == 0 ? v.y : s == 1 ? v.z : v.w;
          b_op[(s + 1) & 1][i] = dequantise_word(w, scale2[i], mask, magic);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    static_assert(kMIC <= kMIR, "a row of matrix instructions for every column block");
    __builtin_amdgcn_s_waitcnt(0xc07f);            // lgkmcnt(0): operand reads done
    __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));     // step + 1 has landed
    lds_barrier();
    read_a(buffer ^ 1u, 0, 0);
    if (kLast) read_b(0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kMIR; ++i) {
#pragma unroll
      for (int j = 0; j < kMIC; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_op[1][i], b_op[1][j], acc[i][j], 0, 0, 0);
      if (!kLast && i < kMIC) b_op[0][i] = dequantise_word(next_words[i].x, next_scale2[i], mask, magic);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!kLast) {
#pragma unroll
      for (int j = 0; j < kMIC; ++j) {
        words[j] = next_words[j];
        scale2[j] = next_scale2[j];
      }
    }
  };
  typedef std::integral_constant<bool, false> no;
  typedef std::integral_constant<bool, true> yes;
  uint32_t step = 0;
  for (; step + 2 < main_steps; step += 2) {
    inner_step(no{}, no{}, step);
    inner_step(yes{}, no{}, step + 1);
  }
  inner_step(no{}, no{}, step);
  inner_step(yes{}, yes{}, step + 1);
  // ---- the columns after the inner values: both operands fp16 tiles loaded from memory
  uint32_t buffer = 0;
  for (step = main_steps; step < steps; ++step) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      stage_a(buffer ^ 1u, step + 1, i);
      stage_extras(buffer ^ 1u, step + 1, i);
    }
#pragma unroll
    for (int s = 0; s < kSub - 1; ++s) {
      __builtin_amdgcn_sched_barrier(0);
      read_a(buffer, s + 1, (s + 1) & 1);
      read_b(buffer, s + 1, (s + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < kMIR; ++i)
#pragma unroll
        for (int j = 0; j < kMIC; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_op[s & 1][i], b_op[s & 1][j], acc[i][j], 0, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_waitcnt(wait_vmcnt(0));
    lds_barrier();
    buffer ^= 1u;
    read_a(buffer, 0, 0);   // (after the last step: tiles nobody uses)
    read_b(buffer, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kMIR; ++i)
#pragma unroll
      for (int j = 0; j < kMIC; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_op[1][i], b_op[1][j], acc[i][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);
  lds_barrier();   // the last reads are done before the tile's stores reuse LDS
  store_tile<kQM, kQN, kWN>(a, acc, gemm_lds, row0, col0);
}

}  // namespace

// Whether gemm_q4_kernel takes the product: whole blocks of eight groups per weight row (a lane
// reads eight scales at a time), packed rows and scale rows 16-byte aligned, 32-bit offsets.
static bool packed_form_fits(const QmmProblem &p, uint32_t kt) {
  static const bool disabled = [] {
    const char *env = getenv("FORJA_HIP_GEMM_PREPARED");   // 1: dequantise to fp16 in memory first
    return env && env[0] == '1';
  }();
  if (disabled) return false;
  if (p.inner % 512 != 0 || p.packed.offset % 4 != 0 || p.scales.offset % 8 != 0) return false;
  if ((uint64_t)p.columns * (p.inner / 2) >= (1ull << 32)) return false;
  if ((uint64_t)p.columns * (kt - p.inner) * 2 >= (1ull << 32)) return false;
  return true;
}

bool launch_quant_gemm(fh_backend *backend, const QmmProblem &p, const uint32_t **refused) {
  if (p.inner / 64 > kMaxGroups) return false;
  const uint32_t kt = padded_inner(p.inner);
  // the GEMM addresses its operand matrices with 32-bit byte offsets
  if ((uint64_t)p.rows * kt * 2 >= (1ull << 32) || (uint64_t)p.columns * kt * 2 >= (1ull << 32))
    return false;
  const bool packed_form = packed_form_fits(p, kt);
  const uint64_t a_bytes = ((uint64_t)p.rows * kt * 2 + 255) / 256 * 256;
  // the weights' side: every column of the operand matrix, or only those after the inner values
  const uint64_t b_bytes = ((uint64_t)p.columns * (packed_form ? kt - p.inner : kt) * 2 + 255) / 256 * 256;
  const uint64_t unscale_bytes = ((uint64_t)p.rows * sizeof(float) + 255) / 256 * 256;
  // the weights' operand: a kept copy when there is one (or room for one), else workspace
  PreparedKey key{};
  bool keepable = p.weight_buffers[0] && p.weight_buffers[1] && p.weight_buffers[2];
  bool fresh = true;
  int verdict = -1;
  char *kept = nullptr;
  if (keepable) {
    for (int i = 0; i < 3; ++i) key.buffers[i] = p.weight_buffers[i];
    key.address[0] = (const uint32_t *)p.packed.base + p.packed.offset;
    key.address[1] = (const uint16_t *)p.scales.base + p.scales.offset;
    key.address[2] = (const uint16_t *)p.biases.base + p.biases.offset;
    key.columns = p.columns;
    key.inner = p.inner;
    kept = backend_prepared_weights(backend, key, b_bytes, &fresh, &verdict);
    if (verdict == 1) return false;   // outside the fp16 scheme: the caller's any-range kernel
    // a kept operand whose verdict could not be read is prepared again: the flag is only raised
    // by the preparation
    if (kept && verdict < 0) fresh = true;
  }
  char *ws = backend_workspace(backend, a_bytes + (kept ? 0 : b_bytes) + unscale_bytes + 256);
  if (!ws) return false;
  hipStream_t stream = backend_stream(backend);
  char *b_operand = kept ? kept : ws + a_bytes;
  char *after = ws + a_bytes + (kept ? 0 : b_bytes);
  // the flag of a kept operand lives behind it (and reads zero once the verdict is in)
  uint32_t *flag = kept ? (uint32_t *)(kept + b_bytes) : (uint32_t *)(after + unscale_bytes);
  GemmArgs a{};
  a.a = (const uint16_t *)ws;
  a.b = (const uint16_t *)b_operand;
  a.packed = (const uint32_t *)p.packed.base + p.packed.offset;
  a.scales = (const uint16_t *)p.scales.base + p.scales.offset;
  a.extras = (const uint16_t *)b_operand;
  a.inner = p.inner;
  a.row_unscale = (const float *)after;
  a.kt = kt;
  a.out = p.out.dtype == FH_F32 ? (void *)((float *)p.out.base + p.out.offset)
                                : (void *)((uint16_t *)p.out.base + p.out.offset);
  a.out_row_stride = p.out.stride[0];
  a.out_f32 = p.out.dtype == FH_F32;
  if (p.residual) {
    a.residual = (const uint16_t *)p.residual->base + p.residual->offset;
    a.residual_row_stride = p.residual->stride[0];
  }
  a.row_stores = !a.out_f32 && p.columns % 8 == 0 && p.out.stride[0] % 8 == 0 && p.out.offset % 8 == 0 &&
                 (!p.residual || (p.residual->stride[0] % 8 == 0 && p.residual->offset % 8 == 0));
  a.rows = p.rows;
  a.columns = p.columns;
  // 256 x 256 tiles unless they are fewer than three quarters of the compute units
  const uint64_t large_tiles = (uint64_t)((p.rows + kBM - 1) / kBM) * ((p.columns + kBN - 1) / kBN);
  // (and for at most 128 rows, which would leave half of every large tile empty)
  const bool small_tiles = large_tiles * 4 < 3ull * backend_compute_units(backend) || p.rows <= 128;
  const uint32_t side = small_tiles ? 128 : 256;
  a.row_tiles = (p.rows + side - 1) / side;
  a.column_tiles = (p.columns + side - 1) / side;
  a.refused = flag;
  static bool configured = false;   // raise the dynamic LDS limit once per process
  if (!configured) {
    const struct { const void *kernel; int bytes; } limits[] = {
        {reinterpret_cast<const void *>(&gemm_f16_wide_kernel<kGemmK>), kWideLds},
        {reinterpret_cast<const void *>(&gemm_f16_kernel<kGemmK, kGemmStages, 64>), gemm_lds_bytes(64)},
        {reinterpret_cast<const void *>(&gemm_q4_kernel<2, 4, 128, 64>), kLargeLds},
        {reinterpret_cast<const void *>(&gemm_q4_kernel<2, 2, 64, 64>), kSmallLds}};
    for (const auto &limit : limits) {
      if (hipFuncSetAttribute(limit.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, limit.bytes) != hipSuccess)
        return false;
    }
    configured = true;
  }
  const uint32_t grid = (a.row_tiles * a.column_tiles + 255) / 256 * 256;
  prepare_rows_kernel<<<(p.rows + 3) / 4, 256, 0, stream>>>(
      (const uint16_t *)p.x.base + p.x.offset, p.x.stride[0], p.rows, p.inner, kt, (uint16_t *)ws,
      (float *)after, flag);
  if (!kept || fresh) {
    if (packed_form) {
      const uint64_t threads = (uint64_t)p.columns * ((kt - p.inner) / 8);
      prepare_extras_kernel<<<(uint32_t)((threads + 255) / 256), 256, 0, stream>>>(
          (const uint16_t *)p.scales.base + p.scales.offset, (const uint16_t *)p.biases.base + p.biases.offset,
          p.columns, p.inner, kt, (uint16_t *)b_operand, flag);
    } else {
      const uint64_t weight_threads = (uint64_t)p.columns * (kt / 64) * 8;
      prepare_weights_kernel<<<(uint32_t)((weight_threads + 255) / 256), 256, 0, stream>>>(
          (const uint32_t *)p.packed.base + p.packed.offset,
          (const uint16_t *)p.scales.base + p.scales.offset,
          (const uint16_t *)p.biases.base + p.biases.offset, p.columns, p.inner, kt,
          (uint16_t *)b_operand, flag);
    }
  }
  if (packed_form) {
    if (small_tiles)
      gemm_q4_kernel<2, 2, 64, 64><<<grid, 256, kSmallLds, stream>>>(a);
    else
      gemm_q4_kernel<2, 4, 128, 64><<<grid, 512, kLargeLds, stream>>>(a);
  } else if (small_tiles) {
    gemm_f16_kernel<kGemmK, kGemmStages, 64><<<grid, 256, gemm_lds_bytes(64), stream>>>(a);
  } else {
    gemm_f16_wide_kernel<kGemmK><<<grid, 512, kWideLds, stream>>>(a);
  }
  *refused = (kept && verdict == 0) ? nullptr : flag;
  // the first product over kept weights learns, once, whether they fit the scheme
  if (kept && fresh) backend_prepared_verdict(backend, key);
  return true;
}

}  // namespace fh
