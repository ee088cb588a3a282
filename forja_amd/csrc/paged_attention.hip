// Paged-KV grouped-query attention over a packed ragged batch (block tables + cu_seqlens).
//
// Reference semantics: CpuPagePool::sdpa (crates/forja-cpu/src/paged.rs:161-259) per lane, after
// the lane's new K/V rows were stored at its q_start (execute_paged_append,
// crates/forja-cpu/src/lib.rs:262-306).  Pools are [P, page_tokens, Hkv, D]; a table entry is
// (physical page, generation) and is valid iff page < P and generations[page] == generation.
#include <cstdlib>

#include "fast_kernels.hpp"

namespace fh {

namespace {

__device__ inline float wave_sum(float v) {
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
  return v;
}

__device__ inline float wave_max(float v) {
  for (int offset = 32; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, 64));
  return v;
}

// Lane owning packed token `token`: the l with cu[l] <= token < cu[l+1].
__device__ inline uint32_t find_lane(const uint32_t *cu, uint32_t lanes, uint32_t token) {
  uint32_t lo = 0, hi = lanes;  // invariant: cu[lo] <= token < cu[hi]
  while (hi - lo > 1) {
    uint32_t mid = (lo + hi) >> 1;
    if (cu[mid] <= token)
      lo = mid;
    else
      hi = mid;
  }
  return lo;
}

__device__ inline bool entry_ok(const uint32_t *table, const uint32_t *generations,
                                uint32_t logical_page, uint32_t table_pages,
                                uint32_t physical_pages, uint32_t *physical) {
  if (logical_page >= table_pages) return false;
  uint32_t page = table[2 * (uint64_t)logical_page];
  uint32_t generation = table[2 * (uint64_t)logical_page + 1];
  if (page >= physical_pages) return false;
  if (generations[page] != generation) return false;
  *physical = page;
  return true;
}

// Stores every lane's new K and V rows (thread per (token, element)).  A row whose page entry is
// not authentic is skipped and reported; it is never written.
__global__ void ragged_append_kernel(RaggedAttention p, ErrorSlot *error,
                                     const uint32_t *malformed) {
  if (malformed[0]) return;   // cu_seqlens refused: nothing is stored
  uint32_t key_row = p.kv_heads * p.width, value_row = p.kv_heads * p.value_width;
  uint32_t per_token = key_row + value_row;
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)p.tokens * per_token) return;
  uint32_t token = (uint32_t)(flat / per_token), element = (uint32_t)(flat % per_token);
  const uint32_t *cu = (const uint32_t *)p.cu_seqlens.base + p.cu_seqlens.offset;
  if (token < cu[0] || token >= cu[p.lanes]) return;
  uint32_t lane = find_lane(cu, p.lanes, token);
  if (p.one_row_per_lane && token != cu[lane]) {   // a second row of a lane: the promise is broken
    if (element == 0) report_error(error + (uint64_t)token * p.error_stride, token);
    return;
  }
  if (p.activity.base && ((const uint32_t *)p.activity.base)[p.activity.offset + lane] == 0) return;
  uint64_t position =
      (uint64_t)((const uint32_t *)p.q_starts.base)[p.q_starts.offset + lane] + (token - cu[lane]);
  const uint32_t *table =
      (const uint32_t *)p.tables.base + p.tables.offset + (uint64_t)lane * p.table_pages * 2;
  const uint32_t *generations = (const uint32_t *)p.generations.base + p.generations.offset;
  uint32_t physical;
  uint64_t logical_page = position / p.page_tokens;
  if (logical_page >= p.table_pages ||
      !entry_ok(table, generations, (uint32_t)logical_page, p.table_pages, p.physical_pages,
                &physical)) {
    if (element == 0) report_error(error + (uint64_t)token * p.error_stride, logical_page > 0xffffffffull ? 0xffffffffu
                                                                       : (uint32_t)logical_page);
    return;
  }
  uint64_t pool_row = (uint64_t)physical * p.page_tokens + position % p.page_tokens;
  if (element < key_row) {
    uint32_t head = element / p.width, c = element % p.width;
    float value = load_float_at(p.k_new, p.k_new.offset + token * p.k_new.stride[0] +
                                             head * p.k_new.stride[1] + c * p.k_new.stride[2]);
    store_float_at(p.key_pool, p.key_pool.offset + pool_row * key_row + element, value);
  } else {
    uint32_t e = element - key_row;
    uint32_t head = e / p.value_width, c = e % p.value_width;
    float value = load_float_at(p.v_new, p.v_new.offset + token * p.v_new.stride[0] +
                                             head * p.v_new.stride[1] + c * p.v_new.stride[2]);
    store_float_at(p.value_pool, p.value_pool.offset + pool_row * value_row + e, value);
  }
}

// The same append for rows and pools of one 2-byte dtype whose head rows are 16-byte aligned: a
// thread moves eight elements.
__global__ __launch_bounds__(256) void ragged_append_pieces_kernel(RaggedAttention p, ErrorSlot *error,
                                                                   const uint32_t *malformed) {
  if (malformed[0]) return;   // cu_seqlens refused: nothing is stored
  const uint32_t key_pieces = p.kv_heads * p.width / 8, value_pieces = p.kv_heads * p.value_width / 8;
  const uint32_t per_token = key_pieces + value_pieces;
  const uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)p.tokens * per_token) return;
  const uint32_t token = (uint32_t)(flat / per_token), piece = (uint32_t)(flat % per_token);
  const uint32_t *cu = (const uint32_t *)p.cu_seqlens.base + p.cu_seqlens.offset;
  if (token < cu[0] || token >= cu[p.lanes]) return;
  const uint32_t lane = find_lane(cu, p.lanes, token);
  if (p.one_row_per_lane && token != cu[lane]) {   // a second row of a lane: the promise is broken
    if (piece == 0) report_error(error + (uint64_t)token * p.error_stride, token);
    return;
  }
  if (p.activity.base && ((const uint32_t *)p.activity.base)[p.activity.offset + lane] == 0) return;
  const uint64_t position =
      (uint64_t)((const uint32_t *)p.q_starts.base)[p.q_starts.offset + lane] + (token - cu[lane]);
  const uint32_t *table =
      (const uint32_t *)p.tables.base + p.tables.offset + (uint64_t)lane * p.table_pages * 2;
  const uint32_t *generations = (const uint32_t *)p.generations.base + p.generations.offset;
  uint32_t physical;
  const uint64_t logical_page = position / p.page_tokens;
  if (logical_page >= p.table_pages ||
      !entry_ok(table, generations, (uint32_t)logical_page, p.table_pages, p.physical_pages,
                &physical)) {
    if (piece == 0) report_error(error + (uint64_t)token * p.error_stride, logical_page > 0xffffffffull ? 0xffffffffu
                                                                     : (uint32_t)logical_page);
    return;
  }
  const uint64_t pool_row = (uint64_t)physical * p.page_tokens + position % p.page_tokens;
  const bool key = piece < key_pieces;
  const uint32_t local = key ? piece : piece - key_pieces;
  const uint32_t row_width = key ? p.width : p.value_width;
  const uint32_t head = 8 * local / row_width, c = 8 * local % row_width;
  const View &src = key ? p.k_new : p.v_new;
  const View &pool = key ? p.key_pool : p.value_pool;
  const uint4 value = *(const uint4 *)((const uint16_t *)src.base + src.offset +
                                       (uint64_t)token * src.stride[0] + head * src.stride[1] + c);
  *(uint4 *)((uint16_t *)pool.base + pool.offset + pool_row * ((uint64_t)p.kv_heads * row_width) +
             8 * local) = value;
}

bool append_by_pieces(const RaggedAttention &p) {
  const uint32_t dtype = p.key_pool.dtype;
  if (dtype != FH_BF16 && dtype != FH_F16) return false;
  for (const View *v : {&p.k_new, &p.v_new})
    if (v->dtype != dtype || v->stride[2] != 1 || v->stride[0] % 8 || v->stride[1] % 8 || v->offset % 8)
      return false;
  for (const View *v : {&p.key_pool, &p.value_pool})
    if (v->dtype != dtype || v->offset % 8) return false;
  return p.width % 8 == 0 && p.value_width % 8 == 0;
}

// Any dtype / width: one wave per (token, query head); per-lane online softmax merged at the end.
template <int kMaxDv>
__global__ void ragged_attention_generic_kernel(RaggedAttention p, ErrorSlot *error,
                                                const uint32_t *malformed) {
  __shared__ float q_row[512];
  __shared__ int bad;
  uint32_t token = blockIdx.x / p.query_heads, head = blockIdx.x % p.query_heads;
  uint32_t lane_id = threadIdx.x;
  const uint32_t *cu = (const uint32_t *)p.cu_seqlens.base + p.cu_seqlens.offset;
  uint64_t out_base = p.out.offset + token * p.out.stride[0] + head * p.out.stride[1];
  bool covered = !malformed[0] && token >= cu[0] && token < cu[p.lanes];
  uint32_t lane = covered ? find_lane(cu, p.lanes, token) : 0;
  bool active = covered && !(p.activity.base &&
                             ((const uint32_t *)p.activity.base)[p.activity.offset + lane] == 0);
  if (!active) {
    for (uint32_t c = lane_id; c < p.value_width; c += 64)
      store_float_at(p.out, out_base + c * p.out.stride[2], 0.0f);
    return;
  }
  uint64_t position =
      (uint64_t)((const uint32_t *)p.q_starts.base)[p.q_starts.offset + lane] + (token - cu[lane]);
  uint64_t attended64 = position + 1;
  const uint32_t *table =
      (const uint32_t *)p.tables.base + p.tables.offset + (uint64_t)lane * p.table_pages * 2;
  const uint32_t *generations = (const uint32_t *)p.generations.base + p.generations.offset;
  if (lane_id == 0) bad = 0;
  __syncthreads();
  uint64_t pages = (attended64 + p.page_tokens - 1) / p.page_tokens;
  if (pages > p.table_pages) {
    if (lane_id == 0) {
      report_error(error + (uint64_t)token * p.error_stride, p.table_pages);
      bad = 1;
    }
    pages = p.table_pages;
  }
  for (uint32_t page = lane_id; page < pages; page += 64) {
    uint32_t physical;
    if (!entry_ok(table, generations, page, p.table_pages, p.physical_pages, &physical)) {
      report_error(error + (uint64_t)token * p.error_stride, page);
      bad = 1;
    }
  }
  for (uint32_t c = lane_id; c < p.width; c += 64)
    q_row[c] = load_float_at(p.q, p.q.offset + token * p.q.stride[0] + head * p.q.stride[1] +
                                      c * p.q.stride[2]);
  __syncthreads();
  if (bad) {
    for (uint32_t c = lane_id; c < p.value_width; c += 64)
      store_float_at(p.out, out_base + c * p.out.stride[2], 0.0f);
    return;
  }
  uint32_t attended = (uint32_t)attended64;
  uint32_t kv_head = head / (p.query_heads / p.kv_heads);
  float m = -__builtin_inff(), l = 0.0f;
  float acc[kMaxDv];
  for (int c = 0; c < kMaxDv; ++c) acc[c] = 0.0f;
  for (uint32_t key = lane_id; key < attended; key += 64) {
    uint32_t physical = table[2 * (uint64_t)(key / p.page_tokens)];
    uint64_t pool_row = (uint64_t)physical * p.page_tokens + key % p.page_tokens;
    uint64_t k_at = p.key_pool.offset + (pool_row * p.kv_heads + kv_head) * p.width;
    float score = 0.0f;
    for (uint32_t c = 0; c < p.width; ++c) score += q_row[c] * load_float_at(p.key_pool, k_at + c);
    score *= p.scale;
    float m_new = fmaxf(m, score);
    float correction = m == -__builtin_inff() ? 0.0f : expf(m - m_new);
    float w = expf(score - m_new);
    l = l * correction + w;
    uint64_t v_at = p.value_pool.offset + (pool_row * p.kv_heads + kv_head) * p.value_width;
    for (int c = 0; c < kMaxDv; ++c)
      if ((uint32_t)c < p.value_width)
        acc[c] = acc[c] * correction + w * load_float_at(p.value_pool, v_at + c);
    m = m_new;
  }
  float m_all = wave_max(m);
  float factor = (m == -__builtin_inff()) ? 0.0f : expf(m - m_all);
  float l_all = wave_sum(l * factor);
  for (int c = 0; c < kMaxDv; ++c) {
    if ((uint32_t)c >= p.value_width) break;
    float total = wave_sum(acc[c] * factor);
    if (lane_id == 0) store_float_at(p.out, out_base + c * p.out.stride[2], total / l_all);
  }
}


// ------------------------------------------------- 2-byte pools (bf16 or f16), D = Dv = 128
//
// The pools' dtype is the matrix cores' operand type (kHalf: f16, else bf16).  Queries are of that
// dtype, or f32 (rounded to the pools' dtype once, as they enter the operand registers: an 11-bit
// significand on one factor of a 128-term dot product moves a score by ~1e-4, the 8 bits of bf16
// by ~1e-3, within the bar the reference holds outputs attended from such pools to); outputs are
// written in any float dtype.
//
// Split-KV decode-style attention on the matrix cores, registers only.  One wave owns
// (token, split, kv head): it streams its span of the lane's K/V pages once, 32 tokens per step.
//   S^T = K . Q^T : v_mfma_f32_16x16x32_bf16, M = 16 tokens, N = the kv head's query heads padded
//                   to 16, K = 32 of the 128 head-dim elements per step (4 steps)
//   O^T = V^T . P^T: M = 16 value columns (8 tiles), N = heads, K = 32 tokens
// Operand layouts are chosen so that every global load is a 16-byte piece of a 256-byte K or V
// row and nothing is staged through LDS:
//   * K: lane (token t, group g) reads bytes [64 step + 16 g, +16) of row t - the A operand.
//   * V: MFMA row m of value tile mt is value column 8 m + mt, so lane (m, g) needs columns
//     [8m, 8m+8) - one 16-byte piece - of the 8 tokens in its contraction slots; an 8x8 in-register
//     transpose (v_perm) turns the 8 pieces into the 8 tiles' A operands.
//   * P: the score accumulators of lane (head h, group g) are exactly the B operand of the second
//     product (contraction slot i of group g = token 4g+i of the first half, 16+4g+i-4 of the
//     second), so probabilities never leave registers.
// Softmax runs in the exp2 domain with one running maximum per head.  HBM-bound: every K/V byte
// is read once; per-split partial (m, l, O) are merged by ragged_reduce_kernel.

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr uint32_t kMinSplitTokens = 128, kMaxSplitTokens = 1024;  // split length bounds
// Groups of several query tokens (prefill) are many and each split of theirs costs a merge of
// `members x heads` partial rows: they are split only beyond this many keys.
constexpr uint32_t kPrefillSplitTokens = 2048;
constexpr uint32_t kTargetItems = 1024;  // (token, split) items wanted per launch of grouped tokens
constexpr uint32_t kTile = 32;          // tokens per inner step

struct TokenPlan {
  uint32_t lane, attended, chunk, splits;  // splits == 0: token produces zeros
  uint32_t leader, members;                // first token of this token's group, group size
};

struct FastRagged {
  const void *q;       // q_dtype elements
  const uint16_t *key_pool, *value_pool;
  void *out;           // out_dtype elements
  uint32_t q_dtype, out_dtype;   // strides below count elements of these
  uint32_t pool_half;            // pools are f16 (else bf16)
  const uint32_t *tables, *generations, *cu, *starts, *activity;
  float *partial_o;    // [T, S, Hq, 128]
  float2 *partial_ml;  // [T, S, Hq]
  uint32_t *bad;       // [T]
  TokenPlan *plans;    // [T]
  uint2 *items;        // [T * S] (group leader token, split) of every live split, compacted
  uint32_t *item_count;   // [0] work items, [1] tokens the merge kernel has work for,
                          // [2] non-zero: cu_seqlens was refused
  uint32_t *merge_tokens; // [T] those tokens (several splits, or a zero row to write)
  uint64_t q_stride_t, q_stride_h, out_stride_t, out_stride_h;
  uint32_t tokens, lanes, query_heads, kv_heads, group, page_tokens, physical_pages, table_pages,
      max_splits, split_tokens;
  // Workgroups of the decode kernel the device holds at once (0: not a decode batch).  The plan
  // sizes the splits so that the items fill these places once.
  uint32_t item_slots;
  // Query tokens of one lane are processed `group_tokens` at a time (they share the lane's K/V
  // stream): 1 for decode batches (a wave per kv head), kSharedWaves * kSharedTiles * (16 / group)
  // for prefill batches (a workgroup per kv head).
  uint32_t group_tokens;
  float scale_log2;
  // Single-lane form (Op::PagedSdpa / Op::PagedSdpaAppend): cu == nullptr, every token belongs
  // to lane 0 whose first query sits at `one_start`; `fixed_attended` != 0 disables the causal
  // limit (every row attends exactly that many keys).
  uint32_t one_start, fixed_attended;
  uint32_t error_stride;  // failures of token t go to error[t * error_stride]
  // In-kernel append (decode batches with one query row per lane): the workgroup of a lane's last
  // split stores the lane's new key and value row before it attends.  k_new / v_new are
  // [T, Hkv, 128] with unit innermost stride; append failures are recorded `append_error_back`
  // records before the attention's.
  const void *k_new, *v_new;   // q_dtype elements
  uint64_t kn_stride_t, kn_stride_h, vn_stride_t, vn_stride_h;
  uint32_t append_in_kernel, append_error_back;
  uint32_t promised;   // one query row per lane, vouched for by the caller: verified by the plan
};

// Splits of a group whose longest member attends `longest` keys: as few as keep each within
// `split_tokens`, of equal length rounded up to whole tiles.
__device__ inline void split_layout(uint32_t longest, uint32_t members, uint32_t split_tokens,
                                    uint32_t max_splits, uint32_t *chunk, uint32_t *splits) {
  if (members > 1 && split_tokens < kPrefillSplitTokens) split_tokens = kPrefillSplitTokens;
  uint32_t want = (longest + split_tokens - 1) / split_tokens;
  if (want > max_splits) want = max_splits;
  const uint32_t even = (longest + want - 1) / want;
  *chunk = (even + kTile - 1) / kTile * kTile;
  *splits = (longest + *chunk - 1) / *chunk;
}

// Work decomposition of one token.  Tokens of a lane are grouped `group_tokens` at a time; a
// group shares its split layout, sized for its last (longest) member, and every member carries
// its own causal limit in `attended`.  attended == 0 with splits == 0 and lane == 0xffffffff
// marks a token whose context exceeds its table (reported as a bad page).
__device__ inline TokenPlan plan_token(const FastRagged &p, uint32_t token, uint32_t split_tokens) {
  TokenPlan plan{0, 0, 0, 0, token, 1};
  uint64_t attended, first_of_lane, lane_tokens, start;
  if (p.cu == nullptr) {
    if (p.activity && p.activity[0] == 0) return plan;
    first_of_lane = 0;
    lane_tokens = p.tokens;
    start = p.one_start;
  } else {
    if (token < p.cu[0] || token >= p.cu[p.lanes]) return plan;
    plan.lane = find_lane(p.cu, p.lanes, token);
    if (p.activity && p.activity[plan.lane] == 0) return plan;
    first_of_lane = p.cu[plan.lane];
    lane_tokens = p.cu[plan.lane + 1] - first_of_lane;
    start = p.starts[plan.lane];
    if (p.promised && lane_tokens > 1) {   // the caller's promise does not hold
      plan.lane = 0xfffffffeu;
      return plan;
    }
  }
  const uint64_t index = token - first_of_lane;
  const uint64_t leader = index - index % p.group_tokens;
  const uint64_t last = min(leader + p.group_tokens, lane_tokens) - 1;
  attended = p.fixed_attended ? p.fixed_attended : start + index + 1;
  const uint64_t group_attended = p.fixed_attended ? p.fixed_attended : start + last + 1;
  if (group_attended > (uint64_t)p.table_pages * p.page_tokens) {
    plan.lane = 0xffffffffu;
    return plan;
  }
  plan.leader = (uint32_t)(first_of_lane + leader);
  plan.members = (uint32_t)(last - leader + 1);
  plan.attended = (uint32_t)attended;
  split_layout((uint32_t)group_attended, plan.members, split_tokens, p.max_splits, &plan.chunk,
               &plan.splits);
  return plan;
}

// One workgroup: plans every token, clears the per-token failure flags and lists the live
// (group leader, split) work items longest first (by split length, 32-token classes), so that the
// hardware, which starts workgroups in list order, ends the launch on its shortest items.
constexpr uint32_t kSizeClasses = 65;   // split length / 32, clamped

// Lowest lane whose token range breaks the cu_seqlens contract (non-decreasing, ending inside
// the packed batch), over the lanes this thread looks at; 0xffffffff when they all keep it.
__device__ inline uint32_t first_malformed_lane(const uint32_t *cu, uint32_t lanes, uint32_t tokens,
                                                uint32_t first, uint32_t step) {
  for (uint32_t lane = first; lane < lanes; lane += step)
    if (cu[lane + 1] < cu[lane] || cu[lane + 1] > tokens) return lane;
  return 0xffffffffu;
}

// For the kernels that do not go through a work plan: raises `flag[0]` and reports the lane when
// cu_seqlens is refused.
__global__ __launch_bounds__(256) void ragged_validate_kernel(const uint32_t *cu, uint32_t lanes,
                                                              uint32_t tokens, uint32_t *flag,
                                                              ErrorSlot *error) {
  __shared__ uint32_t lowest;
  if (threadIdx.x == 0) lowest = 0xffffffffu;
  __syncthreads();
  const uint32_t mine = first_malformed_lane(cu, lanes, tokens, threadIdx.x, 256);
  if (mine != 0xffffffffu) atomicMin(&lowest, mine);
  __syncthreads();
  if (threadIdx.x == 0) {
    flag[0] = lowest != 0xffffffffu;
    if (lowest != 0xffffffffu) report_error(error, lowest);
  }
}

__global__ __launch_bounds__(256) void ragged_plan_kernel(FastRagged p, ErrorSlot *error) {
  __shared__ uint32_t class_items[kSizeClasses];   // items per class, then the class's cursor
  __shared__ unsigned long long total_attended;
  __shared__ uint32_t merge_count, malformed_lane, longest_keys, trial_items;
  constexpr uint32_t kKeysHeld = 4096;   // tokens whose key counts the split search keeps in LDS
  __shared__ uint32_t keys_held[kKeysHeld];
  for (uint32_t c = threadIdx.x; c < kSizeClasses; c += 256) class_items[c] = 0;
  if (threadIdx.x == 0) {
    total_attended = 0;
    longest_keys = 0;
    merge_count = 0;
    malformed_lane = 0xffffffffu;
  }
  __syncthreads();
  // cu_seqlens is device data nobody has looked at: token ranges that run backwards or past the
  // packed batch would send the grouped kernels beyond q, out and the plan itself.  A refused
  // cu_seqlens fails the whole dispatch: every row reads zero, nothing is appended, and the
  // lowest offending lane is reported.
  if (p.cu != nullptr) {
    const uint32_t mine = first_malformed_lane(p.cu, p.lanes, p.tokens, threadIdx.x, 256);
    if (mine != 0xffffffffu) atomicMin(&malformed_lane, mine);
    __syncthreads();
    if (malformed_lane != 0xffffffffu) {
      for (uint32_t token = threadIdx.x; token < p.tokens; token += 256) {
        p.bad[token] = 1;
        p.plans[token] = TokenPlan{0, 0, 0, 0, token, 1};
        p.merge_tokens[token] = token;
      }
      if (threadIdx.x == 0) {
        report_error(error, malformed_lane);
        p.item_count[0] = 0;
        p.item_count[1] = p.tokens;
        p.item_count[2] = 1;
      }
      return;
    }
  }
  if (threadIdx.x == 0) p.item_count[2] = 0;
  // Split length: long enough that a wave's fixed start-up cost (plan, table, query) is small
  // against its stream, short enough that the batch still yields enough work items.
  uint32_t split_tokens = p.split_tokens;
  if (split_tokens == 0) {
    unsigned long long mine = 0;
    uint32_t mine_longest = 0;
    for (uint32_t token = threadIdx.x; token < p.tokens; token += 256) {
      const TokenPlan whole = plan_token(p, token, 1u << 30);
      // the keys of the token's group in whole tiles, for the search below: a decode batch has
      // groups of one token
      const uint32_t keys = whole.splits ? whole.chunk : 0;
      if (token < kKeysHeld) keys_held[token] = keys;
      else if (p.item_slots) p.plans[token].chunk = keys;
      mine += whole.attended / p.group_tokens;
      mine_longest = max(mine_longest, keys);
    }
    for (int offset = 32; offset > 0; offset >>= 1) mine += __shfl_xor(mine, offset, 64);
    if ((threadIdx.x & 63) == 0) atomicAdd(&total_attended, mine);
    atomicMax(&longest_keys, mine_longest);
    __syncthreads();
    if (p.item_slots == 0) {
      unsigned long long per_item = total_attended / kTargetItems;
      split_tokens = (uint32_t)((per_item + kTile - 1) / kTile * kTile);
      if (split_tokens < kMinSplitTokens) split_tokens = kMinSplitTokens;
      if (split_tokens > kMaxSplitTokens) split_tokens = kMaxSplitTokens;
    } else {
      // Decode batches: the shortest split length whose items all find a place on the device at
      // once.  One item per place costs each place one start-up and leaves no second, partly
      // filled round behind (128 lanes of 256 to 32768 keys: 311 us against 330 us for any
      // length that needs two rounds).  When the lanes alone outnumber the places no length
      // achieves that, and one far above the even share would leave the longest lanes running
      // alone at the end: then the even share of a place is the length.
      const unsigned long long share = (total_attended + p.item_slots - 1) / p.item_slots;
      uint32_t even = (uint32_t)((share + kTile - 1) / kTile * kTile);
      if (even < kMinSplitTokens) even = kMinSplitTokens;
      uint32_t low = even / kTile, high = max(longest_keys, even) / kTile;   // in tiles
      while (low < high) {   // smallest length in [low, high] with at most item_slots items
        const uint32_t middle = (low + high) / 2;
        if (threadIdx.x == 0) trial_items = 0;
        __syncthreads();
        uint32_t items = 0;
        for (uint32_t token = threadIdx.x; token < p.tokens; token += 256) {
          const uint32_t keys = token < kKeysHeld ? keys_held[token] : p.plans[token].chunk;
          if (keys == 0) continue;
          uint32_t chunk, splits;
          split_layout(keys, 1, middle * kTile, p.max_splits, &chunk, &splits);
          items += splits;
        }
        if (items) atomicAdd(&trial_items, items);
        __syncthreads();
        const bool fits = trial_items <= p.item_slots;
        __syncthreads();
        if (fits) high = middle; else low = middle + 1;
      }
      split_tokens = low * kTile <= 2 * even ? low * kTile : even;
    }
  }
  auto class_of = [](const TokenPlan &plan) {
    const uint32_t c = plan.chunk / kTile;
    return c < kSizeClasses ? c : kSizeClasses - 1;
  };
  for (uint32_t token = threadIdx.x; token < p.tokens; token += 256) {
    TokenPlan plan = plan_token(p, token, split_tokens);
    uint32_t bad = 0;
    if (plan.lane == 0xffffffffu) {
      report_error(error + (uint64_t)token * p.error_stride, p.table_pages);
      bad = 1;
      plan.lane = 0;
    } else if (plan.lane == 0xfffffffeu) {
      report_error(error + (uint64_t)token * p.error_stride, token);
      bad = 1;
      plan.lane = 0;
    }
    p.bad[token] = bad;
    p.plans[token] = plan;
    if (plan.leader == token && plan.splits) atomicAdd(&class_items[class_of(plan)], plan.splits);
    // tokens with a single split are finished by the attention kernel itself
    if (plan.splits != 1 || bad) p.merge_tokens[atomicAdd(&merge_count, 1u)] = token;
  }
  __syncthreads();
  if (threadIdx.x == 0) {   // class counts -> first item of each class, longest class first
    uint32_t running = 0;
    for (int c = (int)kSizeClasses - 1; c >= 0; --c) {
      const uint32_t count = class_items[c];
      class_items[c] = running;
      running += count;
    }
    p.item_count[0] = running;
    p.item_count[1] = merge_count;
  }
  __syncthreads();
  for (uint32_t token = threadIdx.x; token < p.tokens; token += 256) {
    const TokenPlan plan = p.plans[token];
    if (plan.leader != token || plan.splits == 0) continue;
    const uint32_t first = atomicAdd(&class_items[class_of(plan)], plan.splits);
    for (uint32_t s = 0; s < plan.splits; ++s) p.items[first + s] = make_uint2(token, s);
  }
}

__device__ inline uint32_t pack_bf16(float lo, float hi) {
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

__device__ inline uint32_t pack_f16(float lo, float hi) {
  f16x2 v = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

// Two values as a pair of matrix-core operand elements.
template <bool kHalf>
__device__ inline uint32_t pack_operand(float lo, float hi) {
  return kHalf ? pack_f16(lo, hi) : pack_bf16(lo, hi);
}

template <bool kHalf>
__device__ inline f32x4 mfma_16x16x32(const uint4 &a, const uint4 &b, const f32x4 &c) {
  if constexpr (kHalf)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// Eight query elements from `element` as operand words.  An f32 query is rounded to the pools'
// dtype; against f16 pools an element beyond the f16 range is held at the largest finite f16 (a
// NaN stays a NaN): the scores stay finite, as the reference's.
template <bool kHalf, bool kMixed>
__device__ inline uint4 load_query(const FastRagged &p, uint64_t element) {
  if (!kMixed || p.q_dtype != FH_F32) return *(const uint4 *)((const uint16_t *)p.q + element);
  const float4 lo = *(const float4 *)((const float *)p.q + element);
  const float4 hi = *(const float4 *)((const float *)p.q + element + 4);
  auto held = [](float v) { return kHalf && fabsf(v) > 65504.0f ? copysignf(65504.0f, v) : v; };
  return make_uint4(pack_operand<kHalf>(held(lo.x), held(lo.y)), pack_operand<kHalf>(held(lo.z), held(lo.w)),
                    pack_operand<kHalf>(held(hi.x), held(hi.y)), pack_operand<kHalf>(held(hi.z), held(hi.w)));
}

// Four consecutive output elements from `element` (a multiple of 4 on a row whose strides are).
// kMixed false: queries and outputs are of the pools' dtype, known when the kernel is compiled
// (the attention kernels have no registers to spare for the choice).
template <bool kHalf, bool kMixed>
__device__ inline void store_out4(const FastRagged &p, uint64_t element, float a, float b, float c,
                                  float d) {
  if (!kMixed) {
    *(uint2 *)((uint16_t *)p.out + element) =
        make_uint2(pack_operand<kHalf>(a, b), pack_operand<kHalf>(c, d));
    return;
  }
  if (p.out_dtype == FH_F32)
    *(float4 *)((float *)p.out + element) = make_float4(a, b, c, d);
  else if (p.out_dtype == FH_F16)
    *(uint2 *)((uint16_t *)p.out + element) = make_uint2(pack_f16(a, b), pack_f16(c, d));
  else
    *(uint2 *)((uint16_t *)p.out + element) = make_uint2(pack_bf16(a, b), pack_bf16(c, d));
}

__device__ inline uint32_t dword_of(const uint4 &v, int index) {
  return index == 0 ? v.x : (index == 1 ? v.y : (index == 2 ? v.z : v.w));
}

// Zero output rows of `count` tokens from `first` for the query heads of one kv head (a wave's
// duty when it refuses a page and no merge will follow: the token has a single split).
template <bool kMixed>
__device__ inline void zero_head_rows(const FastRagged &p, uint32_t first, uint32_t count,
                                      uint32_t kv_head, uint32_t lane) {
  for (uint32_t member = 0; member < count; ++member)
    for (uint32_t head = kv_head * p.group; head < (kv_head + 1) * p.group; ++head) {
      const uint64_t element =
          (uint64_t)(first + member) * p.out_stride_t + (uint64_t)head * p.out_stride_h + 2 * lane;
      if (kMixed && p.out_dtype == FH_F32)
        *(uint2 *)((float *)p.out + element) = make_uint2(0, 0);
      else
        *(uint32_t *)((uint16_t *)p.out + element) = 0;
    }
}

struct TileRegs {
  uint4 k[2][4];
  uint4 v[8];
};

struct LaneConst {
  uint32_t k_offset;  // elements from the first row of a 16-token half to this lane's K piece
  uint32_t v_offset;  // likewise for slot 0 of this lane's V pieces
  uint32_t row_elems; // elements per pool token row (Hkv * 128)
};

// Issues the 16 loads of one 32-token tile.  `physical` holds this lane's authenticated page of
// the current 64-page group; a 16-token half never straddles a page, so each half is addressed
// as a wave-uniform base plus a per-lane 32-bit offset.  kMasked tiles (the last, partial tile
// of a split) load zeros past `end`: unused pool slots may hold anything and 0 * NaN would
// poison the sum.
template <bool kMasked>
__device__ inline void load_tile(const FastRagged &p, TileRegs &r, uint32_t tile0, uint32_t end,
                                 uint32_t page0, uint32_t physical, const LaneConst &lc,
                                 uint32_t hl, uint32_t g) {
  const uint32_t pt = p.page_tokens;
  for (int sub = 0; sub < 2; ++sub) {
    const uint32_t tok0 = tile0 + 16 * sub;
    if (kMasked && tok0 >= end) {
      for (int step = 0; step < 4; ++step) r.k[sub][step] = make_uint4(0, 0, 0, 0);
      for (int i = 0; i < 4; ++i) r.v[4 * sub + i] = make_uint4(0, 0, 0, 0);
      continue;
    }
    const uint32_t page =
        __builtin_amdgcn_readfirstlane(__shfl(physical, (int)(tok0 / pt - page0), 64));
    const uint64_t row0 = (uint64_t)page * pt + tok0 % pt;
    const uint16_t *k_base = p.key_pool + row0 * lc.row_elems;
    const uint16_t *v_base = p.value_pool + row0 * lc.row_elems;
    for (int step = 0; step < 4; ++step) {
      r.k[sub][step] = stream_load(k_base + lc.k_offset + 32 * step);
      if (kMasked && tok0 + hl >= end) r.k[sub][step] = make_uint4(0, 0, 0, 0);
    }
    for (int i = 0; i < 4; ++i) {
      r.v[4 * sub + i] = stream_load(v_base + lc.v_offset + i * lc.row_elems);
      if (kMasked && tok0 + 4 * g + i >= end) r.v[4 * sub + i] = make_uint4(0, 0, 0, 0);
    }
  }
}

struct Softmax {
  float m, l;
};

// Scores, online softmax and the value product for one tile of 32 keys against NT query tiles
// (16 query rows each: this lane holds row hl of every tile).  `limit[nt]` is the first key the
// lane's row of tile nt may NOT attend (0 for an unused row); with kMasked false every key of
// the tile is below every limit.
template <int NT, bool kMasked, bool kHalf>
__device__ inline void consume_tile(const TileRegs &cur, const uint4 (&q_reg)[NT][4],
                                    f32x4 (&o)[NT][8], Softmax (&sm)[NT], uint32_t tile0,
                                    const uint32_t (&limit)[NT], float scale_log2, uint32_t g) {
  uint4 p_reg[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float s_val[8];
    for (int sub = 0; sub < 2; ++sub) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      for (int step = 0; step < 4; ++step)
        acc = mfma_16x16x32<kHalf>(cur.k[sub][step], q_reg[nt][step], acc);
      for (int j = 0; j < 4; ++j) {
        s_val[4 * sub + j] = acc[j] * scale_log2;
        if (kMasked && tile0 + 16 * sub + 4 * g + j >= limit[nt]) s_val[4 * sub + j] = -__builtin_inff();
      }
    }
    float tile_max = s_val[0];
    for (int i = 1; i < 8; ++i) tile_max = fmaxf(tile_max, s_val[i]);
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));
    const float m_new = fmaxf(sm[nt].m, tile_max);
    // a row with nothing to attend yet keeps m = -inf; subtract 0 instead so that exp2(-inf) = 0
    const float m_safe = (kMasked && m_new == -__builtin_inff()) ? 0.0f : m_new;
    float p_val[8], p_sum = 0.0f;
    for (int i = 0; i < 8; ++i) {
      p_val[i] = __builtin_amdgcn_exp2f(s_val[i] - m_safe);
      p_sum += p_val[i];
    }
    // The running maximum settles after a few tiles; skip the rescale when no lane's moved.
    if (__any(m_new != sm[nt].m)) {
      const float alpha = __builtin_amdgcn_exp2f(sm[nt].m - m_safe);   // 0 while m is -inf
      sm[nt].l *= alpha;
      for (int mt = 0; mt < 8; ++mt)
        for (int j = 0; j < 4; ++j) o[nt][mt][j] *= alpha;
      sm[nt].m = m_new;
    }
    sm[nt].l += p_sum;
    p_reg[nt] = make_uint4(pack_operand<kHalf>(p_val[0], p_val[1]), pack_operand<kHalf>(p_val[2], p_val[3]),
                           pack_operand<kHalf>(p_val[4], p_val[5]), pack_operand<kHalf>(p_val[6], p_val[7]));
  }
  // O^T += V^T . P^T.  Tile mt takes element mt of each of the lane's 8 token pieces; the
  // transposed value operand serves all NT query tiles.
  for (int mt = 0; mt < 8; ++mt) {
    const uint32_t selector = (mt & 1) ? 0x07060302u : 0x05040100u;
    uint32_t a_words[4];
    for (int pair = 0; pair < 4; ++pair)
      a_words[pair] = __builtin_amdgcn_perm(dword_of(cur.v[2 * pair + 1], mt >> 1),
                                            dword_of(cur.v[2 * pair], mt >> 1), selector);
    const uint4 a_reg = make_uint4(a_words[0], a_words[1], a_words[2], a_words[3]);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      o[nt][mt] = mfma_16x16x32<kHalf>(a_reg, p_reg[nt], o[nt][mt]);
  }
}

// NT query tiles of 16 rows per wave: row hl of tile nt is (query token nt * per_tile + hl / group
// of the item's group, head hl % group of the kv head), per_tile = 16 / group.
template <int NT, bool kHalf, bool kMixed>
__device__ inline void ragged_attention_body(const FastRagged &p, ErrorSlot *error) {
  // a workgroup is one work item; its waves take one kv head each, so the slices of a K/V page
  // (one 256-byte piece of every token row per kv head) are requested close together in time
  const uint32_t lane = threadIdx.x & 63, hl = lane & 15, g = lane >> 4;
  const uint32_t item = blockIdx.x, kv_head = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (item >= p.item_count[0] || kv_head >= p.kv_heads) return;
  const uint2 work = p.items[item];
  const uint32_t leader = work.x, split = work.y;
  const TokenPlan plan = p.plans[leader];
  const uint32_t members = NT == 1 ? 1 : plan.members;
  // the group's split layout is sized for its last member
  const uint32_t longest =
      (NT == 1 || p.fixed_attended) ? plan.attended : plan.attended + members - 1;
  const uint32_t begin = split * plan.chunk;
  const uint32_t end = min(longest, begin + plan.chunk);
  const uint32_t pt = p.page_tokens;
  const uint32_t *table = p.tables + (uint64_t)plan.lane * p.table_pages * 2;
  if (NT == 1 && p.append_in_kernel && split + 1 == plan.splits) {
    // This wave's kv head of the lane's new row goes into the pool before anything is read: the
    // row sits at the last attended position, which only this workgroup's range contains.
    const uint32_t position = plan.attended - 1, logical = position / pt;
    uint32_t physical;
    if (entry_ok(table, p.generations, logical, p.table_pages, p.physical_pages, &physical)) {
      const uint64_t pool_row = (uint64_t)physical * pt + position % pt;
      const uint64_t at = (pool_row * p.kv_heads + kv_head) * 128;
      const uint64_t k_at = (uint64_t)leader * p.kn_stride_t + (uint64_t)kv_head * p.kn_stride_h;
      const uint64_t v_at = (uint64_t)leader * p.vn_stride_t + (uint64_t)kv_head * p.vn_stride_h;
      uint32_t k_pair, v_pair;   // this lane's two elements of the row, in the pools' dtype
      if (kMixed && p.q_dtype == FH_F32) {
        // rounded exactly as a store into the pool rounds (nearest even, NaN kept quiet)
        const float2 k_two = ((const float2 *)((const float *)p.k_new + k_at))[lane];
        const float2 v_two = ((const float2 *)((const float *)p.v_new + v_at))[lane];
        k_pair = kHalf ? f32_to_f16(k_two.x) | (uint32_t)f32_to_f16(k_two.y) << 16
                       : f32_to_bf16(k_two.x) | (uint32_t)f32_to_bf16(k_two.y) << 16;
        v_pair = kHalf ? f32_to_f16(v_two.x) | (uint32_t)f32_to_f16(v_two.y) << 16
                       : f32_to_bf16(v_two.x) | (uint32_t)f32_to_bf16(v_two.y) << 16;
      } else {
        k_pair = ((const uint32_t *)((const uint16_t *)p.k_new + k_at))[lane];
        v_pair = ((const uint32_t *)((const uint16_t *)p.v_new + v_at))[lane];
      }
      ((uint32_t *)(const_cast<uint16_t *>(p.key_pool) + at))[lane] = k_pair;
      ((uint32_t *)(const_cast<uint16_t *>(p.value_pool) + at))[lane] = v_pair;
      // the loads below come from the same wave, after the stores have completed
      __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
    } else if (lane == 0) {
      // not written; the page walk below meets the same entry and ends the workgroup
      report_error(error - p.append_error_back + (uint64_t)leader * p.error_stride, logical);
    }
  }
  LaneConst lc;
  lc.row_elems = p.kv_heads * 128;
  lc.k_offset = (hl * p.kv_heads + kv_head) * 128 + 8 * g;
  lc.v_offset = (4 * g * p.kv_heads + kv_head) * 128 + 8 * hl;

  // Query operands and causal limits of this lane's rows.
  const uint32_t per_tile = NT == 1 ? 1 : 16 / p.group;
  uint4 q_reg[NT][4];
  uint32_t limit[NT], member_of[NT];
  const uint32_t head = kv_head * p.group + (NT == 1 ? hl : hl % p.group);
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    member_of[nt] = NT == 1 ? 0 : nt * per_tile + hl / p.group;
    const bool used = hl < per_tile * p.group && member_of[nt] < members;
    // (a decode row that is only padding keeps the uniform limit: its query is zero anyway)
    limit[nt] = NT == 1 ? end
                        : (!used ? 0
                                 : min(end, p.fixed_attended ? plan.attended
                                                             : plan.attended + member_of[nt]));
    const uint64_t q_row = (uint64_t)(leader + member_of[nt]) * p.q_stride_t +
                           (uint64_t)head * p.q_stride_h;
    for (int step = 0; step < 4; ++step) {  // same head-dim slice per (step, g) as the K operand
      q_reg[nt][step] = make_uint4(0, 0, 0, 0);
      if (used) q_reg[nt][step] = load_query<kHalf, kMixed>(p, q_row + 32 * step + 8 * g);
    }
    if (NT > 1 && !used) member_of[nt] = 0xffffffffu;
  }
  // keys below `unmasked_end` are attended by every used row
  const uint32_t unmasked_end = NT == 1 ? end : min(end, plan.attended);
  f32x4 o[NT][8];
  Softmax sm[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    for (int mt = 0; mt < 8; ++mt) o[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    sm[nt] = Softmax{-__builtin_inff(), 0.0f};
  }

  const uint32_t first_page = begin / pt, last_page = (end - 1) / pt;
  for (uint32_t page0 = first_page; page0 <= last_page; page0 += 64) {
    // Authenticate up to 64 table entries at once; nothing is dereferenced through a bad one.
    uint32_t my_page = page0 + lane, physical = 0;
    bool mine = my_page <= last_page, ok = true;
    if (mine) {
      uint32_t page = table[2 * (uint64_t)my_page], generation = table[2 * (uint64_t)my_page + 1];
      ok = page < p.physical_pages && p.generations[page] == generation;
      physical = page;
    }
    unsigned long long bad_mask = __ballot(mine && !ok);
    if (bad_mask) {
      if (lane == (uint32_t)__ffsll((long long)bad_mask) - 1) {
        report_error(error + (uint64_t)leader * p.error_stride, my_page);
        for (uint32_t member = 0; member < members; ++member) p.bad[leader + member] = 1;
      }
      if (plan.splits == 1) zero_head_rows<kMixed>(p, leader, members, kv_head, lane);
      return;
    }
    const uint32_t tok_lo = max(begin, page0 * pt);
    const uint32_t tok_hi = (uint32_t)min((uint64_t)end, ((uint64_t)page0 + 64) * pt);
    // Tiles wholly below unmasked_end need no bounds logic at all; the rest (at most a few
    // around the causal diagonal and the end of the split) take the masked forms.
    const uint32_t plain_keys = unmasked_end > tok_lo ? min(tok_hi, unmasked_end) - tok_lo : 0;
    const uint32_t full_hi = tok_lo + plain_keys / kTile * kTile;
    TileRegs cur;
    if (tok_lo + kTile <= tok_hi)
      load_tile<false>(p, cur, tok_lo, end, page0, physical, lc, hl, g);
    else
      load_tile<true>(p, cur, tok_lo, end, page0, physical, lc, hl, g);
    // Software pipeline: the next tile's loads are in flight while this one is consumed.
    if constexpr (NT == 1) {
      // a decode split is plain tiles followed by at most one masked tile
      for (uint32_t tile0 = tok_lo; tile0 < full_hi; tile0 += kTile) {
        TileRegs nxt;
        const uint32_t next0 = tile0 + kTile;
        if (next0 < full_hi)
          load_tile<false>(p, nxt, next0, end, page0, physical, lc, hl, g);
        else if (next0 < tok_hi)
          load_tile<true>(p, nxt, next0, end, page0, physical, lc, hl, g);
        consume_tile<NT, false, kHalf>(cur, q_reg, o, sm, tile0, limit, p.scale_log2, g);
        if (next0 < tok_hi) cur = nxt;
      }
      if (full_hi < tok_hi)
        consume_tile<NT, true, kHalf>(cur, q_reg, o, sm, full_hi, limit, p.scale_log2, g);
    } else {
      for (uint32_t tile0 = tok_lo; tile0 < tok_hi; tile0 += kTile) {
        TileRegs nxt;
        const uint32_t next0 = tile0 + kTile;
        if (next0 + kTile <= tok_hi)
          load_tile<false>(p, nxt, next0, end, page0, physical, lc, hl, g);
        else if (next0 < tok_hi)
          load_tile<true>(p, nxt, next0, end, page0, physical, lc, hl, g);
        if (tile0 < full_hi)
          consume_tile<NT, false, kHalf>(cur, q_reg, o, sm, tile0, limit, p.scale_log2, g);
        else
          consume_tile<NT, true, kHalf>(cur, q_reg, o, sm, tile0, limit, p.scale_log2, g);
        if (next0 < tok_hi) cur = nxt;
      }
    }
  }
  // Lane (row hl, group g) holds value columns 32g + 8j + mt of its rows.
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float m_run = sm[nt].m, l_run = sm[nt].l;
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (NT == 1 ? hl >= p.group : member_of[nt] == 0xffffffffu) continue;
    const uint32_t token = leader + member_of[nt];
    if (plan.splits == 1) {
      float inv = 1.0f / l_run;
      const uint64_t out_row = (uint64_t)token * p.out_stride_t + (uint64_t)head * p.out_stride_h;
      for (int j = 0; j < 4; ++j) {
        store_out4<kHalf, kMixed>(p, out_row + 32 * g + 8 * j, o[nt][0][j] * inv, o[nt][1][j] * inv,
                   o[nt][2][j] * inv, o[nt][3][j] * inv);
        store_out4<kHalf, kMixed>(p, out_row + 32 * g + 8 * j + 4, o[nt][4][j] * inv, o[nt][5][j] * inv,
                   o[nt][6][j] * inv, o[nt][7][j] * inv);
      }
      continue;
    }
    uint64_t slot = ((uint64_t)token * p.max_splits + split) * p.query_heads + head;
    float *po = p.partial_o + slot * 128 + 32 * g;
    for (int j = 0; j < 4; ++j) {
      *(float4 *)(po + 8 * j) = make_float4(o[nt][0][j], o[nt][1][j], o[nt][2][j], o[nt][3][j]);
      *(float4 *)(po + 8 * j + 4) = make_float4(o[nt][4][j], o[nt][5][j], o[nt][6][j], o[nt][7][j]);
    }
    if (g == 0) p.partial_ml[slot] = make_float2(m_run, l_run);
  }
}

// ---- prefill: K/V tiles staged in LDS and shared by the four waves of a workgroup -------------
//
// A work item of a prefill batch is (up to kSharedWaves * kSharedTiles * (16 / group) consecutive query
// tokens of a lane, split); blockIdx.y is the kv head.  Wave w owns the w-th slice of those tokens
// (one 16-row query tile: 16 / group tokens x group heads) and all waves walk the same keys, so a
// K/V tile is fetched from memory once per workgroup: each wave moves its share of the tile
// straight into LDS (global_load_lds), double buffered, one barrier per tile.  The softmax is
// vector-ALU and latency heavy, so the kernel is built for occupancy rather than for long
// software pipelines: one query tile per wave keeps it at 168 registers, three waves per SIMD
// (three workgroups per CU).  Rows are 256 bytes (one head of one
// token); the 16-byte piece p of row r sits in slot p ^ (r & 15), which keeps both operand read
// patterns (a K row piece per lane, a V column piece of eight tokens per lane) free of bank
// conflicts.  Keys past the end of the split are staged from its last valid token and masked.
constexpr uint32_t kSharedWaves = 4;    // waves of a prefill workgroup
constexpr int kSharedTiles = 1;          // 16-row query tiles per wave

struct SharedTiles {
  uint4 rows[2][2][kTile][16];   // [buffer][K, V][token][slot]
};

__device__ inline void stage_tile(const FastRagged &p, SharedTiles &lds, uint32_t buffer,
                                  uint32_t tile0, uint32_t end, uint32_t page0, uint32_t physical,
                                  uint32_t kv_head, uint32_t wave, uint32_t lane) {
  const uint32_t pt = p.page_tokens;
  constexpr int kPerWave = kTile / 4 / kSharedWaves;   // instructions per wave and operand
#pragma unroll
  for (int j = 0; j < kPerWave; ++j) {
    const uint32_t row = 4 * kPerWave * wave + 4 * j + (lane >> 4);
    const uint32_t token = min(tile0 + row, end - 1);
    const uint32_t page = (uint32_t)__shfl((int)physical, (int)(token / pt - page0), 64);
    const uint64_t element = (((uint64_t)page * pt + token % pt) * p.kv_heads + kv_head) * 128 +
                             8 * ((lane & 15) ^ (row & 15));
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void *)(p.key_pool + element),
        (__attribute__((address_space(3))) void *)&lds.rows[buffer][0][4 * kPerWave * wave + 4 * j][0], 16, 0, 0);
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void *)(p.value_pool + element),
        (__attribute__((address_space(3))) void *)&lds.rows[buffer][1][4 * kPerWave * wave + 4 * j][0], 16, 0, 0);
  }
}

// The register image load_tile would have produced, read from the staged tile.
__device__ inline void read_tile(const SharedTiles &lds, uint32_t buffer, TileRegs &r, uint32_t hl,
                                 uint32_t g) {
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) {
    const uint32_t k_row = 16 * sub + hl;
#pragma unroll
    for (int step = 0; step < 4; ++step) r.k[sub][step] = lds.rows[buffer][0][k_row][(4 * step + g) ^ hl];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t v_row = 16 * sub + 4 * g + i;
      r.v[4 * sub + i] = lds.rows[buffer][1][v_row][hl ^ (v_row & 15)];
    }
  }
}

template <bool kHalf, bool kMixed>
__global__ __launch_bounds__(64 * kSharedWaves) __attribute__((amdgpu_waves_per_eu(3, 3))) void ragged_attention_prefill_kernel(
    FastRagged p, ErrorSlot *error) {
  constexpr int NT = kSharedTiles;
  __shared__ SharedTiles lds;
  const uint32_t lane = threadIdx.x & 63, hl = lane & 15, g = lane >> 4;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t item = blockIdx.x, kv_head = blockIdx.y;
  if (item >= p.item_count[0]) return;
  const uint2 work = p.items[item];
  const uint32_t leader = work.x, split = work.y;
  const TokenPlan plan = p.plans[leader];
  const uint32_t per_tile = 16 / p.group, per_wave = NT * per_tile;
  const uint32_t first = wave * per_wave;                       // this wave's first member
  const uint32_t members = plan.members > first ? min(plan.members - first, per_wave) : 0;
  // the item's split layout is sized for its last member; a wave stops at its own last member
  const uint32_t longest = p.fixed_attended ? plan.attended : plan.attended + plan.members - 1;
  const uint32_t begin = split * plan.chunk;
  const uint32_t end = min(longest, begin + plan.chunk);
  const uint32_t own_end =
      members == 0 ? begin : min(end, p.fixed_attended ? plan.attended : plan.attended + first + members - 1);
  const uint32_t pt = p.page_tokens;
  const uint32_t *table = p.tables + (uint64_t)plan.lane * p.table_pages * 2;

  uint4 q_reg[NT][4];
  uint32_t limit[NT], member_of[NT];
  const uint32_t head = kv_head * p.group + hl % p.group;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    member_of[nt] = first + nt * per_tile + hl / p.group;
    const bool used = hl < per_tile * p.group && member_of[nt] < plan.members;
    limit[nt] = !used ? 0 : min(end, p.fixed_attended ? plan.attended : plan.attended + member_of[nt]);
    const uint64_t q_row = (uint64_t)(leader + (used ? member_of[nt] : 0)) * p.q_stride_t +
                           (uint64_t)head * p.q_stride_h;
    for (int step = 0; step < 4; ++step) {
      q_reg[nt][step] = make_uint4(0, 0, 0, 0);
      if (used) q_reg[nt][step] = load_query<kHalf, kMixed>(p, q_row + 32 * step + 8 * g);
    }
    if (!used) member_of[nt] = 0xffffffffu;
  }
  // keys below `unmasked_end` are attended by every used row of this wave
  const uint32_t unmasked_end = min(own_end, p.fixed_attended ? plan.attended : plan.attended + first);
  f32x4 o[NT][8];
  Softmax sm[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    for (int mt = 0; mt < 8; ++mt) o[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    sm[nt] = Softmax{-__builtin_inff(), 0.0f};
  }

  const uint32_t first_page = begin / pt, last_page = (end - 1) / pt;
  for (uint32_t page0 = first_page; page0 <= last_page; page0 += 64) {
    // Authenticate up to 64 table entries at once (every wave for itself: same entries, same
    // result); nothing is dereferenced through a bad one.
    uint32_t my_page = page0 + lane, physical = 0;
    bool mine = my_page <= last_page, ok = true;
    if (mine) {
      uint32_t page = table[2 * (uint64_t)my_page], generation = table[2 * (uint64_t)my_page + 1];
      ok = page < p.physical_pages && p.generations[page] == generation;
      physical = page;
    }
    unsigned long long bad_mask = __ballot(mine && !ok);
    if (bad_mask) {
      if (wave == 0 && lane == (uint32_t)__ffsll((long long)bad_mask) - 1) {
        report_error(error + (uint64_t)leader * p.error_stride, my_page);
        for (uint32_t member = 0; member < plan.members; ++member) p.bad[leader + member] = 1;
      }
      if (plan.splits == 1) zero_head_rows<kMixed>(p, leader + first, members, kv_head, lane);
      return;
    }
    const uint32_t tok_lo = max(begin, page0 * pt);
    const uint32_t tok_hi = (uint32_t)min((uint64_t)end, ((uint64_t)page0 + 64) * pt);
    stage_tile(p, lds, 0, tok_lo, end, page0, physical, kv_head, wave, lane);
    uint32_t buffer = 0;
    for (uint32_t tile0 = tok_lo; tile0 < tok_hi; tile0 += kTile, buffer ^= 1) {
      __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): this wave's share of the tile has landed
      __syncthreads();                      // everybody's has, and the other buffer is free
      if (tile0 + kTile < tok_hi)
        stage_tile(p, lds, buffer ^ 1, tile0 + kTile, end, page0, physical, kv_head, wave, lane);
      if (tile0 < own_end) {
        TileRegs cur;
        read_tile(lds, buffer, cur, hl, g);
        if (tile0 + kTile <= unmasked_end)
          consume_tile<NT, false, kHalf>(cur, q_reg, o, sm, tile0, limit, p.scale_log2, g);
        else
          consume_tile<NT, true, kHalf>(cur, q_reg, o, sm, tile0, limit, p.scale_log2, g);
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();   // the next group's first tile goes into buffer 0
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float m_run = sm[nt].m, l_run = sm[nt].l;
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
    if (member_of[nt] == 0xffffffffu) continue;
    const uint32_t token = leader + member_of[nt];
    if (plan.splits == 1) {
      float inv = 1.0f / l_run;
      const uint64_t out_row = (uint64_t)token * p.out_stride_t + (uint64_t)head * p.out_stride_h;
      for (int j = 0; j < 4; ++j) {
        store_out4<kHalf, kMixed>(p, out_row + 32 * g + 8 * j, o[nt][0][j] * inv, o[nt][1][j] * inv,
                   o[nt][2][j] * inv, o[nt][3][j] * inv);
        store_out4<kHalf, kMixed>(p, out_row + 32 * g + 8 * j + 4, o[nt][4][j] * inv, o[nt][5][j] * inv,
                   o[nt][6][j] * inv, o[nt][7][j] * inv);
      }
      continue;
    }
    uint64_t slot = ((uint64_t)token * p.max_splits + split) * p.query_heads + head;
    float *po = p.partial_o + slot * 128 + 32 * g;
    for (int j = 0; j < 4; ++j) {
      *(float4 *)(po + 8 * j) = make_float4(o[nt][0][j], o[nt][1][j], o[nt][2][j], o[nt][3][j]);
      *(float4 *)(po + 8 * j + 4) = make_float4(o[nt][4][j], o[nt][5][j], o[nt][6][j], o[nt][7][j]);
    }
    if (g == 0) p.partial_ml[slot] = make_float2(m_run, l_run);
  }
}

// Decode batches: one query token per wave, two waves per SIMD to hide the K/V stream's latency.
template <bool kHalf, bool kMixed>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void ragged_attention_mfma_kernel(
    FastRagged p, ErrorSlot *error) {
  ragged_attention_body<1, kHalf, kMixed>(p, error);
}

// Merges the per-split partials of one (token, head): out = sum_s O_s 2^(m_s-M) / sum_s l_s
// 2^(m_s-M).  Also writes the zero rows of inactive lanes, uncovered tokens and tokens whose page
// table was refused.  Four waves: every wave finds M and the weights from one (m, l) load per
// lane (a token has at most 64 splits), then wave w folds splits 2w+half, 2w+half+8, ... of its
// lanes' four columns, all loads in flight at once, and the waves' sums meet in LDS.
__global__ __launch_bounds__(256) void ragged_reduce_kernel(FastRagged p) {
  __shared__ float4 folded[3][32];
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t column = (lane & 31) * 4, half = lane >> 5;
  const uint32_t head = blockIdx.x, listed = p.item_count[1];
  // blockIdx.y walks the list of tokens that need the merge (the plan kernel compiled it; the
  // bad-page flags an attention wave may have raised since are re-read here)
  for (uint32_t entry = blockIdx.y; entry < listed; entry += gridDim.y) {
    const uint32_t token = p.merge_tokens[entry];
    const TokenPlan plan = p.plans[token];
    const bool zero = plan.splits == 0 || p.bad[token] != 0;
    const uint64_t dst = (uint64_t)token * p.out_stride_t + (uint64_t)head * p.out_stride_h + column;
    if (zero) {
      if (threadIdx.x < 32) store_out4<false, true>(p, dst, 0.0f, 0.0f, 0.0f, 0.0f);
      continue;
    }
    const uint64_t base = (uint64_t)token * p.max_splits * p.query_heads + head;
    float2 ml = make_float2(-__builtin_inff(), 0.0f);
    if (lane < plan.splits) ml = p.partial_ml[base + (uint64_t)lane * p.query_heads];
    const float m_all = wave_max(ml.x);
    const float weight = lane < plan.splits ? exp2f(ml.x - m_all) : 0.0f;
    const float l_all = wave_sum(ml.y * weight);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {   // 64 splits / (4 waves * 2 halves)
      const uint32_t s = 8 * i + 2 * wave + half;
      const float w = __shfl(weight, (int)(s & 63), 64);
      if (s < plan.splits) {
        const float4 part =
            *(const float4 *)(p.partial_o + (base + (uint64_t)s * p.query_heads) * 128 + column);
        acc.x += part.x * w;
        acc.y += part.y * w;
        acc.z += part.z * w;
        acc.w += part.w * w;
      }
    }
    acc.x += __shfl_xor(acc.x, 32, 64);
    acc.y += __shfl_xor(acc.y, 32, 64);
    acc.z += __shfl_xor(acc.z, 32, 64);
    acc.w += __shfl_xor(acc.w, 32, 64);
    __syncthreads();   // the previous entry's sums have been read
    if (wave != 0 && half == 0) folded[wave - 1][lane] = acc;
    __syncthreads();
    if (threadIdx.x < 32) {
      for (int other = 0; other < 3; ++other) {
        const float4 part = folded[other][lane];
        acc.x += part.x;
        acc.y += part.y;
        acc.z += part.z;
        acc.w += part.w;
      }
      const float inv = 1.0f / l_all;
      store_out4<false, true>(p, dst, acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
    }
  }
}

// Pools of one 2-byte dtype; queries of the same dtype or f32; any float output.
bool fast_dtypes(const View &q, const View &out, const View &key_pool, const View &value_pool) {
  const uint32_t pool = key_pool.dtype;
  if ((pool != FH_BF16 && pool != FH_F16) || value_pool.dtype != pool) return false;
  if (q.dtype != pool && q.dtype != FH_F32) return false;
  return out.dtype == FH_F32 || out.dtype == FH_F16 || out.dtype == FH_BF16;
}

// The decode kernel stores a lane's new row itself when the rows are of the queries' dtype (the
// pools' own, or f32 converted on the way), a lane's two elements are one aligned load, and the
// pool rows are word aligned.
bool append_in_kernel_possible(const RaggedAttention &p) {
  for (const View *v : {&p.k_new, &p.v_new})
    if (v->dtype != p.q.dtype || v->stride[2] != 1 || v->stride[0] % 2 || v->stride[1] % 2 || v->offset % 2)
      return false;
  return p.key_pool.offset % 2 == 0 && p.value_pool.offset % 2 == 0;
}

bool fast_ragged_eligible(const RaggedAttention &p) {
  if (!fast_dtypes(p.q, p.out, p.key_pool, p.value_pool)) return false;
  if (p.k_new.dtype != p.q.dtype || p.v_new.dtype != p.q.dtype) return false;
  if (p.width != 128 || p.value_width != 128 || p.page_tokens % 16 != 0) return false;
  uint32_t group = p.query_heads / p.kv_heads;
  if (group > 16) return false;
  // innermost axis contiguous, 16-byte aligned rows
  if (p.q.stride[2] != 1 || p.out.stride[2] != 1) return false;
  if (p.q.stride[0] % 8 || p.q.stride[1] % 8 || p.q.offset % 8) return false;
  if (p.out.stride[0] % 4 || p.out.stride[1] % 4 || p.out.offset % 4) return false;
  if (p.key_pool.offset % 8 || p.value_pool.offset % 8) return false;
  return true;
}

}  // namespace

namespace {

uint32_t splits_for(uint32_t tokens) {
  uint32_t max_splits = 16384u / (tokens ? tokens : 1);
  if (max_splits > 64) max_splits = 64;
  if (max_splits < 1) max_splits = 1;
  return max_splits;
}

uint32_t forced_split_tokens() {
  static const uint32_t split_tokens = [] {
    const char *env = getenv("FORJA_HIP_SPLIT_TOKENS");
    uint32_t value = env ? (uint32_t)atoi(env) : 0;
    return value >= 32 ? value / 32 * 32 : 0;  // 0 = chosen per launch from the batch
  }();
  return split_tokens;
}

uint64_t round_256(uint64_t bytes) { return (bytes + 255) / 256 * 256; }

// Flags, plans, work items and the item count: everything ragged_plan_kernel writes.
uint64_t plan_storage_bytes(const FastRagged &f) {
  uint64_t slots = (uint64_t)f.tokens * f.max_splits;
  return 2 * round_256((uint64_t)f.tokens * 4) + round_256((uint64_t)f.tokens * sizeof(TokenPlan)) +
         round_256(slots * sizeof(uint2)) + 256;
}

char *carve_plan(FastRagged *f, char *ws) {
  uint64_t slots = (uint64_t)f->tokens * f->max_splits;
  f->bad = (uint32_t *)ws;
  ws += round_256((uint64_t)f->tokens * 4);
  f->merge_tokens = (uint32_t *)ws;
  ws += round_256((uint64_t)f->tokens * 4);
  f->plans = (TokenPlan *)ws;
  ws += round_256((uint64_t)f->tokens * sizeof(TokenPlan));
  f->items = (uint2 *)ws;
  ws += round_256(slots * sizeof(uint2));
  f->item_count = (uint32_t *)ws;
  return ws + 256;
}

// Carves the (m,l) and O partial storage out of the backend workspace, and the plan storage too
// unless `plan_storage` already holds room for it.
bool carve_partials(fh_backend *backend, FastRagged *f, char *plan_storage) {
  f->split_tokens = forced_split_tokens();
  uint64_t slots = (uint64_t)f->tokens * f->max_splits;
  uint64_t ml_bytes = round_256(slots * f->query_heads * sizeof(float2));
  uint64_t o_bytes = slots * f->query_heads * 128 * sizeof(float);
  char *ws = backend_workspace(
      backend, (plan_storage ? 0 : plan_storage_bytes(*f)) + ml_bytes + o_bytes);
  if (!ws) return false;
  if (plan_storage)
    carve_plan(f, plan_storage);
  else
    ws = carve_plan(f, ws);
  f->partial_ml = (float2 *)ws;
  ws += ml_bytes;
  f->partial_o = (float *)ws;
  return true;
}

// Shortens the split count until the partials (and the plan, when it lives in the workspace too)
// fit what the workspace can hand out.
void fit_splits(fh_backend *backend, FastRagged *f, bool plan_in_workspace) {
  const uint64_t limit = backend_workspace_limit(backend);
  auto need = [&] {
    const uint64_t slots = (uint64_t)f->tokens * f->max_splits;
    return (plan_in_workspace ? plan_storage_bytes(*f) : 0) +
           round_256(slots * f->query_heads * sizeof(float2)) +
           slots * f->query_heads * 128 * sizeof(float);
  };
  while (f->max_splits > 1 && need() > limit) --f->max_splits;
}

void launch_plan(hipStream_t stream, const FastRagged &f, ErrorSlot *error) {
  ragged_plan_kernel<<<dim3(1), 256, 0, stream>>>(f, error);
}

// queries or outputs of another dtype than the pools': the kernels choose at run time
bool mixed_dtypes(const FastRagged &f) {
  const uint32_t pool_dtype = f.pool_half ? FH_F16 : FH_BF16;
  return f.q_dtype != pool_dtype || f.out_dtype != pool_dtype;
}

using DecodeKernel = void (*)(FastRagged, ErrorSlot *);

DecodeKernel decode_kernel(const FastRagged &f) {
  const bool mixed = mixed_dtypes(f);
  return f.pool_half ? (mixed ? ragged_attention_mfma_kernel<true, true>
                              : ragged_attention_mfma_kernel<true, false>)
                     : (mixed ? ragged_attention_mfma_kernel<false, true>
                              : ragged_attention_mfma_kernel<false, false>);
}

uint32_t decode_waves(const FastRagged &f) { return f.kv_heads < 8 ? f.kv_heads : 8; }

// Work items of a decode batch the device runs at once: resident workgroups per compute unit
// times compute units, over the workgroups an item takes (one per 8 kv heads).  Needs q_dtype,
// out_dtype, pool_half and kv_heads.
uint32_t decode_item_slots(fh_backend *backend, const FastRagged &f) {
  static uint32_t resident[2][2][9];   // [f16 pools][mixed][waves]; every writer stores the same value
  const uint32_t waves = decode_waves(f);
  uint32_t &known = resident[f.pool_half ? 1 : 0][mixed_dtypes(f) ? 1 : 0][waves];
  uint32_t per_unit = known;
  if (per_unit == 0) {
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, decode_kernel(f), (int)(64 * waves), 0) !=
            hipSuccess ||
        blocks < 1)
      blocks = 1;
    known = per_unit = (uint32_t)blocks;
  }
  const uint32_t per_item = (f.kv_heads + waves - 1) / waves;
  const uint32_t slots = per_unit * backend_compute_units(backend) / per_item;
  return slots ? slots : 1;
}

void launch_fast(fh_backend *backend, hipStream_t stream, const FastRagged &f, ErrorSlot *error) {
  uint64_t groups = f.group_tokens > 1 ? f.tokens / f.group_tokens + f.lanes : f.tokens;
  uint64_t blocks = groups * f.max_splits;
  const bool mixed = mixed_dtypes(f);
  {
    KernelTimer timer(backend, FH_KC_ATTENTION_KERNEL);
    // one workgroup per work item, up to 8 (decode) or 4 (prefill) kv heads of it per workgroup
    if (f.group_tokens > 1) {
      const dim3 grid((unsigned)blocks, f.kv_heads);
      auto *kernel = f.pool_half ? (mixed ? ragged_attention_prefill_kernel<true, true>
                                          : ragged_attention_prefill_kernel<true, false>)
                                 : (mixed ? ragged_attention_prefill_kernel<false, true>
                                          : ragged_attention_prefill_kernel<false, false>);
      kernel<<<grid, 64 * kSharedWaves, 0, stream>>>(f, error);
    } else {
      const uint32_t waves = decode_waves(f);
      const dim3 grid((unsigned)blocks, (f.kv_heads + waves - 1) / waves);
      decode_kernel(f)<<<grid, 64 * waves, 0, stream>>>(f, error);
    }
  }
  ragged_reduce_kernel<<<dim3(f.query_heads, f.tokens < 1024 ? f.tokens : 1024), 256, 0, stream>>>(f);
}

}  // namespace

bool try_fast_lane_attention(fh_backend *backend, const LaneAttention &lane, ErrorSlot *error) {
  if (!fast_dtypes(lane.q, lane.out, lane.key_pool, lane.value_pool)) return false;
  if (lane.width != 128 || lane.value_width != 128 || lane.page_tokens % 16 != 0) return false;
  uint32_t group = lane.query_heads / lane.kv_heads;
  if (group > 16 || lane.query_length == 0) return false;
  if (lane.q.stride[2] != 1 || lane.out.stride[2] != 1) return false;
  if (lane.q.stride[0] % 8 || lane.q.stride[1] % 8 || lane.q.offset % 8) return false;
  if (lane.out.stride[0] % 4 || lane.out.stride[1] % 4 || lane.out.offset % 4) return false;
  if (lane.key_pool.offset % 8 || lane.value_pool.offset % 8) return false;
  FastRagged f{};
  f.tokens = lane.query_length;
  f.lanes = 1;
  f.query_heads = lane.query_heads;
  f.kv_heads = lane.kv_heads;
  f.group = group;
  f.page_tokens = lane.page_tokens;
  f.physical_pages = lane.physical_pages;
  f.table_pages = lane.logical_pages;
  f.max_splits = splits_for(f.tokens);
  fit_splits(backend, &f, true);
  f.group_tokens = f.tokens > 1 ? kSharedWaves * kSharedTiles * (16 / group) : 1;
  f.scale_log2 = lane.scale * 1.4426950408889634f;
  f.one_start = lane.query_start;
  f.fixed_attended = lane.causal ? 0 : lane.key_length;
  if (!carve_partials(backend, &f, nullptr)) return false;
  f.q = (const char *)lane.q.base + lane.q.offset * dtype_size(lane.q.dtype);
  f.out = (char *)lane.out.base + lane.out.offset * dtype_size(lane.out.dtype);
  f.q_dtype = lane.q.dtype;
  f.out_dtype = lane.out.dtype;
  f.pool_half = lane.key_pool.dtype == FH_F16;
  f.key_pool = (const uint16_t *)lane.key_pool.base + lane.key_pool.offset;
  f.value_pool = (const uint16_t *)lane.value_pool.base + lane.value_pool.offset;
  f.tables = (const uint32_t *)lane.table.base + lane.table.offset;
  f.generations = (const uint32_t *)lane.generations.base + lane.generations.offset;
  f.cu = nullptr;
  f.starts = nullptr;
  f.activity =
      lane.activity.base ? (const uint32_t *)lane.activity.base + lane.activity.offset : nullptr;
  f.item_slots = f.group_tokens == 1 ? decode_item_slots(backend, f) : 0;
  // q / out are [Hq, Sq, D] views: the token axis is axis 1.
  f.q_stride_t = lane.q.stride[1];
  f.q_stride_h = lane.q.stride[0];
  f.out_stride_t = lane.out.stride[1];
  f.out_stride_h = lane.out.stride[0];
  hipStream_t stream = backend_stream(backend);
  launch_plan(stream, f, error);
  launch_fast(backend, stream, f, error);
  return true;
}

bool run_ragged_attention(fh_backend *backend, const RaggedAttention &p, ErrorSlot *append_error) {
  hipStream_t stream = backend_stream(backend);
  ErrorSlot *error = append_error ? append_error + p.attention_error_offset : nullptr;
  const bool fast = fast_ragged_eligible(p);
  FastRagged f{};
  if (fast) {
    f.tokens = p.tokens;
    f.lanes = p.lanes;
    f.query_heads = p.query_heads;
    f.kv_heads = p.kv_heads;
    f.group = p.query_heads / p.kv_heads;
    f.group_tokens = p.tokens > p.lanes ? kSharedWaves * kSharedTiles * (16 / f.group) : 1;
    f.page_tokens = p.page_tokens;
    f.physical_pages = p.physical_pages;
    f.table_pages = p.table_pages;
    f.max_splits = splits_for(p.tokens);
    fit_splits(backend, &f, false);
    f.q_dtype = p.q.dtype;
    f.out_dtype = p.out.dtype;
    f.pool_half = p.key_pool.dtype == FH_F16;
    f.item_slots = f.group_tokens == 1 ? decode_item_slots(backend, f) : 0;
    f.error_stride = p.error_stride;
    f.scale_log2 = p.scale * 1.4426950408889634f;
    f.tables = (const uint32_t *)p.tables.base + p.tables.offset;
    f.generations = (const uint32_t *)p.generations.base + p.generations.offset;
    f.cu = (const uint32_t *)p.cu_seqlens.base + p.cu_seqlens.offset;
    f.starts = (const uint32_t *)p.q_starts.base + p.q_starts.offset;
    f.activity = p.activity.base ? (const uint32_t *)p.activity.base + p.activity.offset : nullptr;
    // The plan depends on the lane metadata only, which every layer of a step shares: it is built
    // by the first attention dispatch of a submission and reused until that metadata is written.
    AttentionPlanKey key{};
    for (int i = 0; i < 5; ++i) key.buffers[i] = p.metadata_buffers[i];
    key.address[0] = (uint64_t)f.cu;
    key.address[1] = (uint64_t)f.starts;
    key.address[2] = (uint64_t)f.activity;
    key.address[3] = (uint64_t)f.tables;
    key.address[4] = (uint64_t)f.generations;
    f.promised = p.one_row_per_lane;
    f.append_in_kernel = p.one_row_per_lane && append_in_kernel_possible(p);
    const uint32_t params[13] = {f.tokens, f.lanes, f.group_tokens, f.page_tokens, f.physical_pages,
                                 f.table_pages, f.max_splits, forced_split_tokens(), f.kv_heads,
                                 f.query_heads, f.append_in_kernel, f.promised, f.item_slots};
    for (int i = 0; i < 13; ++i) key.params[i] = params[i];
    bool reuse = false;
    char *plan_storage = backend_attention_plan(backend, key, plan_storage_bytes(f), &reuse);
    if (!plan_storage || !carve_partials(backend, &f, plan_storage)) return false;
    f.q = (const char *)p.q.base + p.q.offset * dtype_size(p.q.dtype);
    f.out = (char *)p.out.base + p.out.offset * dtype_size(p.out.dtype);
    f.key_pool = (const uint16_t *)p.key_pool.base + p.key_pool.offset;
    f.value_pool = (const uint16_t *)p.value_pool.base + p.value_pool.offset;
    f.q_stride_t = p.q.stride[0];
    f.q_stride_h = p.q.stride[1];
    f.out_stride_t = p.out.stride[0];
    f.out_stride_h = p.out.stride[1];
    f.k_new = (const char *)p.k_new.base + p.k_new.offset * dtype_size(p.k_new.dtype);
    f.v_new = (const char *)p.v_new.base + p.v_new.offset * dtype_size(p.v_new.dtype);
    f.kn_stride_t = p.k_new.stride[0];
    f.kn_stride_h = p.k_new.stride[1];
    f.vn_stride_t = p.v_new.stride[0];
    f.vn_stride_h = p.v_new.stride[1];
    f.append_error_back = p.attention_error_offset;
    if (!reuse) launch_plan(stream, f, error);
  }
  if (fast && f.append_in_kernel) {
    launch_fast(backend, stream, f, error);
    return true;
  }
  // Whether cu_seqlens was refused: the work plan records it; without a plan a kernel of its own
  // finds out.
  const uint32_t *malformed = fast ? f.item_count + 2 : nullptr;
  if (!fast) {
    uint32_t *flag = (uint32_t *)backend_workspace(backend, 256);
    if (!flag) return false;
    ragged_validate_kernel<<<dim3(1), 256, 0, stream>>>(
        (const uint32_t *)p.cu_seqlens.base + p.cu_seqlens.offset, p.lanes, p.tokens, flag, error);
    malformed = flag;
  }
  uint64_t append_work =
      (uint64_t)p.tokens * (p.kv_heads * p.width + p.kv_heads * p.value_width);
  if (append_by_pieces(p))
    ragged_append_pieces_kernel<<<dim3((unsigned)((append_work / 8 + 255) / 256)), 256, 0, stream>>>(
        p, append_error, malformed);
  else
    ragged_append_kernel<<<dim3((unsigned)((append_work + 255) / 256)), 256, 0, stream>>>(
        p, append_error, malformed);
  if (fast) {
    launch_fast(backend, stream, f, error);
    return true;
  }
  uint32_t blocks = p.tokens * p.query_heads;
  if (p.value_width <= 64)
    ragged_attention_generic_kernel<64><<<dim3(blocks), 64, 0, stream>>>(p, error, malformed);
  else if (p.value_width <= 128)
    ragged_attention_generic_kernel<128><<<dim3(blocks), 64, 0, stream>>>(p, error, malformed);
  else
    ragged_attention_generic_kernel<256><<<dim3(blocks), 64, 0, stream>>>(p, error, malformed);
  return true;
}

}  // namespace fh
