// Paged-KV grouped-query attention over a packed ragged batch (block tables + cu_seqlens).
//
// Reference semantics: CpuPagePool::sdpa (crates/forja-cpu/src/paged.rs:161-259) per lane, after
// the lane's new K/V rows were stored at its q_start (execute_paged_append,
// crates/forja-cpu/src/lib.rs:262-306).  Pools are [P, page_tokens, Hkv, D]; a table entry is
// (physical page, generation) and is valid iff page < P and generations[page] == generation.
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
__global__ void ragged_append_kernel(RaggedAttention p, ErrorSlot *error) {
  uint32_t key_row = p.kv_heads * p.width, value_row = p.kv_heads * p.value_width;
  uint32_t per_token = key_row + value_row;
  uint64_t flat = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (flat >= (uint64_t)p.tokens * per_token) return;
  uint32_t token = (uint32_t)(flat / per_token), element = (uint32_t)(flat % per_token);
  const uint32_t *cu = (const uint32_t *)p.cu_seqlens.base + p.cu_seqlens.offset;
  if (token < cu[0] || token >= cu[p.lanes]) return;
  uint32_t lane = find_lane(cu, p.lanes, token);
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
    if (element == 0) report_error(error, logical_page > 0xffffffffull ? 0xffffffffu
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

// Any dtype / width: one wave per (token, query head); per-lane online softmax merged at the end.
template <int kMaxDv>
__global__ void ragged_attention_generic_kernel(RaggedAttention p, ErrorSlot *error) {
  __shared__ float q_row[512];
  __shared__ int bad;
  uint32_t token = blockIdx.x / p.query_heads, head = blockIdx.x % p.query_heads;
  uint32_t lane_id = threadIdx.x;
  const uint32_t *cu = (const uint32_t *)p.cu_seqlens.base + p.cu_seqlens.offset;
  uint64_t out_base = p.out.offset + token * p.out.stride[0] + head * p.out.stride[1];
  bool covered = token >= cu[0] && token < cu[p.lanes];
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
      report_error(error, p.table_pages);
      bad = 1;
    }
    pages = p.table_pages;
  }
  for (uint32_t page = lane_id; page < pages; page += 64) {
    uint32_t physical;
    if (!entry_ok(table, generations, page, p.table_pages, p.physical_pages, &physical)) {
      report_error(error, page);
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

}  // namespace

bool try_fast_lane_attention(fh_backend *, const LaneAttention &, ErrorSlot *) { return false; }

bool run_ragged_attention(fh_backend *backend, const RaggedAttention &p, ErrorSlot *error) {
  hipStream_t stream = backend_stream(backend);
  uint64_t append_work =
      (uint64_t)p.tokens * (p.kv_heads * p.width + p.kv_heads * p.value_width);
  ragged_append_kernel<<<dim3((unsigned)((append_work + 255) / 256)), 256, 0, stream>>>(p, error);
  uint32_t blocks = p.tokens * p.query_heads;
  if (p.value_width <= 64)
    ragged_attention_generic_kernel<64><<<dim3(blocks), 64, 0, stream>>>(p, error);
  else if (p.value_width <= 128)
    ragged_attention_generic_kernel<128><<<dim3(blocks), 64, 0, stream>>>(p, error);
  else
    ragged_attention_generic_kernel<256><<<dim3(blocks), 64, 0, stream>>>(p, error);
  return true;
}

}  // namespace fh
