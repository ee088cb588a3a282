// Kernels behind the fusion of a run of per-lane attention dispatches into one ragged launch.
//
// The engines record one Op::PagedSdpaAppend per decode lane and layer
// (engines/qwen3-coder/src/lib.rs:917-935), each with the lane's own block-table allocation
// (crates/forja-host/src/lib.rs:4466-4480), a freshly allocated output row
// (crates/forja-sdk/src/paged.rs:525-528) and a following Op::Copy of that row into the packed
// activation.  The ragged attention kernels want one table tensor and one output tensor, so a
// fused run first gathers the lanes' metadata into contiguous arrays, attends into a contiguous
// scratch, and then scatters the scratch rows to the places the dispatches named.  The scattered
// addresses travel as kernel arguments (a few KB per launch), so nothing is staged through
// host-visible memory and the host buffers can be reused as soon as the launch call returns.
//
// A sequence's prefill chunk recorded on its own (two Op::PagedCopy of its rows and one causal
// Op::PagedSdpa over them: the multi-row branch of paged_cache_attention,
// engines/qwen3-coder/src/lib.rs:685-707) joins such a run as a member with several query rows; the
// second half of this file is the same glue for runs that have such members.
#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace fh {

namespace {

// One workgroup per lane: copies the lane's block table and writes its scalars.
__global__ __launch_bounds__(256) void gather_lane_metadata_kernel(
    LaneSources sources, uint32_t first, uint32_t count, uint32_t lanes, uint32_t table_words,
    uint32_t *tables, uint32_t *activity, uint32_t *starts, uint32_t *cu) {
  const uint32_t local = blockIdx.x;
  if (local >= count) return;
  const uint32_t lane = first + local;
  if (lane == 0 && threadIdx.x == 0) cu[lanes + 1] = 0;   // the overlap flag of lane_conflict_kernel
  const uint32_t *table = sources.table[local];
  uint32_t *target = tables + (uint64_t)lane * table_words;
  for (uint32_t word = threadIdx.x; word < table_words; word += blockDim.x)
    target[word] = table[word];
  if (threadIdx.x == 0) {
    const uint32_t *flag = sources.activity[local];
    activity[lane] = flag ? flag[0] : 1u;
    starts[lane] = sources.start[local];
    cu[lane] = lane;
    if (lane + 1 == lanes) cu[lanes] = lanes;
  }
}

// One workgroup per lane (the reader): does any OTHER active lane append into a slot this lane
// attends?  A fused run performs every append before every attention; lane by lane, a reader
// that comes first sees the slot's old contents, and two lanes that append to one slot each see
// their own value.  The host keeps pages copy-on-write, so this does not happen
// (crates/forja-host/src/lib.rs:5408-5470); tables are caller data all the same, so it is checked
// and a run with such an overlap is executed dispatch by dispatch instead.
// Dynamic LDS: 2 * lanes words (each lane's destination page and slot).
__global__ __launch_bounds__(256) void lane_conflict_kernel(const uint32_t *tables, const uint32_t *activity,
                                                            const uint32_t *starts, uint32_t lanes,
                                                            uint32_t table_pages, uint32_t page_tokens,
                                                            uint32_t *conflict) {
  extern __shared__ uint32_t destinations[];   // [lanes] page, [lanes] slot (kNone: appends nothing)
  constexpr uint32_t kNone = 0xffffffffu;
  uint32_t *pages = destinations, *slots = destinations + lanes;
  for (uint32_t writer = threadIdx.x; writer < lanes; writer += blockDim.x) {
    const uint32_t logical = starts[writer] / page_tokens;
    const bool appends = activity[writer] != 0 && logical < table_pages;
    pages[writer] = appends ? tables[((uint64_t)writer * table_pages + logical) * 2] : kNone;
    slots[writer] = appends ? starts[writer] % page_tokens : kNone;
  }
  __syncthreads();
  const uint32_t reader = blockIdx.x;
  if (activity[reader] == 0) return;
  const uint64_t attended = (uint64_t)starts[reader] + 1;   // positions [0, attended)
  const uint64_t attended_pages = (attended + page_tokens - 1) / page_tokens;
  const uint32_t limit = (uint32_t)(attended_pages < table_pages ? attended_pages : table_pages);
  bool found = false;
  for (uint32_t logical = threadIdx.x; logical < limit; logical += blockDim.x) {
    const uint32_t page = tables[((uint64_t)reader * table_pages + logical) * 2];
    for (uint32_t writer = 0; writer < lanes; ++writer)
      if (writer != reader && slots[writer] != kNone && pages[writer] == page &&
          (uint64_t)logical * page_tokens + slots[writer] < attended)
        found = true;
  }
  if (found) *conflict = 1u;
}

// One workgroup per lane: copies the lane's attended row to one or two destinations.
__global__ __launch_bounds__(256) void scatter_lane_rows_kernel(LaneRows targets, const char *rows,
                                                                uint32_t first, uint32_t count,
                                                                uint32_t row_bytes) {
  const uint32_t local = blockIdx.x;
  if (local >= count) return;
  const char *source = rows + (uint64_t)(first + local) * row_bytes;
  char *destinations[2] = {(char *)targets.first[local], (char *)targets.second[local]};
  for (int which = 0; which < 2; ++which) {
    char *target = destinations[which];
    if (!target) continue;
    const bool wide = (((uint64_t)target | (uint64_t)source | row_bytes) & 15u) == 0;
    if (wide) {
      for (uint32_t piece = threadIdx.x; piece < row_bytes / 16; piece += blockDim.x)
        ((uint4 *)target)[piece] = ((const uint4 *)source)[piece];
    } else {
      // every element type here is at least two bytes wide and so is every alignment
      for (uint32_t piece = threadIdx.x; piece < row_bytes / 2; piece += blockDim.x)
        ((uint16_t *)target)[piece] = ((const uint16_t *)source)[piece];
    }
  }
}

// ---- runs with prefill chunks: a member has cu[m + 1] - cu[m] query rows ----

__global__ __launch_bounds__(256) void gather_chunk_metadata_kernel(
    ChunkSources sources, uint32_t first, uint32_t count, uint32_t lanes, uint32_t tokens,
    uint32_t table_words, uint32_t *tables, uint32_t *activity, uint32_t *starts, uint32_t *cu,
    uint32_t *records) {
  const uint32_t local = blockIdx.x;
  if (local >= count) return;
  const uint32_t lane = first + local;
  if (lane == 0 && threadIdx.x == 0) cu[lanes + 1] = 0;   // the overlap flag of chunk_conflict_kernel
  const uint32_t *table = sources.table[local];
  uint32_t *target = tables + (uint64_t)lane * table_words;
  for (uint32_t word = threadIdx.x; word < table_words; word += blockDim.x)
    target[word] = table[word];
  if (threadIdx.x == 0) {
    const uint32_t *flag = sources.activity[local];
    activity[lane] = flag ? flag[0] : 1u;
    starts[lane] = sources.start[local];
    cu[lane] = sources.first_token[local];
    if (lane + 1 == lanes) cu[lanes] = tokens;
    records[lane] = sources.append_record[local];
    records[lanes + lane] = sources.attention_record[local];
  }
}

// One workgroup per member (the reader): does any OTHER active member store a row into a slot
// this member attends?  Member w stores positions [starts[w], starts[w] + rows of w) through its
// own table; the reader attends positions [0, starts[r] + rows of r) through its own.
__global__ __launch_bounds__(256) void chunk_conflict_kernel(const uint32_t *tables, const uint32_t *activity,
                                                             const uint32_t *starts, const uint32_t *cu,
                                                             uint32_t lanes, uint32_t table_pages,
                                                             uint32_t page_tokens, uint32_t *conflict) {
  const uint32_t reader = blockIdx.x;
  if (activity[reader] == 0) return;
  const uint64_t attended = (uint64_t)starts[reader] + (cu[reader + 1] - cu[reader]);
  const uint64_t attended_pages = (attended + page_tokens - 1) / page_tokens;
  const uint32_t limit = (uint32_t)(attended_pages < table_pages ? attended_pages : table_pages);
  bool found = false;
  for (uint32_t logical = threadIdx.x; logical < limit; logical += blockDim.x) {
    const uint32_t page = tables[((uint64_t)reader * table_pages + logical) * 2];
    for (uint32_t writer = 0; writer < lanes; ++writer) {
      const uint32_t rows = cu[writer + 1] - cu[writer];
      if (writer == reader || activity[writer] == 0 || rows == 0) continue;
      const uint64_t from = starts[writer], last = from + rows - 1;
      const uint64_t first_page = from / page_tokens;
      uint64_t last_page = last / page_tokens;
      if (last_page >= table_pages) last_page = table_pages ? table_pages - 1 : 0;
      for (uint64_t at = first_page; at <= last_page && at < table_pages; ++at) {
        if (tables[((uint64_t)writer * table_pages + at) * 2] != page) continue;
        const uint64_t slot = at == first_page ? from % page_tokens : 0;   // the first slot stored in that page
        if ((uint64_t)logical * page_tokens + slot < attended) found = true;
      }
    }
  }
  if (found) *conflict = 1u;
}

// One workgroup per query row: the row's heads go to one or two destinations with strides of
// their own.
__global__ __launch_bounds__(256) void scatter_chunk_rows_kernel(ChunkTargets targets, const char *rows,
                                                                 uint32_t count, uint32_t heads,
                                                                 uint32_t row_bytes) {
  const uint32_t token = targets.first_token[0] + blockIdx.x;
  if (token >= targets.first_token[count]) return;
  uint32_t member = 0;
  while (member + 1 < count && token >= targets.first_token[member + 1]) ++member;
  const uint32_t local = token - targets.first_token[member];
  const char *source = rows + (uint64_t)token * heads * row_bytes;
  for (int which = 0; which < 2; ++which) {
    char *target = (char *)targets.target[which][member];
    if (!target) continue;
    const uint32_t token_stride = targets.token_stride[which][member];
    const uint32_t head_stride = targets.head_stride[which][member];
    target += (uint64_t)local * token_stride;
    const bool wide = (((uint64_t)target | (uint64_t)source | row_bytes | head_stride) & 15u) == 0;
    const uint32_t piece_bytes = wide ? 16 : 2;   // every element type here is at least two bytes wide
    const uint32_t per_head = row_bytes / piece_bytes;
    for (uint32_t piece = threadIdx.x; piece < heads * per_head; piece += blockDim.x) {
      const uint32_t head = piece / per_head, inside = (piece % per_head) * piece_bytes;
      const char *from = source + (uint64_t)head * row_bytes + inside;
      char *to = target + (uint64_t)head * head_stride + inside;
      if (wide)
        *(uint4 *)to = *(const uint4 *)from;
      else
        *(uint16_t *)to = *(const uint16_t *)from;
    }
  }
}

__global__ __launch_bounds__(256) void fold_chunk_errors_kernel(ErrorSlot *staged, ErrorSlot *records_of_run,
                                                                const uint32_t *cu, const uint32_t *records,
                                                                uint32_t lanes, uint32_t tokens) {
  const uint32_t token = blockIdx.x * blockDim.x + threadIdx.x;
  if (token >= tokens) return;
  uint32_t lo = 0, hi = lanes;   // cu[lo] <= token < cu[hi]
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) / 2;
    if (cu[mid] <= token) lo = mid; else hi = mid;
  }
  for (uint32_t kind = 0; kind < 2; ++kind) {
    ErrorSlot *slot = staged + 2ull * token + kind;
    if (slot->flag) {
      report_error(records_of_run + records[kind * lanes + lo], slot->value);
      slot->flag = 0;
      slot->value = 0xffffffffu;
    }
  }
}

}  // namespace

void launch_gather_chunk_metadata(hipStream_t stream, const ChunkSources &sources, uint32_t first,
                                  uint32_t count, uint32_t lanes, uint32_t tokens,
                                  uint32_t table_words, uint32_t *tables, uint32_t *activity,
                                  uint32_t *starts, uint32_t *cu, uint32_t *records) {
  if (count == 0 || count > kChunkMembers || first + count > lanes) return;
  gather_chunk_metadata_kernel<<<dim3(count), 256, 0, stream>>>(sources, first, count, lanes, tokens,
                                                                 table_words, tables, activity, starts,
                                                                 cu, records);
}

void launch_chunk_conflict_check(hipStream_t stream, const uint32_t *tables, const uint32_t *activity,
                                 const uint32_t *starts, const uint32_t *cu, uint32_t lanes,
                                 uint32_t table_pages, uint32_t page_tokens, uint32_t *conflict) {
  if (lanes == 0 || page_tokens == 0) return;
  chunk_conflict_kernel<<<dim3(lanes), 256, 0, stream>>>(tables, activity, starts, cu, lanes, table_pages,
                                                          page_tokens, conflict);
}

void launch_scatter_chunk_rows(hipStream_t stream, const ChunkTargets &targets, const void *rows,
                               uint32_t count, uint32_t heads, uint32_t row_bytes) {
  if (count == 0 || count > kChunkMembers || row_bytes % 2 != 0) return;
  const uint32_t tokens = targets.first_token[count] - targets.first_token[0];
  if (tokens == 0) return;
  scatter_chunk_rows_kernel<<<dim3(tokens), 256, 0, stream>>>(targets, (const char *)rows, count, heads,
                                                               row_bytes);
}

void launch_fold_chunk_errors(hipStream_t stream, ErrorSlot *staged, ErrorSlot *records_of_run,
                              const uint32_t *cu, const uint32_t *records, uint32_t lanes,
                              uint32_t tokens) {
  if (tokens == 0 || lanes == 0) return;
  fold_chunk_errors_kernel<<<dim3((tokens + 255) / 256), 256, 0, stream>>>(staged, records_of_run, cu,
                                                                            records, lanes, tokens);
}

void launch_gather_lane_metadata(hipStream_t stream, const LaneSources &sources, uint32_t first,
                                 uint32_t count, uint32_t lanes, uint32_t table_words,
                                 uint32_t *tables, uint32_t *activity, uint32_t *starts,
                                 uint32_t *cu) {
  if (count == 0 || count > kLaneChunk || first + count > lanes) return;
  gather_lane_metadata_kernel<<<dim3(count), 256, 0, stream>>>(sources, first, count, lanes,
                                                                table_words, tables, activity,
                                                                starts, cu);
}

bool launch_lane_conflict_check(hipStream_t stream, const uint32_t *tables, const uint32_t *activity,
                                const uint32_t *starts, uint32_t lanes, uint32_t table_pages,
                                uint32_t page_tokens, uint32_t *conflict) {
  const uint64_t shared = 2ull * lanes * sizeof(uint32_t);
  if (lanes == 0 || page_tokens == 0 || shared > 48u * 1024) return false;
  lane_conflict_kernel<<<dim3(lanes), 256, shared, stream>>>(tables, activity, starts, lanes, table_pages,
                                                             page_tokens, conflict);
  return true;
}

void launch_scatter_lane_rows(hipStream_t stream, const LaneRows &targets, const void *rows,
                              uint32_t first, uint32_t count, uint32_t row_bytes) {
  if (count == 0 || count > kLaneChunk || row_bytes % 2 != 0) return;
  scatter_lane_rows_kernel<<<dim3(count), 256, 0, stream>>>(targets, (const char *)rows, first,
                                                            count, row_bytes);
}

}  // namespace fh
