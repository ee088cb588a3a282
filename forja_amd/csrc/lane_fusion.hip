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

}  // namespace

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
