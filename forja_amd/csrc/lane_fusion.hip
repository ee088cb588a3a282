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

void launch_scatter_lane_rows(hipStream_t stream, const LaneRows &targets, const void *rows,
                              uint32_t first, uint32_t count, uint32_t row_bytes) {
  if (count == 0 || count > kLaneChunk || row_bytes % 2 != 0) return;
  scatter_lane_rows_kernel<<<dim3(count), 256, 0, stream>>>(targets, (const char *)rows, first,
                                                            count, row_bytes);
}

}  // namespace fh
