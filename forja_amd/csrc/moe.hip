// GPU-side token->expert packing for routed (MoE) projections.
//
// Behavioural reference: count_expert_routes / plan_expert_routes / arrange_expert_routes
// (crates/forja-metal/src/quant_matmul.metal:1217-1357): per-expert counts, exclusive offsets,
// and `sorted_routes` = route ids r*k+s grouped by expert with ascending route id inside an
// expert (a stable counting sort), plus (expert,start,count<=tile_rows) row blocks for a grouped
// GEMM.  Pure integer work: results are bit-exact against the closed form.
#include "kernels.hpp"

namespace fh {

namespace {

// One wave does the whole plan: at decode sizes (<= a few thousand routes) the work is a handful
// of 64-route rounds and a single launch beats three.
__global__ void route_pack_kernel(View indices, uint32_t rows, uint32_t k, uint32_t experts,
                                  uint32_t tile_rows, uint32_t *counts, uint32_t *offsets,
                                  uint32_t *sorted_routes, uint32_t *blocks, uint32_t max_blocks,
                                  uint32_t *n_blocks, ErrorSlot *error) {
  extern __shared__ uint32_t lds[];
  uint32_t *lds_counts = lds;            // [experts]
  uint32_t *lds_cursor = lds + experts;  // [experts]
  const uint32_t lane = threadIdx.x;
  const uint32_t routes = rows * k;
  for (uint32_t e = lane; e < experts; e += 64) lds_counts[e] = 0;
  __syncthreads();
  for (uint32_t route = lane; route < routes; route += 64) {
    uint32_t expert = load_u32_at(indices, indices.offset + (uint64_t)(route / k) * indices.stride[0] +
                                               (uint64_t)(route % k) * indices.stride[1]);
    if (expert >= experts)
      report_error(error, expert);
    else
      atomicAdd(&lds_counts[expert], 1u);
  }
  __syncthreads();
  // Exclusive scan of counts, 64 experts per round.
  uint32_t running = 0;
  for (uint32_t base = 0; base < experts; base += 64) {
    uint32_t e = base + lane;
    uint32_t c = e < experts ? lds_counts[e] : 0;
    uint32_t inclusive = c;
    for (int offset = 1; offset < 64; offset <<= 1) {
      uint32_t other = __shfl_up(inclusive, offset, 64);
      if ((int)lane >= offset) inclusive += other;
    }
    uint32_t exclusive = running + inclusive - c;
    if (e < experts) {
      counts[e] = c;
      offsets[e] = exclusive;
      lds_cursor[e] = exclusive;
    }
    running += __shfl(inclusive, 63, 64);
  }
  if (lane == 0) offsets[experts] = running;
  __syncthreads();
  // Stable arrange: within a round, a route's rank is the number of lower lanes naming the same
  // expert; rounds run in ascending route order.
  for (uint32_t base = 0; base < routes; base += 64) {
    uint32_t route = base + lane;
    uint32_t expert = 0xffffffffu;
    if (route < routes)
      expert = load_u32_at(indices, indices.offset + (uint64_t)(route / k) * indices.stride[0] +
                                        (uint64_t)(route % k) * indices.stride[1]);
    bool valid = route < routes && expert < experts;
    unsigned long long same = __ballot(valid);
    for (uint32_t bit = 0; (experts - 1) >> bit; ++bit) {
      unsigned long long set = __ballot(valid && ((expert >> bit) & 1u));
      same &= ((expert >> bit) & 1u) ? set : ~set;
    }
    uint32_t rank = __popcll(same & ((1ull << lane) - 1ull));
    uint32_t group = __popcll(same);
    uint32_t position = 0;
    if (valid) position = lds_cursor[expert] + rank;
    __syncthreads();
    if (valid) {
      sorted_routes[position] = route;
      if (rank + 1 == group) lds_cursor[expert] = position + 1;
    }
    __syncthreads();
  }
  // Row blocks in ascending (expert, start) order.
  uint32_t block_running = 0;
  for (uint32_t base = 0; base < experts; base += 64) {
    uint32_t e = base + lane;
    uint32_t c = e < experts ? lds_counts[e] : 0;
    uint32_t tiles = (c + tile_rows - 1) / tile_rows;
    uint32_t inclusive = tiles;
    for (int offset = 1; offset < 64; offset <<= 1) {
      uint32_t other = __shfl_up(inclusive, offset, 64);
      if ((int)lane >= offset) inclusive += other;
    }
    uint32_t first = block_running + inclusive - tiles;
    if (e < experts) {
      uint32_t start = lds_cursor[e] - c;  // cursor now sits at the end of the expert's span
      for (uint32_t t = 0; t < tiles; ++t) {
        uint32_t b = first + t;
        if (b >= max_blocks) break;
        uint32_t remaining = c - t * tile_rows;
        blocks[3 * b + 0] = e;
        blocks[3 * b + 1] = start + t * tile_rows;
        blocks[3 * b + 2] = remaining < tile_rows ? remaining : tile_rows;
      }
    }
    block_running += __shfl(inclusive, 63, 64);
  }
  if (lane == 0) n_blocks[0] = block_running < max_blocks ? block_running : max_blocks;
  for (uint32_t b = block_running + lane; b < max_blocks; b += 64) {
    blocks[3 * b + 0] = 0xffffffffu;
    blocks[3 * b + 1] = 0;
    blocks[3 * b + 2] = 0;
  }
}

}  // namespace

void launch_route_pack(hipStream_t s, const View &indices, uint32_t rows, uint32_t k,
                       uint32_t experts, uint32_t tile_rows, uint32_t *counts, uint32_t *offsets,
                       uint32_t *sorted_routes, uint32_t *blocks, uint32_t max_blocks,
                       uint32_t *n_blocks, ErrorSlot *error) {
  size_t lds = (size_t)experts * 2 * sizeof(uint32_t);
  route_pack_kernel<<<dim3(1), 64, lds, s>>>(indices, rows, k, experts, tile_rows, counts, offsets,
                                             sorted_routes, blocks, max_blocks, n_blocks, error);
}

}  // namespace fh
