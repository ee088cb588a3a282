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

// One workgroup of 16 waves does the whole plan in a single launch: at decode sizes (a few
// thousand routes) everything fits one or two 1024-route rounds, and what matters is the number
// of dependent memory round trips, not throughput.
constexpr uint32_t kPackThreads = 1024, kPackWaves = kPackThreads / 64;

__global__ __launch_bounds__(1024) void route_pack_kernel(
    View indices, uint32_t rows, uint32_t k, uint32_t experts, uint32_t tile_rows, uint32_t *counts,
    uint32_t *offsets, uint32_t *sorted_routes, uint32_t *blocks, uint32_t max_blocks,
    uint32_t *n_blocks, uint32_t *zero_rows, uint32_t zero_row_words, ErrorSlot *error) {
  extern __shared__ uint32_t lds[];
  uint32_t *lds_counts = lds;                    // [experts]
  uint32_t *lds_cursor = lds + experts;          // [experts] next free position per expert
  uint32_t *wave_counts = lds + 2 * experts;     // [kPackWaves][experts] per round
  uint32_t *scan = lds + (2 + kPackWaves) * experts;  // [kPackWaves + 1]
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t routes = rows * k;
  auto expert_of = [&](uint32_t route) {
    return load_u32_at(indices, indices.offset + (uint64_t)(route / k) * indices.stride[0] +
                                    (uint64_t)(route % k) * indices.stride[1]);
  };
  for (uint32_t e = tid; e < experts; e += kPackThreads) lds_counts[e] = 0;
  __syncthreads();
  // the first round's expert ids stay in a register for the arrange pass
  const uint32_t first_expert = tid < routes ? expert_of(tid) : 0xffffffffu;
  for (uint32_t route = tid; route < routes; route += kPackThreads) {
    const uint32_t expert = route == tid ? first_expert : expert_of(route);
    if (expert >= experts) {
      report_error(error, expert);
      // a bad route is never packed: its output row (if the caller has one) is cleared here
      if (zero_rows)
        for (uint32_t w = 0; w < zero_row_words; ++w) zero_rows[(uint64_t)route * zero_row_words + w] = 0;
    } else
      atomicAdd(&lds_counts[expert], 1u);
  }
  __syncthreads();
  // Exclusive scans over the experts of the route counts (-> offsets) and of the tile counts
  // (-> first row block of each expert): one expert per thread per round, wave scans stitched
  // through LDS.
  uint32_t running = 0, block_running = 0;
  for (uint32_t base = 0; base < experts; base += kPackThreads) {
    const uint32_t e = base + tid;
    const uint32_t c = e < experts ? lds_counts[e] : 0;
    const uint32_t tiles = (c + tile_rows - 1) / tile_rows;
    uint32_t inclusive = c, inclusive_tiles = tiles;
    for (int offset = 1; offset < 64; offset <<= 1) {
      const uint32_t other = __shfl_up(inclusive, offset, 64);
      const uint32_t other_tiles = __shfl_up(inclusive_tiles, offset, 64);
      if ((int)lane >= offset) {
        inclusive += other;
        inclusive_tiles += other_tiles;
      }
    }
    if (lane == 63) {
      scan[wave] = inclusive;
      scan[kPackWaves + 1 + wave] = inclusive_tiles;
    }
    __syncthreads();
    uint32_t before = running, before_tiles = block_running, total = 0, total_tiles = 0;
    for (uint32_t w = 0; w < kPackWaves; ++w) {
      if (w < wave) {
        before += scan[w];
        before_tiles += scan[kPackWaves + 1 + w];
      }
      total += scan[w];
      total_tiles += scan[kPackWaves + 1 + w];
    }
    if (e < experts) {
      const uint32_t start = before + inclusive - c;
      counts[e] = c;
      offsets[e] = start;
      lds_cursor[e] = start;
      const uint32_t first = before_tiles + inclusive_tiles - tiles;
      for (uint32_t t = 0; t < tiles; ++t) {
        const uint32_t b = first + t;
        if (b >= max_blocks) break;
        const uint32_t remaining = c - t * tile_rows;
        blocks[3 * b + 0] = e;
        blocks[3 * b + 1] = start + t * tile_rows;
        blocks[3 * b + 2] = remaining < tile_rows ? remaining : tile_rows;
      }
    }
    running += total;
    block_running += total_tiles;
    __syncthreads();
  }
  if (tid == 0) {
    offsets[experts] = running;
    n_blocks[0] = block_running < max_blocks ? block_running : max_blocks;
  }
  for (uint32_t b = block_running + tid; b < max_blocks; b += kPackThreads) {
    blocks[3 * b + 0] = 0xffffffffu;
    blocks[3 * b + 1] = 0;
    blocks[3 * b + 2] = 0;
  }
  // Stable arrange, 1024 routes per round in ascending route order: a route's position is its
  // expert's cursor + the routes of the same expert in lower waves of the round + its rank among
  // the lower lanes of its own wave.
  for (uint32_t base = 0; base < routes; base += kPackThreads) {
    const uint32_t route = base + tid;
    for (uint32_t i = tid; i < kPackWaves * experts; i += kPackThreads) wave_counts[i] = 0;
    uint32_t expert = 0xffffffffu;
    if (route < routes) expert = base == 0 ? first_expert : expert_of(route);
    const bool valid = route < routes && expert < experts;
    unsigned long long same = __ballot(valid);
    for (uint32_t bit = 0; (experts - 1) >> bit; ++bit) {
      const unsigned long long set = __ballot(valid && ((expert >> bit) & 1u));
      same &= ((expert >> bit) & 1u) ? set : ~set;
    }
    const uint32_t rank = __popcll(same & ((1ull << lane) - 1ull));
    __syncthreads();  // wave_counts cleared
    if (valid && rank == 0) wave_counts[wave * experts + expert] = __popcll(same);
    __syncthreads();
    if (valid) {
      uint32_t position = lds_cursor[expert] + rank;
      for (uint32_t w = 0; w < wave; ++w) position += wave_counts[w * experts + expert];
      sorted_routes[position] = route;
    }
    __syncthreads();
    for (uint32_t e = tid; e < experts; e += kPackThreads) {
      uint32_t added = 0;
      for (uint32_t w = 0; w < kPackWaves; ++w) added += wave_counts[w * experts + e];
      lds_cursor[e] += added;
    }
    __syncthreads();
  }
}

}  // namespace

void launch_route_pack(hipStream_t s, const View &indices, uint32_t rows, uint32_t k,
                       uint32_t experts, uint32_t tile_rows, uint32_t *counts, uint32_t *offsets,
                       uint32_t *sorted_routes, uint32_t *blocks, uint32_t max_blocks,
                       uint32_t *n_blocks, ErrorSlot *error, uint32_t *zero_rows,
                       uint32_t zero_row_words) {
  size_t lds = ((size_t)experts * (2 + kPackWaves) + 2 * (kPackWaves + 1)) * sizeof(uint32_t);
  route_pack_kernel<<<dim3(1), kPackThreads, lds, s>>>(indices, rows, k, experts, tile_rows, counts, offsets,
                                             sorted_routes, blocks, max_blocks, n_blocks, zero_rows,
                                             zero_row_words, error);
}

}  // namespace fh
