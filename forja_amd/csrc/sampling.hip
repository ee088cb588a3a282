// Op::Sample / Op::SampleMasked: one token per row by Gumbel-max over counter-based noise, after
// temperature, top-k and top-p, following crates/forja-cpu/src/lib.rs:1545-1700 step by step:
//
//   * parameters are live device words (temperature, top_k, top_p, seed) and are validated when
//     the dispatch runs (SamplingParameters::from_words, lib.rs:1553-1575), as is the allow mask
//     (validate_allow_mask, lib.rs:1639-1652); a refusal is recorded in the dispatch's error slot;
//   * temperature 0 or top_k 1: the largest value, the largest index among equals;
//   * otherwise the candidates are ordered by descending value, ties by descending index
//     (lib.rs:1616-1620), cut to top_k, then to the shortest prefix whose probability reaches
//     top_p, with the weights and both running sums accumulated in f32 in that order
//     (truncate_top_p, lib.rs:1654-1679), because the cut depends on the rounding of those sums;
//   * the winner maximises logit / temperature - ln(-ln(u)), u from splitmix64 of
//     seed ^ position << 32 ^ index (sampled_score, lib.rs:1681-1692); non-finite logits keep
//     their own value as score.
//
// One workgroup of 1024 threads per row.  Ordering work is only done when the cut needs it: no
// ordering for "all candidates, top_p = 1"; up to 256 candidates are extracted largest first by
// repeated block-wide maxima; more than that takes a stable LSD radix sort of (value key, index)
// pairs in global scratch, after which one lane walks the sums through LDS-staged weights.
// exp and ln are evaluated in f64 and rounded to f32, i.e. the correctly rounded f32 functions up
// to double rounding; an f32 libm may differ from that in the last place.
#include <hip/hip_runtime.h>

#include "kernels.hpp"

namespace fh {

namespace {

constexpr uint32_t kSampleThreads = 1024;
constexpr uint32_t kSampleWaves = kSampleThreads / 64;
constexpr uint32_t kSmallCandidates = 256;
constexpr uint32_t kStage = 4096;

struct SampleArgs {
  View logits;             // [rows, width]
  View out;                // u32, `rows` elements in logical order
  const uint32_t *params;  // temperature bits, top_k, top_p bits, seed low, seed high
  uint64_t param_stride;   // elements between consecutive parameter words
  const uint32_t *allow;   // one bit per column, or null
  uint2 *scratch;          // [gridDim.x][2][width] (inverted value key, index)
  uint32_t rows, width, position;
};

struct alignas(16) SampleShared {
  uint32_t wave_count[kSampleWaves][256];
  uint32_t base[256];
  alignas(16) float stage[kStage];
  uint64_t small[kSmallCandidates];
  float small_weight[kSmallCandidates];
  uint64_t reduce[kSampleWaves];
  uint32_t word[4];
  float real[2];
};

__device__ inline uint32_t ordered_key(float value) {
  return (uint32_t)total_key(value) ^ 0x80000000u;
}

// (value, index) as one unsigned number ordered like total_cmp then index; +1 so that 0 is "none"
// (an index never reaches 2^32 - 1, so the sum cannot wrap).
__device__ inline uint64_t candidate(float value, uint32_t index) {
  return (((uint64_t)ordered_key(value) << 32) | index) + 1;
}

__device__ inline bool is_finite(float value) {
  return (__float_as_uint(value) & 0x7f800000u) != 0x7f800000u;
}

__device__ inline uint64_t splitmix64(uint64_t value) {
  value += 0x9e3779b97f4a7c15ull;
  value = (value ^ (value >> 30)) * 0xbf58476d1ce4e5b9ull;
  value = (value ^ (value >> 27)) * 0x94d049bb133111ebull;
  return value ^ (value >> 31);
}

__device__ inline float sampled_score(float logit, float temperature, uint64_t seed,
                                      uint32_t position, uint32_t index) {
  if (!is_finite(logit)) return logit;
  const uint64_t counter = seed ^ ((uint64_t)position << 32) ^ (uint64_t)index;
  const uint32_t mantissa = (uint32_t)(splitmix64(counter) >> 40);
  const float uniform = ((float)mantissa + 0.5f) * (1.0f / 16777216.0f);
  const float inner = (float)log((double)uniform);
  const float outer = (float)log((double)(-inner));
  return logit / temperature - outer;
}

// Largest value over the workgroup, known to every thread afterwards.
__device__ inline uint64_t block_max(uint64_t mine, SampleShared &s) {
  for (int offset = 32; offset > 0; offset >>= 1) {
    uint64_t other = __shfl_xor(mine, offset, 64);
    mine = other > mine ? other : mine;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s.reduce[threadIdx.x >> 6] = mine;
  __syncthreads();
  uint64_t best = s.reduce[0];
  for (uint32_t wave = 1; wave < kSampleWaves; ++wave)
    best = s.reduce[wave] > best ? s.reduce[wave] : best;
  return best;
}

__device__ inline uint32_t block_sum(uint32_t mine, SampleShared &s) {
  for (int offset = 32; offset > 0; offset >>= 1) mine += __shfl_xor(mine, offset, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) s.reduce[threadIdx.x >> 6] = mine;
  __syncthreads();
  uint32_t total = 0;
  for (uint32_t wave = 0; wave < kSampleWaves; ++wave) total += (uint32_t)s.reduce[wave];
  return total;
}

struct Row {
  const SampleArgs &a;
  uint64_t base;
  bool vector;  // bf16 with unit column stride and a 16-byte aligned start: eight values per load
  __device__ float value(uint32_t index) const {
    return load_float_at(a.logits, base + (uint64_t)index * a.logits.stride[1]);
  }
  __device__ bool allowed(uint32_t index) const {
    return a.allow == nullptr || ((a.allow[index >> 5] >> (index & 31)) & 1u) != 0;
  }
  // The columns of the row are dealt to the 1024 threads in fixed hands (eight adjacent columns
  // at a time where the row can be read in 16-byte pieces).  visit(index, value) for every
  // allowed column of thread `owner`'s hand, taking pieces first, first + step, ...
  template <typename Visit>
  __device__ void for_hand(uint32_t owner, uint32_t first, uint32_t step, Visit visit) const {
    uint32_t done = 0;
    if (vector) {
      const uint16_t *x = (const uint16_t *)a.logits.base + base;
      done = a.width & ~7u;
#pragma unroll 4
      for (uint64_t c = owner * 8 + (uint64_t)first * kSampleThreads * 8; c < done;
           c += (uint64_t)step * kSampleThreads * 8) {
        const uint4 v = *(const uint4 *)(x + c);
        const uint32_t words[4] = {v.x, v.y, v.z, v.w};
        const uint32_t permitted = a.allow ? (a.allow[c >> 5] >> (c & 31)) & 0xffu : 0xffu;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if ((permitted >> (2 * i)) & 1u)
            visit((uint32_t)c + 2 * i, __uint_as_float(words[i] << 16));
          if ((permitted >> (2 * i + 1)) & 1u)
            visit((uint32_t)c + 2 * i + 1, __uint_as_float(words[i] & 0xffff0000u));
        }
      }
    }
    for (uint64_t index = done + owner + (uint64_t)first * kSampleThreads; index < a.width;
         index += (uint64_t)step * kSampleThreads)
      if (allowed((uint32_t)index)) visit((uint32_t)index, value((uint32_t)index));
  }
  // visit(index, value) for every allowed column, each exactly once over the workgroup
  template <typename Visit>
  __device__ void for_each_allowed(Visit visit) const {
    for_hand(threadIdx.x, 0, 1, visit);
  }
  // Largest candidate below `below` in the hand of thread `owner`, found by the calling wave
  // together (one piece per lane at a time); every lane of the wave gets the result.
  __device__ uint64_t best_of_hand_below(uint32_t owner, uint64_t below) const {
    uint64_t next = 0;
    for_hand(owner, threadIdx.x & 63, 64, [&](uint32_t index, float value) {
      const uint64_t mine = candidate(value, index);
      if (mine < below && mine > next) next = mine;
    });
    for (int offset = 32; offset > 0; offset >>= 1) {
      const uint64_t other = __shfl_xor(next, offset, 64);
      next = other > next ? other : next;
    }
    return next;
  }
};

// One tile of a stable counting scatter: the thread's element (if `valid`) goes to
// s.base[digit] + (elements of the same digit held by lower threads of the tile), and s.base
// advances by the tile's count of every digit.
__device__ inline void scatter_tile(bool valid, uint32_t digit, uint2 element, uint2 *target,
                                    SampleShared &s) {
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (uint32_t slot = threadIdx.x; slot < kSampleWaves * 256; slot += kSampleThreads)
    (&s.wave_count[0][0])[slot] = 0;
  unsigned long long same = __ballot(valid);
  for (uint32_t bit = 0; bit < 8; ++bit) {
    const bool set = ((digit >> bit) & 1u) != 0;
    const unsigned long long with = __ballot(valid && set);
    same &= set ? with : ~with;
  }
  const uint32_t rank = (uint32_t)__popcll(same & ((1ull << lane) - 1ull));
  __syncthreads();
  if (valid && rank == 0) s.wave_count[wave][digit] = (uint32_t)__popcll(same);
  __syncthreads();
  if (threadIdx.x < 256) {
    uint32_t running = s.base[threadIdx.x];
    for (uint32_t w = 0; w < kSampleWaves; ++w) {
      const uint32_t count = s.wave_count[w][threadIdx.x];
      s.wave_count[w][threadIdx.x] = running;
      running += count;
    }
    s.base[threadIdx.x] = running;
  }
  __syncthreads();
  if (valid) target[s.wave_count[wave][digit] + rank] = element;
  __syncthreads();
}

// Walks `count` weights (read through `weight_at`) in order on lane 0: first their f32 sum, then
// the first position where the running sum of weight / total reaches top_p.  Returns the number
// of leading candidates kept (truncate_top_p, lib.rs:1654-1679).
template <typename WeightAt>
__device__ inline uint32_t top_p_keep(uint32_t count, float top_p, WeightAt weight_at,
                                      SampleShared &s) {
  const float4 *staged = (const float4 *)s.stage;
  float total = 0.0f;
  for (uint32_t first = 0; first < count; first += kStage) {
    const uint32_t chunk = min(kStage, count - first);
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < kStage; i += kSampleThreads)
      s.stage[i] = i < chunk ? weight_at(first + i) : 0.0f;
    __syncthreads();
    if (threadIdx.x == 0) {
      // adding the +0.0 padding of the last chunk changes nothing: the weights are not negative
#pragma unroll 4
      for (uint32_t i = 0; i < (chunk + 3) / 4; ++i) {
        const float4 v = staged[i];
        total += v.x;
        total += v.y;
        total += v.z;
        total += v.w;
      }
    }
  }
  if (threadIdx.x == 0) {
    s.real[0] = total;
    s.word[0] = 0xffffffffu;
  }
  __syncthreads();
  total = s.real[0];
  if (!(is_finite(total) && total > 0.0f)) return 1;
  float cumulative = 0.0f;
  for (uint32_t first = 0; first < count; first += kStage) {
    const uint32_t chunk = min(kStage, count - first);
    __syncthreads();
    // the quotients are independent of each other: every thread divides, one lane accumulates
    for (uint32_t i = threadIdx.x; i < chunk; i += kSampleThreads)
      s.stage[i] = weight_at(first + i) / total;
    __syncthreads();
    if (threadIdx.x == 0) {
      for (uint32_t i = 0; i < chunk; ++i) {
        cumulative += s.stage[i];
        if (cumulative >= top_p) {
          s.word[0] = first + i;
          break;
        }
      }
    }
    __syncthreads();
    if (s.word[0] != 0xffffffffu) break;
  }
  const uint32_t position = s.word[0];
  return position == 0xffffffffu ? count : position + 1;
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(SampleArgs a, ErrorSlot *error) {
  __shared__ SampleShared s;
  // ---- live parameters (identical for every row)
  const float temperature = __uint_as_float(a.params[0]);
  const uint32_t top_k = a.params[a.param_stride];
  const float top_p = __uint_as_float(a.params[2 * a.param_stride]);
  const uint64_t seed =
      (uint64_t)a.params[3 * a.param_stride] | ((uint64_t)a.params[4 * a.param_stride] << 32);
  bool refused = !is_finite(temperature) || temperature < 0.0f || !is_finite(top_p) ||
                 !(top_p >= 0.0f && top_p <= 1.0f) || top_p == 0.0f;
  if (a.allow != nullptr) {
    const uint32_t words = (a.width + 31) / 32, remainder = a.width % 32;
    uint32_t any = 0;
    for (uint32_t word = threadIdx.x; word < words; word += kSampleThreads) any |= a.allow[word];
    const uint32_t set = block_sum(any != 0 ? 1u : 0u, s);
    if (set == 0) refused = true;
    if (remainder != 0 && (a.allow[words - 1] & ~((1u << remainder) - 1u)) != 0) refused = true;
  }
  if (refused) {
    if (threadIdx.x == 0 && blockIdx.x == 0) report_error(error, 0);
    return;
  }
  const bool greedy = temperature == 0.0f || top_k == 1;
  uint2 *sorted = a.scratch + (uint64_t)blockIdx.x * 2 * a.width;
  uint2 *other = sorted + a.width;

  for (uint32_t row_index = blockIdx.x; row_index < a.rows; row_index += gridDim.x) {
    const uint64_t row_base = a.logits.offset + (uint64_t)row_index * a.logits.stride[0];
    const Row row{a, row_base,
                  a.logits.dtype == FH_BF16 && a.logits.stride[1] == 1 &&
                      (((uint64_t)a.logits.base + row_base * 2) & 15u) == 0};
    uint32_t *out = (uint32_t *)a.out.base + view_offset(a.out, row_index);
    if (greedy) {
      uint64_t best = 0;
      row.for_each_allowed([&](uint32_t index, float value) {
        const uint64_t mine = candidate(value, index);
        best = mine > best ? mine : best;
      });
      best = block_max(best, s);
      if (threadIdx.x == 0) *out = (uint32_t)(best - 1);
      continue;
    }
    // ---- how many candidates survive top_k
    uint32_t limit = top_k;  // 0: all
    if (top_k == 0 || top_k > kSmallCandidates) {
      uint32_t allowed = a.width;
      if (a.allow != nullptr) {
        uint32_t mine = 0;
        for (uint32_t index = threadIdx.x; index < a.width; index += kSampleThreads)
          mine += row.allowed(index) ? 1u : 0u;
        allowed = block_sum(mine, s);
      }
      limit = top_k == 0 ? allowed : min(top_k, allowed);
      if (limit == allowed && !(top_p < 1.0f)) {
        // every allowed column competes: no ordering needed
        uint64_t best = 0;
        row.for_each_allowed([&](uint32_t index, float value) {
          const uint64_t mine =
              candidate(sampled_score(value, temperature, seed, a.position, index), index);
          best = mine > best ? mine : best;
        });
        best = block_max(best, s);
        if (threadIdx.x == 0) *out = (uint32_t)(best - 1);
        continue;
      }
    }
    if (limit <= kSmallCandidates) {
      // ---- the `limit` largest, extracted one by one in descending order.  Every thread keeps
      // the best of its own columns that is still below the last extracted candidate; a round is
      // one block-wide maximum, after which the winner's wave looks through the winner's columns
      // again, one piece per lane.
      uint64_t local = 0;
      row.for_each_allowed([&](uint32_t index, float value) {
        const uint64_t mine = candidate(value, index);
        local = mine > local ? mine : local;
      });
      uint32_t count = 0;
      for (; count < limit; ++count) {
        const uint64_t best = block_max(local, s);
        if (best == 0) break;
        if (threadIdx.x == 0) s.small[count] = best - 1;
        const unsigned long long owners = __ballot(local == best);   // one lane of one wave
        if (owners != 0) {
          const uint32_t owner_lane = (uint32_t)__ffsll((long long)owners) - 1;
          const uint64_t next =
              row.best_of_hand_below((threadIdx.x & ~63u) + owner_lane, best);
          if ((threadIdx.x & 63) == owner_lane) local = next;
        }
      }
      __syncthreads();
      if (top_p < 1.0f) {
        const float maximum = row.value((uint32_t)s.small[0]);
        if (threadIdx.x < count)
          s.small_weight[threadIdx.x] = (float)exp(
              (double)((row.value((uint32_t)s.small[threadIdx.x]) - maximum) / temperature));
        __syncthreads();
        const uint32_t keep = top_p_keep(count, top_p, [&](uint32_t i) { return s.small_weight[i]; }, s);
        count = min(count, max(keep, 1u));
      }
      uint64_t best = 0;
      if (threadIdx.x < count) {
        const uint32_t index = (uint32_t)s.small[threadIdx.x];
        best = candidate(sampled_score(row.value(index), temperature, seed, a.position, index), index);
      }
      best = block_max(best, s);
      if (threadIdx.x == 0) *out = (uint32_t)(best - 1);
      __syncthreads();
      continue;
    }
    // ---- general case: order all allowed columns.  Start from descending index so that the
    // stable passes leave equal values in descending index order.
    if (threadIdx.x < 256) s.base[threadIdx.x] = 0;
    __syncthreads();
    for (uint32_t first = 0; first < a.width; first += kSampleThreads) {
      const uint32_t at = first + threadIdx.x;
      const bool in_range = at < a.width;
      const uint32_t index = in_range ? a.width - 1 - at : 0;
      const bool valid = in_range && row.allowed(index);
      uint2 element = make_uint2(0, index);
      if (valid) element.x = ~ordered_key(row.value(index));
      scatter_tile(valid, 0, element, sorted, s);
    }
    const uint32_t allowed = s.base[0];
    uint2 *from = sorted, *to = other;
    for (uint32_t shift = 0; shift < 32; shift += 8) {
      __syncthreads();
      if (threadIdx.x < 256) s.base[threadIdx.x] = 0;
      __syncthreads();
      for (uint32_t i = threadIdx.x; i < allowed; i += kSampleThreads)
        atomicAdd(&s.base[(from[i].x >> shift) & 255u], 1u);
      __syncthreads();
      if (threadIdx.x == 0) {
        uint32_t running = 0;
        for (uint32_t digit = 0; digit < 256; ++digit) {
          const uint32_t count = s.base[digit];
          s.base[digit] = running;
          running += count;
        }
      }
      __syncthreads();
      for (uint32_t first = 0; first < allowed; first += kSampleThreads) {
        const uint32_t at = first + threadIdx.x;
        const bool valid = at < allowed;
        const uint2 element = valid ? from[at] : make_uint2(0, 0);
        scatter_tile(valid, (element.x >> shift) & 255u, element, to, s);
      }
      uint2 *swap = from;
      from = to;
      to = swap;
    }
    // four passes: the ordered pairs are back in `sorted`, `other` is free for the weights
    uint32_t count = min(limit, allowed);
    if (top_p < 1.0f) {
      float *weights = (float *)other;
      const float maximum = row.value(sorted[0].y);
      for (uint32_t i = threadIdx.x; i < count; i += kSampleThreads)
        weights[i] = (float)exp((double)((row.value(sorted[i].y) - maximum) / temperature));
      __syncthreads();
      const uint32_t keep = top_p_keep(count, top_p, [&](uint32_t i) { return weights[i]; }, s);
      count = min(count, max(keep, 1u));
    }
    uint64_t best = 0;
    for (uint32_t i = threadIdx.x; i < count; i += kSampleThreads) {
      const uint32_t index = sorted[i].y;
      const uint64_t mine =
          candidate(sampled_score(row.value(index), temperature, seed, a.position, index), index);
      best = mine > best ? mine : best;
    }
    best = block_max(best, s);
    if (threadIdx.x == 0) *out = (uint32_t)(best - 1);
    __syncthreads();
  }
}

}  // namespace

uint64_t sample_scratch_bytes(uint32_t rows, uint32_t width) {
  return (uint64_t)(rows < kSampleGrid ? rows : kSampleGrid) * 2 * width * sizeof(uint2);
}

void launch_sample(hipStream_t stream, const View &logits, const View &params, const View *allow,
                   const View &out, uint32_t rows, uint32_t width, uint32_t position,
                   void *scratch, ErrorSlot *error) {
  if (rows == 0 || width == 0) return;
  SampleArgs a{};
  a.logits = logits;
  a.out = out;
  a.params = (const uint32_t *)params.base + params.offset;
  a.param_stride = params.stride[0];
  a.allow = allow ? (const uint32_t *)allow->base + allow->offset : nullptr;
  a.scratch = (uint2 *)scratch;
  a.rows = rows;
  a.width = width;
  a.position = position;
  sample_kernel<<<dim3(rows < kSampleGrid ? rows : kSampleGrid), kSampleThreads, 0, stream>>>(a, error);
}

}  // namespace fh
