/*
 * CPU restatement of forja-cpu for the ragged continuous-batch forward step.
 * TEST INFRASTRUCTURE ONLY: see forja_cpu_oracle.h.  Build: gcc -O2 -ffp-contract=off -fopenmp.
 *
 * OpenMP only ever splits work over *independent output elements*; each element is still one
 * sequential left-to-right f32 fold, so results are bit-identical for any thread count.
 * orc_set_threads(1) gives the reference's single-threaded execution for baseline timing.
 *
 * Pinning of each routine (exercised in tests/test_oracle_golden.py):
 *   conversions ........ exhaustive bf16 round trip, RNE ties, f16 subnormals; reference test
 *                        paged_copy_converts_directly_into_reduced_storage (lib.rs:1883-1924)
 *   quant dot / matmul . quant_matmul_dequantizes_q4_and_q8_in_mlx_order (lib.rs:2786-2845);
 *                        numpy float64 dequantise-then-matmul; tiny-model fixture vectors
 *   gather variants .... lib.rs:2848-2951 ([256,320,0,64,256,320], bad index 7),
 *                        lib.rs:2954-3017 ([473.5,582.0])
 *   top-k / argmax ..... lib.rs:2386-2447 (ties, NaN payload order, normalise closed form)
 *   route pack ......... closed form: numpy stable argsort
 *   page table / copy .. core paged.rs:381-420, lib.rs:1883-1924, cpu paged.rs:408-419
 *   paged sdpa ......... cpu paged.rs:457-476 (e/(e+1)), lib.rs:1926-1970, numpy float64 softmax
 *   interpreter ........ interpreter.rs:437-609 ([1e20,-1e20,3] -> 3), lib.rs:2688-2711
 *   rms_norm / rope .... lib.rs:2688-2757 (float64 independent computation)
 */
#include "forja_cpu_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 0; /* 0 = OpenMP default */

void orc_set_threads(int threads) {
  g_threads = threads;
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#endif
}

/* ------------------------------------------------------------------ conversions */

static uint32_t f32_bits(float value) {
  uint32_t bits;
  memcpy(&bits, &value, 4);
  return bits;
}

static float bits_f32(uint32_t bits) {
  float value;
  memcpy(&value, &bits, 4);
  return value;
}

/* half::bf16::from_f32: NaN keeps its top payload bits and is forced quiet; otherwise
 * round-to-nearest-even on bit 16. */
uint16_t orc_f32_to_bf16(float value) {
  uint32_t x = f32_bits(value);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
  uint32_t round_bit = 0x00008000u;
  if ((x & round_bit) != 0 && (x & (3 * round_bit - 1)) != 0) return (uint16_t)((x >> 16) + 1);
  return (uint16_t)(x >> 16);
}

float orc_bf16_to_f32(uint16_t bits) {
  if ((bits & 0x7fffu) > 0x7f80u) return bits_f32(((uint32_t)bits | 0x0040u) << 16);
  return bits_f32((uint32_t)bits << 16);
}

/* half::f16::from_f32 (software path): RNE, overflow to infinity, gradual underflow. */
uint16_t orc_f32_to_f16(float value) {
  uint32_t x = f32_bits(value);
  uint32_t sign = x & 0x80000000u;
  uint32_t exp = x & 0x7f800000u;
  uint32_t man = x & 0x007fffffu;
  if (exp == 0x7f800000u) {
    uint32_t nan_bit = man == 0 ? 0 : 0x0200u;
    return (uint16_t)((sign >> 16) | 0x7c00u | nan_bit | (man >> 13));
  }
  uint32_t half_sign = sign >> 16;
  int32_t unbiased = (int32_t)(exp >> 23) - 127;
  int32_t half_exp = unbiased + 15;
  if (half_exp >= 0x1f) return (uint16_t)(half_sign | 0x7c00u);
  if (half_exp <= 0) {
    if (14 - half_exp > 24) return (uint16_t)half_sign;
    man |= 0x00800000u;
    uint32_t half_man = man >> (14 - half_exp);
    uint32_t round_bit = 1u << (13 - half_exp);
    if ((man & round_bit) != 0 && (man & (3 * round_bit - 1)) != 0) half_man += 1;
    return (uint16_t)(half_sign | half_man);
  }
  uint32_t he = (uint32_t)half_exp << 10;
  uint32_t hm = man >> 13;
  uint32_t round_bit = 0x00001000u;
  if ((man & round_bit) != 0 && (man & (3 * round_bit - 1)) != 0)
    return (uint16_t)((half_sign | he | hm) + 1);
  return (uint16_t)(half_sign | he | hm);
}

float orc_f16_to_f32(uint16_t bits) {
  uint32_t i = bits;
  if ((i & 0x7fffu) == 0) return bits_f32(i << 16);
  uint32_t half_sign = i & 0x8000u;
  uint32_t half_exp = i & 0x7c00u;
  uint32_t half_man = i & 0x03ffu;
  if (half_exp == 0x7c00u) {
    if (half_man == 0) return bits_f32((half_sign << 16) | 0x7f800000u);
    return bits_f32((half_sign << 16) | 0x7fc00000u | (half_man << 13));
  }
  uint32_t sign = half_sign << 16;
  int32_t unbiased = (int32_t)(half_exp >> 10) - 15;
  if (half_exp == 0) {
    /* subnormal: normalise */
    int e = 0;
    uint32_t m = half_man;
    while ((m & 0x0400u) == 0) {
      m <<= 1;
      e += 1;
    }
    m &= 0x03ffu;
    uint32_t exp = (uint32_t)(127 - 15 - e + 1) << 23;
    return bits_f32(sign | exp | (m << 13));
  }
  uint32_t exp = (uint32_t)(unbiased + 127) << 23;
  return bits_f32(sign | exp | (half_man << 13));
}

int orc_decode(const void *source, int dtype, size_t count, float *out) {
  switch (dtype) {
  case ORC_F32:
    memcpy(out, source, count * 4);
    return ORC_OK;
  case ORC_F16:
    for (size_t i = 0; i < count; ++i) out[i] = orc_f16_to_f32(((const uint16_t *)source)[i]);
    return ORC_OK;
  case ORC_BF16:
    for (size_t i = 0; i < count; ++i) out[i] = orc_bf16_to_f32(((const uint16_t *)source)[i]);
    return ORC_OK;
  default:
    return ORC_EXECUTION_FAILED;
  }
}

int orc_encode(const float *source, int dtype, size_t count, void *out) {
  switch (dtype) {
  case ORC_F32:
    memcpy(out, source, count * 4);
    return ORC_OK;
  case ORC_F16:
    for (size_t i = 0; i < count; ++i) ((uint16_t *)out)[i] = orc_f32_to_f16(source[i]);
    return ORC_OK;
  case ORC_BF16:
    for (size_t i = 0; i < count; ++i) ((uint16_t *)out)[i] = orc_f32_to_bf16(source[i]);
    return ORC_OK;
  default:
    return ORC_EXECUTION_FAILED;
  }
}

/* ------------------------------------------------------------------ strided views */

static uint64_t element_count(int rank, const uint32_t *shape) {
  uint64_t count = 1;
  for (int axis = 0; axis < rank; ++axis) count *= shape[axis];
  return count;
}

/* element_offsets (lib.rs:1736-1745): row-major logical order, last axis fastest. */
static uint64_t element_offset(uint64_t linear, int rank, const uint32_t *shape,
                               const uint64_t *strides, uint64_t offset) {
  for (int axis = rank - 1; axis >= 0; --axis) {
    offset += (linear % shape[axis]) * strides[axis];
    linear /= shape[axis];
  }
  return offset;
}

int orc_gather(const uint8_t *source, size_t source_len, int elem_size, int rank,
               const uint32_t *shape, const uint64_t *strides, uint64_t offset, uint8_t *out) {
  uint64_t count = element_count(rank, shape);
  for (uint64_t linear = 0; linear < count; ++linear) {
    uint64_t start = element_offset(linear, rank, shape, strides, offset) * (uint64_t)elem_size;
    if (start + (uint64_t)elem_size > source_len) return ORC_INVALID_INPUT;
    memcpy(out + linear * (uint64_t)elem_size, source + start, (size_t)elem_size);
  }
  return ORC_OK;
}

int orc_scatter(uint8_t *target, size_t target_len, int elem_size, int rank, const uint32_t *shape,
                const uint64_t *strides, uint64_t offset, const uint8_t *source) {
  uint64_t count = element_count(rank, shape);
  for (uint64_t linear = 0; linear < count; ++linear) {
    uint64_t start = element_offset(linear, rank, shape, strides, offset) * (uint64_t)elem_size;
    if (start + (uint64_t)elem_size > target_len) return ORC_INVALID_INPUT;
    memcpy(target + start, source + linear * (uint64_t)elem_size, (size_t)elem_size);
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------ quantised matmul */

/* affine_quant_dot (lib.rs:1277-1310): value i lives in bits [bits*(i%vpw), ...) of word i/vpw;
 * the dequantised weight scale*q+bias is formed in f32 first, then multiplied and added. */
float orc_affine_quant_dot(const float *activation, size_t inner, const uint32_t *packed,
                           const float *scales, const float *biases, size_t packed_row,
                           size_t group_row, size_t group_size, int bits) {
  size_t values_per_word = 32u / (size_t)bits;
  uint32_t mask = (1u << bits) - 1u;
  float sum = 0.0f;
  for (size_t index = 0; index < inner; ++index) {
    uint32_t word = packed[packed_row + index / values_per_word];
    uint32_t shift = (uint32_t)((index % values_per_word) * (size_t)bits);
    uint32_t quantized = (word >> shift) & mask;
    size_t group = group_row + index / group_size;
    float weight = scales[group] * (float)quantized + biases[group];
    sum = sum + activation[index] * weight;
  }
  return sum;
}

int orc_quant_matmul(const float *x, const uint32_t *packed, const float *scales,
                     const float *biases, size_t rows, size_t inner, size_t columns, int bits,
                     size_t group_size, float *out) {
  if ((bits != 4 && bits != 8) || group_size == 0 || inner % group_size != 0)
    return ORC_INVALID_INPUT;
  size_t packed_width = inner * (size_t)bits / 32u;
  size_t group_count = inner / group_size;
  long total = (long)(rows * columns);
#pragma omp parallel for schedule(static)
  for (long flat = 0; flat < total; ++flat) {
    size_t row = (size_t)flat / columns, column = (size_t)flat % columns;
    out[flat] = orc_affine_quant_dot(x + row * inner, inner, packed, scales, biases,
                                     column * packed_width, column * group_count, group_size,
                                     bits);
  }
  return ORC_OK;
}

static void record_invalid(uint32_t invalid[2], uint32_t index) {
  if (!invalid[0] || index < invalid[1]) invalid[1] = index;
  invalid[0] = 1;
}

/* gather_quant_projection_values (lib.rs:1025-1106). */
int orc_gather_quant_projection(const float *x, const uint32_t *packed, const float *scales,
                                const float *biases, const uint32_t *indices, size_t rows,
                                size_t inner, size_t experts, size_t columns, size_t k, int bits,
                                size_t group_size, float *out, uint32_t invalid[2]) {
  if ((bits != 4 && bits != 8) || group_size == 0 || inner % group_size != 0)
    return ORC_INVALID_INPUT;
  size_t packed_width = inner * (size_t)bits / 32u;
  size_t group_count = inner / group_size;
  size_t expert_packed = columns * packed_width;
  size_t expert_groups = columns * group_count;
  invalid[0] = 0;
  invalid[1] = 0;
  for (size_t route = 0; route < rows * k; ++route)
    if (indices[route] >= experts) record_invalid(invalid, indices[route]);
  long total = (long)(rows * k * columns);
#pragma omp parallel for schedule(static)
  for (long flat = 0; flat < total; ++flat) {
    size_t route = (size_t)flat / columns, column = (size_t)flat % columns;
    size_t row = route / k;
    uint32_t expert = indices[route];
    if (expert >= experts) {
      out[flat] = 0.0f;
      continue;
    }
    out[flat] = orc_affine_quant_dot(x + row * inner, inner, packed, scales, biases,
                                     expert * expert_packed + column * packed_width,
                                     expert * expert_groups + column * group_count, group_size,
                                     bits);
  }
  return ORC_OK;
}

/* execute_gather_quant_weighted_sum (lib.rs:1108-1204): routes are folded in ascending slot
 * order, `destination += weight * value`, starting from the residual or zero. */
int orc_gather_quant_weighted_sum(const float *x, const uint32_t *packed, const float *scales,
                                  const float *biases, const uint32_t *indices,
                                  const float *weights, const float *residual, size_t rows,
                                  size_t routes, size_t inner, size_t experts, size_t columns,
                                  int bits, size_t group_size, float *out, uint32_t invalid[2]) {
  if ((bits != 4 && bits != 8) || group_size == 0 || inner % group_size != 0)
    return ORC_INVALID_INPUT;
  size_t packed_width = inner * (size_t)bits / 32u;
  size_t group_count = inner / group_size;
  size_t expert_packed = columns * packed_width;
  size_t expert_groups = columns * group_count;
  invalid[0] = 0;
  invalid[1] = 0;
  for (size_t route = 0; route < rows * routes; ++route)
    if (indices[route] >= experts) record_invalid(invalid, indices[route]);
  long total = (long)(rows * columns);
#pragma omp parallel for schedule(static)
  for (long flat = 0; flat < total; ++flat) {
    size_t row = (size_t)flat / columns, column = (size_t)flat % columns;
    float value = residual ? residual[flat] : 0.0f;
    for (size_t route = 0; route < routes; ++route) {
      size_t route_offset = row * routes + route;
      uint32_t expert = indices[route_offset];
      if (expert >= experts) continue;
      float dot = orc_affine_quant_dot(x + route_offset * inner, inner, packed, scales, biases,
                                       expert * expert_packed + column * packed_width,
                                       expert * expert_groups + column * group_count, group_size,
                                       bits);
      value += weights[route_offset] * dot;
    }
    out[flat] = value;
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------ selection */

/* f32::total_cmp key: IEEE-754 totalOrder as a signed integer comparison. */
static int32_t total_key(float value) {
  int32_t bits = (int32_t)f32_bits(value);
  return bits ^ (int32_t)(((uint32_t)(bits >> 31)) >> 1);
}

/* execute_argmax (lib.rs:519-550): Iterator::max_by keeps the last maximal element. */
int orc_argmax(const float *values, size_t rows, size_t width, uint32_t *out) {
  if (width == 0) return ORC_EXECUTION_FAILED;
  for (size_t row = 0; row < rows; ++row) {
    const float *r = values + row * width;
    size_t best = 0;
    for (size_t index = 1; index < width; ++index)
      if (total_key(r[index]) >= total_key(r[best])) best = index;
    out[row] = (uint32_t)best;
  }
  return ORC_OK;
}

typedef struct {
  int32_t key;
  uint32_t index;
} topk_item;

static int topk_compare(const void *left, const void *right) {
  const topk_item *l = (const topk_item *)left, *r = (const topk_item *)right;
  if (l->key != r->key) return l->key > r->key ? -1 : 1; /* descending value */
  return l->index < r->index ? -1 : (l->index > r->index ? 1 : 0);
}

/* ---- Op::Sample / Op::SampleMasked (crates/forja-cpu/src/lib.rs:1545-1700) ----
 * Pinned by the reference's own tests restated in tests/test_oracle_golden.py: the chi-squared
 * checks against known probabilities (lib.rs:2636-2662, 3283-3306), the exact truncation sets of
 * top_k / top_p, masks in every mode, the all-allowed mask, mask refusals, the 1025-candidate
 * nucleus, counter determinism and the parameter refusals; plus the closed form P(i) =
 * softmax(logits / T) at other temperatures and the max_by tie rule.
 * PARITY UNPINNED: the token drawn for a given seed.  The reference holds no token vectors and
 * does not promise tokens across builds or backends (crates/forja-core/src/ops.rs:206-208); a
 * slip in the counter formula that keeps the noise uniform would pass every check above. */

/* SamplingParameters::from_words (lib.rs:1553-1575). */
static int sampling_parameters(const uint32_t words[5], float *temperature, uint32_t *top_k,
                               float *top_p, uint64_t *seed) {
  memcpy(temperature, &words[0], 4);
  memcpy(top_p, &words[2], 4);
  if (!isfinite(*temperature) || *temperature < 0.0f || !isfinite(*top_p) ||
      !(*top_p >= 0.0f && *top_p <= 1.0f) || *top_p == 0.0f)
    return ORC_INVALID_INPUT;
  *top_k = words[1];
  *seed = (uint64_t)words[3] | ((uint64_t)words[4] << 32);
  return ORC_OK;
}

/* validate_allow_mask (lib.rs:1639-1652). */
int orc_validate_allow_mask(const uint32_t *allow, size_t words, size_t width) {
  size_t remainder = width % 32;
  if (remainder != 0 &&
      (words == 0 || (allow[words - 1] & ~((1u << remainder) - 1u)) != 0))
    return ORC_INVALID_INPUT;
  for (size_t word = 0; word < words; ++word)
    if (allow[word] != 0) return ORC_OK;
  return ORC_INVALID_INPUT;
}

/* f32::ln and f32::exp go to the platform's libm, whose f32 routines are not correctly rounded
 * and differ between platforms in the last place (the reference says as much: tokens are not
 * promised across builds, ops.rs:206-208).  The restatement uses the correctly rounded value
 * (f64 evaluation rounded once), the function those routines approximate. */
static float ln_f32(float value) { return (float)log((double)value); }
static float exp_f32(float value) { return (float)exp((double)value); }

/* sampled_score (lib.rs:1681-1692): Gumbel-max noise from a counter-based stream. */
static float sampled_score(float logit, float temperature, uint64_t seed, uint32_t position,
                           size_t index) {
  if (!isfinite(logit)) return logit;
  uint64_t counter = seed ^ ((uint64_t)position << 32) ^ (uint64_t)index;
  uint64_t random = orc_splitmix64(counter);
  uint32_t mantissa = (uint32_t)(random >> 40);
  float uniform = ((float)mantissa + 0.5f) * (1.0f / 16777216.0f);
  return logit / temperature - ln_f32(-ln_f32(uniform));
}

typedef struct {
  int32_t key;
  uint32_t index;
} sample_item;

/* sort_unstable_by(row[right].total_cmp(row[left]).then(right.cmp(left))) (lib.rs:1616-1620):
 * descending value, ties by descending index; the order is total, so stability is moot. */
static int sample_compare(const void *left, const void *right) {
  const sample_item *l = (const sample_item *)left, *r = (const sample_item *)right;
  if (l->key != r->key) return l->key > r->key ? -1 : 1;
  return l->index > r->index ? -1 : (l->index < r->index ? 1 : 0);
}

/* truncate_top_p (lib.rs:1654-1679): number of leading candidates kept. */
static size_t top_p_keep(const float *row, const sample_item *sorted, size_t count,
                         float temperature, float top_p, float *weights) {
  if (count == 0) return 0;
  float maximum = row[sorted[0].index];
  float total = 0.0f;
  for (size_t i = 0; i < count; ++i) {
    weights[i] = exp_f32((row[sorted[i].index] - maximum) / temperature);
    total += weights[i];
  }
  if (!(isfinite(total) && total > 0.0f)) return 1;
  float cumulative = 0.0f;
  for (size_t i = 0; i < count; ++i) {
    cumulative += weights[i] / total;
    if (cumulative >= top_p) return i + 1;
  }
  return count;
}

/* The candidates truncate_top_p keeps out of a whole row (for the reference's own test of it). */
int orc_top_p_keep(const float *row, size_t width, float temperature, float top_p, size_t *keep) {
  sample_item *items = (sample_item *)malloc((width + 1) * sizeof(sample_item));
  float *weights = (float *)malloc((width + 1) * sizeof(float));
  if (!items || !weights) {
    free(items);
    free(weights);
    return ORC_EXECUTION_FAILED;
  }
  for (size_t i = 0; i < width; ++i) {
    items[i].key = total_key(row[i]);
    items[i].index = (uint32_t)i;
  }
  qsort(items, width, sizeof(sample_item), sample_compare);
  *keep = top_p_keep(row, items, width, temperature, top_p, weights);
  free(items);
  free(weights);
  return ORC_OK;
}

/* sample_allowed (lib.rs:1599-1637) over the indices `allow` permits (all when null). */
int orc_sample_row(const float *row, size_t width, const uint32_t params[5], uint32_t position,
                   const uint32_t *allow, uint32_t *out) {
  float temperature, top_p;
  uint32_t top_k;
  uint64_t seed;
  int status = sampling_parameters(params, &temperature, &top_k, &top_p, &seed);
  if (status != ORC_OK) return status;
  sample_item *items = (sample_item *)malloc((width + 1) * sizeof(sample_item));
  float *weights = (float *)malloc((width + 1) * sizeof(float));
  if (!items || !weights) {
    free(items);
    free(weights);
    return ORC_EXECUTION_FAILED;
  }
  size_t count = 0;
  for (size_t i = 0; i < width; ++i) {
    if (allow && !(allow[i / 32] & (1u << (i % 32)))) continue;
    items[count].key = total_key(row[i]);
    items[count].index = (uint32_t)i;
    ++count;
  }
  status = ORC_OK;
  if (temperature == 0.0f || top_k == 1) {
    /* max_by(total_cmp.then(index)): the largest value, the largest index among equals */
    if (count == 0) {
      status = ORC_INVALID_INPUT;
    } else {
      size_t best = 0;
      for (size_t i = 1; i < count; ++i)
        if (items[i].key >= items[best].key) best = i;
      *out = items[best].index;
    }
  } else {
    qsort(items, count, sizeof(sample_item), sample_compare);
    size_t cap = top_k == 0 ? count : (size_t)top_k;
    if (cap < count) count = cap;
    if (top_p < 1.0f) {
      size_t keep = top_p_keep(row, items, count, temperature, top_p, weights);
      if (count == 0) status = ORC_EXECUTION_FAILED;
      if (keep < 1) keep = 1;
      if (keep < count) count = keep;
    }
    if (count == 0) {
      if (status == ORC_OK) status = ORC_EXECUTION_FAILED;
    } else {
      size_t best = 0;
      int32_t best_key = 0;
      for (size_t i = 0; i < count; ++i) {
        int32_t key = total_key(sampled_score(row[items[i].index], temperature, seed, position,
                                              items[i].index));
        if (i == 0 || key > best_key ||
            (key == best_key && items[i].index > items[best].index)) {
          best = i;
          best_key = key;
        }
      }
      *out = items[best].index;
    }
  }
  free(items);
  free(weights);
  return status;
}

/* execute_sample / execute_sample_masked (lib.rs:610-678): one parameter block for all rows. */
int orc_sample(const float *values, size_t rows, size_t width, const uint32_t params[5],
               uint32_t position, const uint32_t *allow, uint32_t *out) {
  if (width == 0) return ORC_EXECUTION_FAILED;
  float temperature, top_p;
  uint32_t top_k;
  uint64_t seed;
  int status = sampling_parameters(params, &temperature, &top_k, &top_p, &seed);
  if (status != ORC_OK) return status;
  if (allow) {
    status = orc_validate_allow_mask(allow, (width + 31) / 32, width);
    if (status != ORC_OK) return status;
  }
  for (size_t row = 0; row < rows; ++row) {
    status = orc_sample_row(values + row * width, width, params, position, allow, &out[row]);
    if (status != ORC_OK) return status;
  }
  return ORC_OK;
}

/* execute_top_k (lib.rs:552-608). */
int orc_top_k(const float *values, size_t rows, size_t width, size_t k, int normalize,
              float *out_values, uint32_t *out_indices) {
  if (k == 0 || k > width) return ORC_EXECUTION_FAILED;
  topk_item *items = (topk_item *)malloc(width * sizeof(topk_item));
  if (!items) return ORC_EXECUTION_FAILED;
  for (size_t row = 0; row < rows; ++row) {
    const float *r = values + row * width;
    for (size_t index = 0; index < width; ++index) {
      items[index].key = total_key(r[index]);
      items[index].index = (uint32_t)index;
    }
    qsort(items, width, sizeof(topk_item), topk_compare);
    float *selected = out_values + row * k;
    for (size_t slot = 0; slot < k; ++slot) {
      selected[slot] = r[items[slot].index];
      out_indices[row * k + slot] = items[slot].index;
    }
    if (normalize) {
      float maximum = selected[0];
      for (size_t slot = 0; slot < k; ++slot) selected[slot] = expf(selected[slot] - maximum);
      float sum = 0.0f;
      for (size_t slot = 0; slot < k; ++slot) sum += selected[slot];
      for (size_t slot = 0; slot < k; ++slot) selected[slot] /= sum;
    }
  }
  free(items);
  return ORC_OK;
}

/* ------------------------------------------------------------------ route packing */

long orc_route_pack(const uint32_t *indices, size_t rows, size_t k, size_t experts,
                    size_t tile_rows, uint32_t *counts, uint32_t *offsets,
                    uint32_t *sorted_routes, uint32_t *blocks, size_t max_blocks,
                    uint32_t invalid[2]) {
  if (tile_rows == 0) return -ORC_INVALID_INPUT;
  size_t routes = rows * k;
  invalid[0] = 0;
  invalid[1] = 0;
  memset(counts, 0, experts * sizeof(uint32_t));
  for (size_t route = 0; route < routes; ++route) {
    if (indices[route] >= experts)
      record_invalid(invalid, indices[route]);
    else
      counts[indices[route]] += 1;
  }
  offsets[0] = 0;
  for (size_t expert = 0; expert < experts; ++expert)
    offsets[expert + 1] = offsets[expert] + counts[expert];
  uint32_t *cursor = (uint32_t *)malloc((experts + 1) * sizeof(uint32_t));
  if (!cursor) return -ORC_EXECUTION_FAILED;
  memcpy(cursor, offsets, (experts + 1) * sizeof(uint32_t));
  for (size_t route = 0; route < routes; ++route)
    if (indices[route] < experts) sorted_routes[cursor[indices[route]]++] = (uint32_t)route;
  free(cursor);
  size_t block = 0;
  for (size_t expert = 0; expert < experts; ++expert) {
    for (uint32_t start = 0; start < counts[expert]; start += (uint32_t)tile_rows) {
      if (block >= max_blocks) return -ORC_INVALID_INPUT;
      uint32_t remaining = counts[expert] - start;
      blocks[3 * block + 0] = (uint32_t)expert;
      blocks[3 * block + 1] = offsets[expert] + start;
      blocks[3 * block + 2] = remaining < tile_rows ? remaining : (uint32_t)tile_rows;
      block += 1;
    }
  }
  return (long)block;
}

/* ------------------------------------------------------------------ paged storage */

#define POISON_GENERATION 0xffffffffu

static int validate_entry(uint32_t page, uint32_t generation, const uint32_t *generations,
                          size_t physical_pages) {
  if (page >= physical_pages) return ORC_INVALID_INPUT;
  if (generations[page] != generation) return ORC_INVALID_INPUT;
  return ORC_OK;
}

/* PageTable::from_padded (core paged.rs:97-121): every non-poison entry of the fixed-width table
 * is authenticated, whether or not the operation will touch it.  cpu_page_table maps a refusal to
 * ExecutionFailed (lib.rs:1534). */
int orc_page_table_from_padded(const uint32_t *entries, size_t logical_pages,
                               const uint32_t *generations, size_t physical_pages) {
  for (size_t logical = 0; logical < logical_pages; ++logical) {
    uint32_t page = entries[2 * logical], generation = entries[2 * logical + 1];
    if (page != 0 || generation != POISON_GENERATION)
      if (validate_entry(page, generation, generations, physical_pages) != ORC_OK)
        return ORC_EXECUTION_FAILED;
  }
  return ORC_OK;
}

/* PageTable::resolve (core paged.rs:146-163): rechecks the generation, so a poison entry is
 * refused when dereferenced. */
int orc_page_table_resolve(const uint32_t *entries, size_t logical_pages,
                           const uint32_t *generations, size_t physical_pages,
                           uint32_t logical_page, uint32_t *physical) {
  if (logical_page >= logical_pages) return ORC_INVALID_INPUT;
  uint32_t page = entries[2 * (size_t)logical_page];
  if (validate_entry(page, entries[2 * (size_t)logical_page + 1], generations, physical_pages))
    return ORC_INVALID_INPUT;
  *physical = page;
  return ORC_OK;
}

/* CpuPagePool::token_range (cpu paged.rs:283-315). */
static int token_start(size_t physical_pages, size_t page_tokens, size_t row_bytes,
                       const uint32_t *entries, size_t logical_pages, const uint32_t *generations,
                       uint64_t logical_token, uint64_t *start) {
  uint64_t logical_page = logical_token / page_tokens;
  if (logical_page > 0xffffffffull) return ORC_INVALID_INPUT;
  uint32_t physical;
  int status = orc_page_table_resolve(entries, logical_pages, generations, physical_pages,
                                      (uint32_t)logical_page, &physical);
  if (status) return status;
  *start = (uint64_t)physical * page_tokens * row_bytes + (logical_token % page_tokens) * row_bytes;
  return ORC_OK;
}

int orc_paged_copy_in(uint8_t *pool, size_t physical_pages, size_t page_tokens, size_t row_bytes,
                      const uint32_t *entries, size_t logical_pages, const uint32_t *generations,
                      uint64_t start, uint64_t tokens, const uint8_t *rows) {
  for (uint64_t token = 0; token < tokens; ++token) {
    uint64_t destination;
    int status = token_start(physical_pages, page_tokens, row_bytes, entries, logical_pages,
                             generations, start + token, &destination);
    if (status) return status;
    memcpy(pool + destination, rows + token * row_bytes, row_bytes);
  }
  return ORC_OK;
}

int orc_paged_copy_out(const uint8_t *pool, size_t physical_pages, size_t page_tokens,
                       size_t row_bytes, const uint32_t *entries, size_t logical_pages,
                       const uint32_t *generations, uint64_t start, uint64_t tokens,
                       uint8_t *rows) {
  for (uint64_t token = 0; token < tokens; ++token) {
    uint64_t source;
    int status = token_start(physical_pages, page_tokens, row_bytes, entries, logical_pages,
                             generations, start + token, &source);
    if (status) return status;
    memcpy(rows + token * row_bytes, pool + source, row_bytes);
  }
  return ORC_OK;
}

static size_t dtype_size(int dtype) { return dtype == ORC_F32 ? 4 : 2; }

static float load_element(const void *base, int dtype, uint64_t element) {
  switch (dtype) {
  case ORC_F32:
    return ((const float *)base)[element];
  case ORC_F16:
    return orc_f16_to_f32(((const uint16_t *)base)[element]);
  default:
    return orc_bf16_to_f32(((const uint16_t *)base)[element]);
  }
}

/* CpuPagePool::sdpa (cpu paged.rs:161-259) with its softmax (:378-388). */
int orc_paged_sdpa(const float *query, const void *key_pool, const void *value_pool,
                   int key_dtype, int value_dtype, size_t physical_pages, size_t page_tokens,
                   const uint32_t *entries, size_t logical_pages, const uint32_t *generations,
                   uint32_t query_heads, uint32_t query_length, uint32_t kv_heads, uint32_t width,
                   uint32_t value_width, uint32_t key_length, uint32_t query_start, float scale,
                   int causal, float *out) {
  if (query_heads == 0 || kv_heads == 0 || query_heads % kv_heads != 0 || !isfinite(scale))
    return ORC_INVALID_INPUT;
  if (key_dtype > ORC_BF16 || value_dtype > ORC_BF16) return ORC_INVALID_INPUT;
  uint32_t heads_per_group = query_heads / kv_heads;
  size_t key_row = (size_t)kv_heads * width, value_row = (size_t)kv_heads * value_width;
  /* Resolve every attended token once; a refusal anywhere fails the whole op, as in the
   * reference where `load` propagates the error. */
  uint32_t longest = key_length;
  if (causal) {
    uint64_t last = (uint64_t)query_start + query_length;
    if (query_length == 0) last = 0;
    if (last < longest) longest = (uint32_t)last;
  }
  uint64_t *rows = (uint64_t *)malloc(((size_t)longest + 1) * sizeof(uint64_t));
  if (!rows) return ORC_EXECUTION_FAILED;
  for (uint32_t token = 0; token < longest; ++token) {
    uint64_t start;
    int status = token_start(physical_pages, page_tokens, 1, entries, logical_pages, generations,
                             token, &start);
    if (status) {
      free(rows);
      return status;
    }
    rows[token] = start; /* pool row index */
  }
  int failed = 0;
  long work = (long)query_heads * (long)query_length;
#pragma omp parallel for schedule(dynamic, 1)
  for (long item = 0; item < work; ++item) {
    uint32_t head = (uint32_t)(item / query_length), query_row = (uint32_t)(item % query_length);
    uint32_t kv_head = head / heads_per_group;
    const float *q = query + ((size_t)head * query_length + query_row) * width;
    uint32_t attended = key_length;
    if (causal) {
      uint64_t limit = (uint64_t)query_start + query_row + 1;
      if (limit < attended) attended = (uint32_t)limit;
    }
    float *scores = (float *)malloc(((size_t)attended + 1) * sizeof(float));
    if (!scores) {
      failed = 1;
      continue;
    }
    for (uint32_t key = 0; key < attended; ++key) {
      float score = 0.0f;
      uint64_t base = rows[key] * key_row + (uint64_t)kv_head * width;
      for (uint32_t column = 0; column < width; ++column)
        score += q[column] * load_element(key_pool, key_dtype, base + column);
      scores[key] = score * scale;
    }
    float maximum = -INFINITY;
    for (uint32_t key = 0; key < attended; ++key) maximum = fmaxf(maximum, scores[key]);
    float sum = 0.0f;
    for (uint32_t key = 0; key < attended; ++key) {
      scores[key] = expf(scores[key] - maximum);
      sum += scores[key];
    }
    for (uint32_t key = 0; key < attended; ++key) scores[key] /= sum;
    float *o = out + ((size_t)head * query_length + query_row) * value_width;
    for (uint32_t column = 0; column < value_width; ++column) {
      float acc = 0.0f;
      for (uint32_t key = 0; key < attended; ++key)
        acc += scores[key] * load_element(value_pool, value_dtype,
                                          rows[key] * value_row + (uint64_t)kv_head * value_width +
                                              column);
      o[column] = acc;
    }
    free(scores);
  }
  free(rows);
  (void)dtype_size;
  return failed ? ORC_EXECUTION_FAILED : ORC_OK;
}

/* ------------------------------------------------------------------ scalar programs */

typedef struct {
  int type; /* 0 f32, 1 u32, 2 bool */
  union {
    float f;
    uint32_t u;
  } v;
} scalar;

static float propagating_min(float l, float r) { return (isnan(l) || isnan(r)) ? NAN : fminf(l, r); }
static float propagating_max(float l, float r) { return (isnan(l) || isnan(r)) ? NAN : fmaxf(l, r); }

static uint32_t saturating_u32(float value) {
  if (isnan(value) || value <= 0.0f) return 0;
  if (value >= 4294967296.0f) return 0xffffffffu;
  return (uint32_t)value;
}

static int eval_unary(uint32_t op, scalar in, scalar *out) {
  if (in.type != 0) return ORC_EXECUTION_FAILED;
  float x = in.v.f, y;
  switch (op) {
  case 0: y = -x; break;
  case 1: y = fabsf(x); break;
  case 2: case 13: y = expf(x); break;
  case 3: y = logf(x); break;
  case 4: y = sqrtf(x); break;
  case 5: y = 1.0f / sqrtf(x); break;
  case 6: y = sinf(x); break;
  case 7: y = cosf(x); break;
  case 8: y = tanhf(x); break;
  case 9: y = 1.0f / (1.0f + expf(-x)); break;
  case 10: y = 1.0f / x; break;
  case 11: y = floorf(x); break;
  case 12: y = log1pf(x); break;
  default: return ORC_EXECUTION_FAILED;
  }
  out->type = 0;
  out->v.f = y;
  return ORC_OK;
}

static int eval_binary(uint32_t op, scalar l, scalar r, scalar *out) {
  if (l.type == 0 && r.type == 0) {
    float a = l.v.f, b = r.v.f;
    out->type = op >= 7 ? 2 : 0;
    switch (op) {
    case 0: out->v.f = a + b; break;
    case 1: out->v.f = a - b; break;
    case 2: out->v.f = a * b; break;
    case 3: out->v.f = a / b; break;
    case 4: out->v.f = propagating_min(a, b); break;
    case 5: out->v.f = propagating_max(a, b); break;
    case 6: out->v.f = powf(a, b); break;
    case 7: out->v.u = a < b; break;
    case 8: out->v.u = a <= b; break;
    case 9: out->v.u = a == b; break;
    case 10: out->v.u = a != b; break;
    case 11: out->v.u = a >= b; break;
    case 12: out->v.u = a > b; break;
    default: return ORC_EXECUTION_FAILED;
    }
    return ORC_OK;
  }
  if (l.type == 1 && r.type == 1) {
    uint32_t a = l.v.u, b = r.v.u;
    out->type = op >= 7 ? 2 : 1;
    switch (op) {
    case 0: out->v.u = a + b; break;
    case 1: out->v.u = a - b; break;
    case 2: out->v.u = a * b; break;
    case 4: out->v.u = a < b ? a : b; break;
    case 5: out->v.u = a > b ? a : b; break;
    case 7: out->v.u = a < b; break;
    case 8: out->v.u = a <= b; break;
    case 9: out->v.u = a == b; break;
    case 10: out->v.u = a != b; break;
    case 11: out->v.u = a >= b; break;
    case 12: out->v.u = a > b; break;
    default: return ORC_EXECUTION_FAILED; /* div, pow */
    }
    return ORC_OK;
  }
  return ORC_EXECUTION_FAILED;
}

static scalar eval_cast(uint32_t to, scalar in) {
  scalar out;
  out.type = (int)to;
  switch (to) {
  case 0:
    out.v.f = in.type == 0 ? in.v.f : (in.type == 1 ? (float)in.v.u : (in.v.u ? 1.0f : 0.0f));
    break;
  case 1:
    out.v.u = in.type == 0 ? saturating_u32(in.v.f) : (in.type == 1 ? in.v.u : (in.v.u ? 1u : 0u));
    break;
  default:
    out.v.u = in.type == 0 ? (in.v.f != 0.0f) : (in.v.u != 0);
    break;
  }
  return out;
}

static int eval_inst(const orc_inst *inst, const uint32_t *coordinates, int rank,
                     const uint32_t *shape, const orc_program_input *inputs, size_t input_count,
                     size_t linear, const scalar *values, size_t produced, scalar *out) {
  switch (inst->kind) {
  case 0:
    if (inst->a >= input_count) return ORC_EXECUTION_FAILED;
    if (inputs[inst->a].is_u32) {
      out->type = 1;
      out->v.u = ((const uint32_t *)inputs[inst->a].data)[linear];
    } else {
      out->type = 0;
      out->v.f = ((const float *)inputs[inst->a].data)[linear];
    }
    return ORC_OK;
  case 1:
    out->type = 0;
    out->v.f = bits_f32(inst->a);
    return ORC_OK;
  case 2:
    if ((int)inst->op >= rank) return ORC_EXECUTION_FAILED;
    out->type = 1;
    out->v.u = coordinates[inst->op];
    return ORC_OK;
  case 3:
    if ((int)inst->op >= rank) return ORC_EXECUTION_FAILED;
    out->type = 1;
    out->v.u = shape[inst->op];
    return ORC_OK;
  case 4:
    if (inst->a >= produced) return ORC_EXECUTION_FAILED;
    return eval_unary(inst->op, values[inst->a], out);
  case 5:
    if (inst->a >= produced || inst->b >= produced) return ORC_EXECUTION_FAILED;
    return eval_binary(inst->op, values[inst->a], values[inst->b], out);
  case 6:
    if (inst->a >= produced || inst->b >= produced || inst->c >= produced)
      return ORC_EXECUTION_FAILED;
    if (values[inst->a].type != 2) return ORC_EXECUTION_FAILED;
    *out = values[inst->a].v.u ? values[inst->b] : values[inst->c];
    return ORC_OK;
  case 7:
    if (inst->a >= produced) return ORC_EXECUTION_FAILED;
    *out = eval_cast(inst->op, values[inst->a]);
    return ORC_OK;
  default:
    return ORC_EXECUTION_FAILED;
  }
}

static void decode_coordinates(size_t linear, int rank, const uint32_t *shape,
                               uint32_t *coordinates) {
  for (int axis = rank - 1; axis >= 0; --axis) {
    coordinates[axis] = (uint32_t)(linear % shape[axis]);
    linear /= shape[axis];
  }
}

/* interpret_map / interpret_row (interpreter.rs:38-150).  Row programs evaluate instruction by
 * instruction across the whole row ("columns"); a reduction folds its operand column left to
 * right in f32 and broadcasts the result. */
int orc_interpret(int program_kind, const orc_inst *insts, size_t inst_count,
                  const uint32_t *outputs, size_t output_pairs, size_t output_count, int rank,
                  const uint32_t *shape, const orc_program_input *inputs, size_t input_count,
                  float *const *out) {
  if (rank <= 0 || rank > 8 || inst_count == 0 || inst_count > 256) return ORC_EXECUTION_FAILED;
  size_t elements = (size_t)element_count(rank, shape);
  for (size_t pair = 0; pair < output_pairs; ++pair)
    if (outputs[2 * pair] >= output_count || outputs[2 * pair + 1] >= inst_count)
      return ORC_EXECUTION_FAILED;
  uint32_t coordinates[8];
  if (program_kind == 0) {
    scalar values[256];
    for (size_t linear = 0; linear < elements; ++linear) {
      decode_coordinates(linear, rank, shape, coordinates);
      for (size_t index = 0; index < inst_count; ++index) {
        if (insts[index].kind == 8) return ORC_EXECUTION_FAILED;
        int status = eval_inst(&insts[index], coordinates, rank, shape, inputs, input_count,
                               linear, values, index, &values[index]);
        if (status) return status;
      }
      for (size_t pair = 0; pair < output_pairs; ++pair) {
        scalar value = values[outputs[2 * pair + 1]];
        if (value.type != 0) return ORC_EXECUTION_FAILED;
        out[outputs[2 * pair]][linear] = value.v.f;
      }
    }
    return ORC_OK;
  }
  size_t row_width = shape[rank - 1];
  if (row_width == 0) return ORC_EXECUTION_FAILED;
  size_t row_count = elements / row_width;
  scalar *columns = (scalar *)malloc(inst_count * row_width * sizeof(scalar));
  scalar lane_values[256];
  if (!columns) return ORC_EXECUTION_FAILED;
  int status = ORC_OK;
  for (size_t row = 0; row < row_count && !status; ++row) {
    size_t row_start = row * row_width;
    for (size_t index = 0; index < inst_count && !status; ++index) {
      scalar *column = columns + index * row_width;
      if (insts[index].kind == 8) {
        if (insts[index].a >= index) {
          status = ORC_EXECUTION_FAILED;
          break;
        }
        const scalar *operand = columns + (size_t)insts[index].a * row_width;
        if (operand[0].type != 0) {
          status = ORC_EXECUTION_FAILED;
          break;
        }
        float acc;
        if (insts[index].op == 0) {
          acc = 0.0f;
          for (size_t lane = 0; lane < row_width; ++lane) acc = acc + operand[lane].v.f;
        } else {
          acc = operand[0].v.f;
          for (size_t lane = 1; lane < row_width; ++lane)
            acc = insts[index].op == 1 ? propagating_max(acc, operand[lane].v.f)
                                       : propagating_min(acc, operand[lane].v.f);
        }
        for (size_t lane = 0; lane < row_width; ++lane) {
          column[lane].type = 0;
          column[lane].v.f = acc;
        }
        continue;
      }
      for (size_t lane = 0; lane < row_width; ++lane) {
        size_t linear = row_start + lane;
        decode_coordinates(linear, rank, shape, coordinates);
        /* gather this lane's earlier values only for the operands the instruction names */
        const orc_inst *inst = &insts[index];
        if (inst->kind >= 4) {
          if (inst->a < index) lane_values[inst->a] = columns[(size_t)inst->a * row_width + lane];
          if (inst->kind == 5 || inst->kind == 6)
            if (inst->b < index) lane_values[inst->b] = columns[(size_t)inst->b * row_width + lane];
          if (inst->kind == 6)
            if (inst->c < index) lane_values[inst->c] = columns[(size_t)inst->c * row_width + lane];
        }
        status = eval_inst(inst, coordinates, rank, shape, inputs, input_count, linear,
                           lane_values, index, &column[lane]);
        if (status) break;
      }
    }
    if (status) break;
    for (size_t pair = 0; pair < output_pairs; ++pair) {
      const scalar *column = columns + (size_t)outputs[2 * pair + 1] * row_width;
      for (size_t lane = 0; lane < row_width; ++lane) {
        if (column[lane].type != 0) {
          status = ORC_EXECUTION_FAILED;
          break;
        }
        out[outputs[2 * pair]][row_start + lane] = column[lane].v.f;
      }
    }
  }
  free(columns);
  return status;
}

/* ------------------------------------------------------------------ glue */

/* execute_rms_norm (lib.rs:495-517): the count is accumulated as f32 ones. */
int orc_rms_norm(const float *values, const float *weights, size_t rows, size_t width, float eps,
                 float *out) {
  for (size_t row = 0; row < rows; ++row) {
    const float *r = values + row * width;
    float sum = 0.0f, count = 0.0f;
    for (size_t index = 0; index < width; ++index) sum = sum + r[index] * r[index];
    for (size_t index = 0; index < width; ++index) count = count + 1.0f;
    float scale = 1.0f / sqrtf(sum / count + eps);
    for (size_t index = 0; index < width; ++index)
      out[row * width + index] = r[index] * scale * weights[index];
  }
  return ORC_OK;
}

/* execute_rope (lib.rs:681-710): half-split pairs (i, i+width/2). */
int orc_rope(float *values, const uint32_t *positions, size_t rows, size_t heads, size_t width,
             float theta) {
  size_t half = width / 2;
  for (size_t row = 0; row < rows; ++row) {
    for (size_t head = 0; head < heads; ++head) {
      float *h = values + (row * heads + head) * width;
      for (size_t index = 0; index < half; ++index) {
        float frequency = 1.0f / powf(theta, 2.0f * (float)index / (float)width);
        float angle = (float)positions[row] * frequency;
        float s = sinf(angle), c = cosf(angle);
        float first = h[index], second = h[index + half];
        h[index] = first * c - second * s;
        h[index + half] = second * c + first * s;
      }
    }
  }
  return ORC_OK;
}

/* execute_quant_embed (lib.rs:748-813). */
int orc_quant_embed(const uint32_t *packed, const float *scales, const float *biases,
                    const uint32_t *ids, size_t id_count, size_t vocab, size_t packed_width,
                    int bits, size_t group_size, float *out, uint32_t invalid[2]) {
  if ((bits != 4 && bits != 8) || group_size == 0) return ORC_INVALID_INPUT;
  size_t values_per_word = 32u / (size_t)bits;
  size_t width = packed_width * values_per_word;
  size_t groups = width / group_size;
  uint32_t mask = (1u << bits) - 1u;
  invalid[0] = 0;
  invalid[1] = 0;
  for (size_t item = 0; item < id_count; ++item) {
    float *row_out = out + item * width;
    uint32_t id = ids[item];
    if (id >= vocab) {
      memset(row_out, 0, width * sizeof(float));
      record_invalid(invalid, id);
      continue;
    }
    for (size_t column = 0; column < width; ++column) {
      uint32_t word = packed[(size_t)id * packed_width + column / values_per_word];
      uint32_t quantized = (word >> ((column % values_per_word) * (size_t)bits)) & mask;
      size_t group = (size_t)id * groups + column / group_size;
      row_out[column] = scales[group] * (float)quantized + biases[group];
    }
  }
  return ORC_OK;
}

/* execute_matmul (lib.rs:815-848): rank-3 batches of [rows,inner]x[inner,columns]. */
int orc_matmul(const float *left, const float *right, size_t batches, size_t rows, size_t inner,
               size_t columns, float *out) {
  for (size_t batch = 0; batch < batches; ++batch) {
    const float *l = left + batch * rows * inner, *r = right + batch * inner * columns;
    float *o = out + batch * rows * columns;
    for (size_t row = 0; row < rows; ++row)
      for (size_t column = 0; column < columns; ++column) {
        float sum = 0.0f;
        for (size_t index = 0; index < inner; ++index)
          sum = sum + l[row * inner + index] * r[index * columns + column];
        o[row * columns + column] = sum;
      }
  }
  return ORC_OK;
}

/* ------------------------------------------------------------------ seeded synthetic data */

uint64_t orc_splitmix64(uint64_t value) {
  value += 0x9e3779b97f4a7c15ull;
  value = (value ^ (value >> 30)) * 0xbf58476d1ce4e5b9ull;
  value = (value ^ (value >> 27)) * 0x94d049bb133111ebull;
  return value ^ (value >> 31);
}

/* Counter-based: any element of any stream is computable independently. */
uint64_t orc_stream_u64(uint64_t seed, uint64_t stream, uint64_t index) {
  uint64_t key = orc_splitmix64(seed + 0x632be59bd9b4e019ull * (stream + 1));
  return orc_splitmix64(key ^ index);
}

void orc_fill_words(uint64_t seed, uint64_t stream, uint64_t first, size_t count, uint32_t *out) {
  for (size_t i = 0; i < count; ++i) out[i] = (uint32_t)(orc_stream_u64(seed, stream, first + i) >> 32);
}

static float uniform_value(uint64_t seed, uint64_t stream, uint64_t index, float lo, float hi) {
  float unit = (float)(orc_stream_u64(seed, stream, index) >> 40) * (1.0f / 16777216.0f);
  float span = hi - lo;
  float scaled = unit * span;
  return lo + scaled;
}

/* Irwin-Hall(8) on 16-bit lanes: integer sum, one subtraction, one multiplication - no
 * transcendental, so host and device produce identical bits.  Mean 0, variance 1. */
static float normal_value(uint64_t seed, uint64_t stream, uint64_t index) {
  uint64_t a = orc_stream_u64(seed, stream, 2 * index), b = orc_stream_u64(seed, stream, 2 * index + 1);
  int32_t sum = 0;
  for (int lane = 0; lane < 4; ++lane) {
    sum += (int32_t)((a >> (16 * lane)) & 0xffff);
    sum += (int32_t)((b >> (16 * lane)) & 0xffff);
  }
  float centred = (float)(sum - 262140);
  return centred * (1.0f / 53509.91796875f);
}

void orc_fill_uniform_bf16(uint64_t seed, uint64_t stream, uint64_t first, size_t count, float lo,
                           float hi, uint16_t *out) {
  for (size_t i = 0; i < count; ++i)
    out[i] = orc_f32_to_bf16(uniform_value(seed, stream, first + i, lo, hi));
}

void orc_fill_normal_bf16(uint64_t seed, uint64_t stream, uint64_t first, size_t count,
                          uint16_t *out) {
  for (size_t i = 0; i < count; ++i) out[i] = orc_f32_to_bf16(normal_value(seed, stream, first + i));
}

void orc_fill_normal_f32(uint64_t seed, uint64_t stream, uint64_t first, size_t count, float *out) {
  for (size_t i = 0; i < count; ++i) out[i] = normal_value(seed, stream, first + i);
}
