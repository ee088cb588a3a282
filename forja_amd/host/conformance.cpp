// Known-answer checks of the HIP backend through the C++ host interface.  Every case restates a
// test the reference keeps for its own backends (cited per case) with the same inputs and the
// same closed-form expectations; nothing here depends on another implementation.
// Exit code 0 = all passed.  Needs a gfx950 device.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "forja_hip.hpp"

using namespace forja_hip;

namespace {

int failures = 0;

void check(bool condition, const char *what) {
  if (!condition) {
    std::fprintf(stderr, "FAILED: %s\n", what);
    ++failures;
  }
}

uint16_t f32_to_bf16(float value) {
  uint32_t bits;
  std::memcpy(&bits, &value, 4);
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return (uint16_t)(bits >> 16);
}

// IEEE binary16 of values that are exactly representable (all that the cases below use).
uint16_t f32_to_f16_exact(float value) {
  uint32_t bits;
  std::memcpy(&bits, &value, 4);
  if ((bits & 0x7fffffffu) == 0) return (uint16_t)(bits >> 16);
  uint32_t sign = (bits >> 16) & 0x8000u;
  int32_t exponent = (int32_t)((bits >> 23) & 0xffu) - 127 + 15;
  return (uint16_t)(sign | ((uint32_t)exponent << 10) | ((bits >> 13) & 0x3ffu));
}

template <class T>
Tensor upload(HipBackend &backend, DType dtype, const std::vector<uint32_t> &shape, const std::vector<T> &values) {
  Result<Tensor> tensor = backend.alloc(dtype, shape);
  check(tensor.ok(), "alloc");
  check(backend.write(tensor.value, values.data(), values.size() * sizeof(T)).ok(), "write");
  return tensor.value;
}

std::vector<float> read_f32(HipBackend &backend, const Tensor &tensor) {
  Result<std::vector<uint8_t>> bytes = backend.read(tensor);
  check(bytes.ok(), "read");
  std::vector<float> out(bytes.value.size() / 4);
  std::memcpy(out.data(), bytes.value.data(), out.size() * 4);
  return out;
}

BackendError run(HipBackend &backend, const CommandList &commands) {
  Result<Submission> submission = backend.submit(commands);
  if (!submission.ok()) return submission.error;
  return submission.value.wait().error;
}

// quant_matmul_dequantizes_q4_and_q8_in_mlx_order, crates/forja-cpu/src/lib.rs:2786-2845 (q4, bf16
// parameters): rows of words 0, 0x11111111 and 0xffffffff give sum(x)*bias, sum(x)*(scale+bias),
// sum(x)*(15*scale+bias).
void quant_matmul_known_answers(HipBackend &backend) {
  for (uint32_t rows : {1u, 7u, 33u}) {
    const uint32_t inner = 64;
    std::vector<float> x(rows * inner);
    for (uint32_t i = 0; i < rows * inner; ++i) x[i] = (float)(i % 17) / 8.0f - 1.0f;
    std::vector<uint32_t> words;
    for (uint32_t pattern : {0u, 0x11111111u, 0xffffffffu})
      for (uint32_t w = 0; w < inner / 8; ++w) words.push_back(pattern);
    const float scale[3] = {0.5f, -0.25f, 0.125f}, bias[3] = {1.0f, 2.0f, -1.0f};
    std::vector<uint16_t> scales, biases;
    for (int n = 0; n < 3; ++n) {
      scales.push_back(f32_to_bf16(scale[n]));
      biases.push_back(f32_to_bf16(bias[n]));
    }
    Tensor xt = upload(backend, DType::F32, {rows, inner}, x);
    Tensor packed = upload(backend, DType::U32, {3, inner / 8}, words);
    Tensor st = upload(backend, DType::BF16, {3, 1}, scales);
    Tensor bt = upload(backend, DType::BF16, {3, 1}, biases);
    Tensor out = backend.alloc(DType::F32, {rows, 3}).value;
    CommandList commands;
    commands.dispatch(Op::quant_matmul(4, 64), {xt, packed, st, bt}, {out});
    check(run(backend, commands).ok(), "quant matmul runs");
    std::vector<float> y = read_f32(backend, out);
    for (uint32_t r = 0; r < rows; ++r) {
      float sum = 0.0f;
      for (uint32_t i = 0; i < inner; ++i) sum += x[r * inner + i];
      const float expected[3] = {sum * bias[0], sum * (scale[1] + bias[1]), sum * (scale[2] * 15.0f + bias[2])};
      for (int n = 0; n < 3; ++n)
        check(std::fabs(y[r * 3 + n] - expected[n]) <= 1e-5f + 1e-5f * std::fabs(expected[n]),
              "quant matmul closed form");
    }
    for (const Tensor &t : {xt, packed, st, bt, out}) backend.release(t);
  }
}

// argmax_prefers_the_last_equal_value, crates/forja-cpu/src/lib.rs:2386-2395.
void argmax_prefers_last(HipBackend &backend) {
  Tensor x = upload<float>(backend, DType::F32, {1, 5}, {1.0f, 9.0f, 2.0f, 9.0f, 3.0f});
  Tensor out = backend.alloc(DType::U32, {1}).value;
  CommandList commands;
  commands.dispatch(Op::argmax(), {x}, {out});
  check(run(backend, commands).ok(), "argmax runs");
  Result<std::vector<uint8_t>> bytes = backend.read(out);
  uint32_t index = 0;
  std::memcpy(&index, bytes.value.data(), 4);
  check(index == 3, "argmax picks the last of equal maxima");
}

// top_k normalisation, crates/forja-cpu/src/lib.rs:2398-2447: values [0,2,0,1] with k=2 select
// indices [1,3] and weights [1/(1+e^-1), e^-1/(1+e^-1)].
void top_k_normalises(HipBackend &backend) {
  Tensor x = upload<float>(backend, DType::F32, {1, 4}, {0.0f, 2.0f, 0.0f, 1.0f});
  Tensor values = backend.alloc(DType::F32, {1, 2}).value;
  Tensor indices = backend.alloc(DType::U32, {1, 2}).value;
  CommandList commands;
  commands.dispatch(Op::top_k(2, true), {x}, {values, indices});
  check(run(backend, commands).ok(), "top-k runs");
  std::vector<float> v = read_f32(backend, values);
  Result<std::vector<uint8_t>> bytes = backend.read(indices);
  uint32_t idx[2];
  std::memcpy(idx, bytes.value.data(), 8);
  const float e = std::exp(-1.0f);
  check(idx[0] == 1 && idx[1] == 3, "top-k indices");
  check(std::fabs(v[0] - 1.0f / (1.0f + e)) < 1e-6f && std::fabs(v[1] - e / (1.0f + e)) < 1e-6f,
        "top-k normalised weights");
}

// sample_refuses_invalid_live_parameters, crates/forja-cpu/src/lib.rs:2664-2686 (a NaN temperature
// read when the dispatch runs is InvalidInput), the greedy rule of sample_allowed (:1605-1614:
// temperature 0 takes the largest value, the largest index among equals), and
// top_k_and_top_p_keep_only_the_exact_allowed_set (:2536-2547): with top_k 3 over
// [10,9,8,1,0,-1,-2] every draw is one of the first three.
void sampling_known_answers(HipBackend &backend) {
  Tensor logits = upload<float>(backend, DType::F32, {7}, {10.0f, 9.0f, 8.0f, 1.0f, 0.0f, -1.0f, -2.0f});
  Tensor out = backend.alloc(DType::U32, {1}).value;
  auto bits = [](float value) {
    uint32_t word;
    std::memcpy(&word, &value, 4);
    return word;
  };
  auto draw = [&](const std::vector<uint32_t> &words, uint32_t position, uint32_t *index) {
    Tensor params = upload<uint32_t>(backend, DType::U32, {5}, words);
    CommandList commands;
    commands.dispatch(Op::sample(position), {logits, params}, {out});
    BackendError error = run(backend, commands);
    Result<std::vector<uint8_t>> bytes = backend.read(out);
    std::memcpy(index, bytes.value.data(), 4);
    return error;
  };
  uint32_t index = 99;
  check(draw({bits(NAN), 0, bits(1.0f), 0, 0}, 0, &index).code == FH_INVALID_INPUT,
        "NaN temperature is refused when the dispatch runs");
  check(draw({bits(0.0f), 0, bits(1.0f), 0, 0}, 0, &index).ok() && index == 0, "greedy sample");
  Tensor ties = upload<float>(backend, DType::F32, {5}, {1.0f, 9.0f, 2.0f, 9.0f, 3.0f});
  Tensor params = upload<uint32_t>(backend, DType::U32, {5}, {bits(0.0f), 0, bits(1.0f), 0, 0});
  CommandList commands;
  commands.dispatch(Op::sample(0), {ties, params}, {out});
  check(run(backend, commands).ok(), "greedy sample over ties runs");
  std::memcpy(&index, backend.read(out).value.data(), 4);
  check(index == 3, "greedy sample picks the last of equal maxima");
  bool inside = true;
  for (uint32_t position = 0; position < 64; ++position) {
    check(draw({bits(1.0f), 3, bits(1.0f), 11, 0}, position, &index).ok(), "top-k sample runs");
    inside = inside && index <= 2;
  }
  check(inside, "top_k 3 keeps the draws inside the three largest");
}

// paged_append_stores_both_planes_before_attention, crates/forja-cpu/src/lib.rs:1926-1970: all-ones
// V gives output exactly 1.0; the first 2048 bytes of the f16 value pool are f16(1.0), the rest 0.
void paged_append_stores_both_planes(HipBackend &backend) {
  Tensor query = backend.alloc(DType::F32, {16, 1, 128}).value;
  Tensor key = backend.alloc(DType::F32, {1, 8, 128}).value;
  Tensor value = upload(backend, DType::F32, {1, 8, 128}, std::vector<float>(8 * 128, 1.0f));
  Tensor table = upload<uint32_t>(backend, DType::U32, {1, 2}, {0u, 1u});
  Tensor generations = upload<uint32_t>(backend, DType::U32, {1}, {1u});
  Tensor key_pages = backend.alloc(DType::F16, {1, 16, 8, 128}).value;
  Tensor value_pages = backend.alloc(DType::F16, {1, 16, 8, 128}).value;
  Tensor output = backend.alloc(DType::F32, {16, 1, 128}).value;
  CommandList commands;
  commands.dispatch(Op::paged_sdpa_append(0.125f, 0, 16), {query, key, value, table, generations},
                    {output, key_pages, value_pages});
  check(run(backend, commands).ok(), "paged append runs");
  bool ones = true;
  for (float v : read_f32(backend, output)) ones = ones && v == 1.0f;
  check(ones, "attention over a single all-ones value row is exactly one");
  Result<std::vector<uint8_t>> raw = backend.read(value_pages);
  const uint16_t one = f32_to_f16_exact(1.0f);
  bool stored = true, untouched = true;
  for (size_t i = 0; i < 1024; ++i) {
    uint16_t half;
    std::memcpy(&half, raw.value.data() + 2 * i, 2);
    stored = stored && half == one;
  }
  for (size_t i = 2048; i < raw.value.size(); ++i) untouched = untouched && raw.value[i] == 0;
  check(stored, "value plane row stored as f16 ones");
  check(untouched, "rest of the value plane untouched");
}

// paged_attention_matches_a_hand_checked_case, crates/forja-cpu/src/paged.rs:457-476: two keys
// (1,0) and (0,1) in physical page 1, query (1,0), scale 1: probabilities e/(e+1), 1/(e+1).
void paged_attention_hand_checked(HipBackend &backend) {
  std::vector<float> pool(2 * 4 * 1 * 2, 0.0f);
  pool[(1 * 4 + 0) * 2 + 0] = 1.0f;
  pool[(1 * 4 + 1) * 2 + 1] = 1.0f;
  Tensor keys = upload(backend, DType::F32, {2, 4, 1, 2}, pool);
  Tensor values = upload(backend, DType::F32, {2, 4, 1, 2}, pool);
  Tensor table = upload<uint32_t>(backend, DType::U32, {2, 2}, {1u, 4u, 0u, 3u});
  Tensor generations = upload<uint32_t>(backend, DType::U32, {2}, {3u, 4u});
  Tensor query = upload<float>(backend, DType::F32, {1, 1, 2}, {1.0f, 0.0f});
  Tensor out = backend.alloc(DType::F32, {1, 1, 2}).value;
  CommandList commands;
  commands.dispatch(Op::paged_sdpa(1.0f, false, 0, 2, 4), {query, keys, values, table, generations}, {out});
  check(run(backend, commands).ok(), "paged sdpa runs");
  std::vector<float> y = read_f32(backend, out);
  const float expected = std::exp(1.0f) / (std::exp(1.0f) + 1.0f);
  check(std::fabs(y[0] - expected) < 1e-6f && std::fabs(y[1] - (1.0f - expected)) < 1e-6f,
        "two-key softmax closed form");
  // a stale generation must be reported, never dereferenced (crates/forja-core/src/paged.rs:381-420)
  Tensor stale = upload<uint32_t>(backend, DType::U32, {2}, {3u, 5u});
  CommandList bad;
  bad.dispatch(Op::paged_sdpa(1.0f, false, 0, 2, 4), {query, keys, values, table, stale}, {out});
  check(!run(backend, bad).ok(), "stale page generation is an error");
}

// Backend::write refuses non-contiguous views and wrong lengths with InvalidInput
// (crates/forja-cpu/src/lib.rs:113-134); released tensors are no longer valid.
void write_and_release_contract(HipBackend &backend) {
  Tensor t = backend.alloc(DType::F32, {4, 4}).value;
  std::vector<float> zeros = read_f32(backend, t);
  bool all_zero = true;
  for (float v : zeros) all_zero = all_zero && v == 0.0f;
  check(all_zero, "alloc is zero-initialised");
  std::vector<float> data(16, 2.0f);
  check(backend.write(t, data.data(), 60).error.code == FH_INVALID_INPUT, "short write refused");
  Tensor strided = t.slice({{0, 2, 2}, {0, 4, 1}});
  check(backend.write(strided, data.data(), 32).error.code == FH_INVALID_INPUT, "strided write refused");
  check(backend.write(t, data.data(), 64).ok(), "exact write accepted");
  std::vector<float> view = read_f32(backend, t.permute({1, 0}).narrow(0, 1, 2));
  check(view.size() == 8 && view[0] == 2.0f, "read gathers a permuted view");
  check(backend.release(t).ok(), "release");
  check(!backend.read(t).ok(), "released tensor is rejected");
}

// Backend::submit_profiled_retained / Submission::profile (crates/forja-core/src/backend.rs:455-579)
// and Backend::set_memory_limit (:683-686).
void profile_and_quota_contract(HipBackend &backend) {
  Tensor a = backend.alloc(DType::F32, {64, 64}).value, b = backend.alloc(DType::F32, {64, 64}).value;
  CommandList commands;
  commands.dispatch(Op::copy(), {a}, {b});
  commands.dispatch(Op::copy(), {b}, {a});
  Result<Submission> submitted = backend.submit_profiled(commands);
  check(submitted.ok() && submitted.value.wait().ok(), "profiled submission runs");
  std::vector<fh_dispatch_timing> timeline = submitted.value.profile();
  check(timeline.size() == 2 && timeline[0].dispatch == 0 && timeline[1].dispatch == 1 &&
            timeline[0].start_ns <= timeline[0].end_ns && timeline[0].end_ns <= timeline[1].start_ns,
        "one ordered timeline entry per dispatch");
  const uint64_t held = backend.memory_usage().value;
  check(backend.set_memory_limit(held).ok(), "set_memory_limit");
  check(backend.alloc(DType::F32, {1u << 20, 64}).error.code == FH_QUOTA_EXCEEDED, "allocation beyond the limit refused");
  check(backend.set_memory_limit(0).ok() && backend.alloc(DType::F32, {1024}).ok(), "limit lifted");
}

}  // namespace

int main() {
  Result<HipBackend *> created = HipBackend::create(0);
  if (!created.ok()) {
    std::fprintf(stderr, "no gfx950 device: fh_create returned %d\n", (int)created.error.code);
    return 2;
  }
  HipBackend &backend = *created.value;
  quant_matmul_known_answers(backend);
  argmax_prefers_last(backend);
  top_k_normalises(backend);
  sampling_known_answers(backend);
  paged_append_stores_both_planes(backend);
  paged_attention_hand_checked(backend);
  write_and_release_contract(backend);
  profile_and_quota_contract(backend);
  delete created.value;
  if (failures == 0) std::printf("conformance: all checks passed\n");
  return failures == 0 ? 0 : 1;
}
