// Measurement probes used by bench.py only (built into libforja_probes.so, not part of the
// backend library): what the matrix cores sustain from registers, with nothing else going on.
// The rate depends on the operand data: with all-zero operands the device holds its peak clock,
// with random operands the same loop is power-limited to about two thirds of it.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// 16 independent 32x32 accumulators per wave (the arrangement of the GEMM kernel), operands held
// in registers, one wave per SIMD.
__global__ __launch_bounds__(256) void mfma_f16_loop(float *out, int iterations, int random_data) {
  f32x16 acc[16];
  for (int i = 0; i < 16; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  f16x8 a[4], b[4];
  uint32_t state = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 8; ++e) {
      state = state * 1664525u + 1013904223u;
      a[i][e] = (_Float16)(random_data ? (float)((state >> 8) & 0xffffu) / 32768.0f - 1.0f : 0.0f);
      state = state * 1664525u + 1013904223u;
      b[i][e] = (_Float16)(random_data ? (float)((state >> 8) & 0xffffu) / 32768.0f - 1.0f : 0.0f);
    }
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[4 * i + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[4 * i + j], 0, 0, 0);
  }
  float sum = 0.0f;
  for (int i = 0; i < 16; ++i)
    for (int r = 0; r < 16; ++r) sum += acc[i][r];
  out[blockIdx.x * 256 + threadIdx.x] = sum;
}

}  // namespace

// TFLOP/s of v_mfma_f32_32x32x16_f16 sustained over roughly `iterations` * 16 instructions per
// wave on every compute unit; negative on a HIP error.
extern "C" __attribute__((visibility("default"))) double fh_probe_mfma_f16_tflops(int iterations,
                                                                               int random_data) {
  hipDeviceProp_t props;
  if (hipGetDeviceProperties(&props, 0) != hipSuccess) return -1.0;
  const int blocks = props.multiProcessorCount;
  float *out = nullptr;
  if (hipMalloc(&out, (size_t)blocks * 256 * sizeof(float)) != hipSuccess) return -1.0;
  hipEvent_t start, stop;
  (void)hipEventCreate(&start);
  (void)hipEventCreate(&stop);
  mfma_f16_loop<<<blocks, 256>>>(out, 1000, random_data);   // warm-up
  (void)hipEventRecord(start);
  mfma_f16_loop<<<blocks, 256>>>(out, iterations, random_data);
  (void)hipEventRecord(stop);
  double result = -1.0;
  float ms = 0.0f;
  if (hipEventSynchronize(stop) == hipSuccess && hipEventElapsedTime(&ms, start, stop) == hipSuccess &&
      ms > 0.0f)
    result = (double)blocks * 4 * iterations * 16 * 32768.0 / (ms * 1e-3) / 1e12;
  (void)hipEventDestroy(start);
  (void)hipEventDestroy(stop);
  (void)hipFree(out);
  return result;
}
