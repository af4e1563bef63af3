// A probe, not a GEMM: the rate at which this chip sustains the matrix instruction the kernels are
// built on (v_mfma_f32_32x32x16_bf16), with all operands and accumulators held in registers and
// no memory traffic at all.  On operands whose bits vary like real activations the chip lowers
// its clock to stay inside its power limit; on all-zero operands it does not.  The first figure
// is therefore the ceiling of any bf16 GEMM on this device and data, whatever its memory system
// does; the benchmark prints both next to the GEMM's own rate.
//
// A helper of bench.py only (built as libbench_mfma_probe.so next to it, loaded through ctypes):
// no part of libgrouped_gemm_hip.so or of its header.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

using bf16x8 = __attribute__((ext_vector_type(8))) __bf16;
using f32x16 = __attribute__((ext_vector_type(16))) float;

constexpr int kProbeWaves = 4, kProbeBlocks = 4;   // 4 x 4 blocks of 32 x 32 per wave: 256 accumulator registers

// Eight bf16 values distributed like randn * 0.02 (the sum of four uniform numbers stands in for
// the normal distribution), from a per-lane integer hash: signs, exponents and mantissas then
// toggle from value to value as they do in activations and weights.
__device__ __forceinline__ bf16x8 probe_operand(uint32_t seed, bool zeros) {
  bf16x8 v;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    seed = seed * 1664525u + 1013904223u;
    const uint32_t h = seed ^ (seed >> 15);
    const float sum = (float)(h & 255u) + (float)((h >> 8) & 255u) + (float)((h >> 16) & 255u) + (float)(h >> 24);
    const float normal = (sum - 510.0f) * (1.7320508f / 255.0f);   // mean 0, variance 1
    v[i] = zeros ? (__bf16)0.0f : (__bf16)(0.02f * normal);
  }
  return v;
}

__global__ __launch_bounds__(kProbeWaves * 64) void mfma_probe_kernel(int iterations, int zeros, float* sink) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t id = blockIdx.x * blockDim.x + threadIdx.x;
  bf16x8 a[kProbeBlocks], b[kProbeBlocks];
#pragma unroll
  for (int i = 0; i < kProbeBlocks; ++i) {
    a[i] = probe_operand(id * 8u + i, zeros != 0);
    b[i] = probe_operand(id * 8u + 4u + i, zeros != 0);
  }
  f32x16 acc[kProbeBlocks][kProbeBlocks];
#pragma unroll
  for (int i = 0; i < kProbeBlocks; ++i)
#pragma unroll
    for (int j = 0; j < kProbeBlocks; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int j = 0; j < kProbeBlocks; ++j)
#pragma unroll
      for (int i = 0; i < kProbeBlocks; ++i) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
    // new operand values every step, as a depth loop would bring them (the elements of two
    // fragments rotate: register moves only)
    a[0] = __builtin_shufflevector(a[0], a[0], 1, 2, 3, 4, 5, 6, 7, 0);
    b[1] = __builtin_shufflevector(b[1], b[1], 1, 2, 3, 4, 5, 6, 7, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < kProbeBlocks; ++i)
#pragma unroll
    for (int j = 0; j < kProbeBlocks; ++j) s += acc[i][j][0];
  if (s == 12345.678f) sink[0] = s;   // never true for these operands; keeps the loop alive
#endif
}

// Launches the probe `launches` + 1 times on `stream` (the first untimed) with one workgroup per
// compute unit and returns the rate of the timed ones in TFLOP/s through `tflops`.
hipError_t run_mfma_probe(int cus, int zeros, int launches, float* sink, hipStream_t stream, float* tflops) {
  constexpr int kIterations = 8192;
  hipEvent_t e0, e1;
  hipError_t err = hipEventCreate(&e0);
  if (err != hipSuccess) return err;
  err = hipEventCreate(&e1);
  if (err != hipSuccess) {
    (void)hipEventDestroy(e0);
    return err;
  }
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(cus), dim3(kProbeWaves * 64), 0, stream, kIterations, zeros, sink);
  err = hipEventRecord(e0, stream);
  for (int i = 0; i < launches && err == hipSuccess; ++i) {
    hipLaunchKernelGGL(mfma_probe_kernel, dim3(cus), dim3(kProbeWaves * 64), 0, stream, kIterations, zeros, sink);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipEventRecord(e1, stream);
  if (err == hipSuccess) err = hipEventSynchronize(e1);
  float ms = 0.0f;
  if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (err != hipSuccess) return err;
  const double flop = (double)launches * cus * kProbeWaves * (double)kIterations * kProbeBlocks * kProbeBlocks * (2.0 * 32 * 32 * 16);
  *tflops = (float)(flop / ((double)ms * 1e-3) / 1e12);
  return hipSuccess;
}

}  // namespace

// TFLOP/s of `launches` probe launches of about 2 ms each on the current device's null stream
// (waits for them); zero_operands != 0: all-zero operands.  Returns a hipError_t as int.
extern "C" int bench_mfma_rate(int zero_operands, int launches, float* tflops) {
  if (tflops == nullptr || launches < 1 || launches > 1000) return (int)hipErrorInvalidValue;
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return (int)err;
  hipDeviceProp_t prop;
  err = hipGetDeviceProperties(&prop, dev);
  if (err != hipSuccess) return (int)err;
  float* sink = nullptr;
  err = hipMalloc(&sink, 256);
  if (err != hipSuccess) return (int)err;
  err = run_mfma_probe(prop.multiProcessorCount, zero_operands != 0, launches, sink, nullptr, tflops);
  (void)hipFree(sink);
  return (int)err;
}
