// Measurement aid: what do the MFMA pipes of this device sustain with nothing else going on?
// A register-resident loop of independent MFMAs (four accumulator blocks per wavefront, up to four
// wavefronts per SIMD), no memory traffic.  For bf16 the rate depends on the operand values (the
// matrix cores are power-limited there, and constant operands toggle fewer wires than random
// mantissas) and on the instruction: v_mfma_f32_16x16x32_bf16, which the large bf16 GEMM uses,
// sustains 2 060 TFLOP/s on random operands, v_mfma_f32_32x32x16_bf16 1 800 (operands = 3), both
// 2 460-2 480 on zeros; for fp32 the rate does not depend on the values (155 TFLOP/s).  The
// GEMM kernels are priced against the published peak; this number says how much of the distance
// to that peak is the device's and how much the kernels'.  No counterpart in the reference.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mi {

typedef float pf32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 pbf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ unsigned probe_hash(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// operands: 0 zeros, 1 ones, 2 (and 3) pseudo-random in [-1, 1), distinct per lane and register
__device__ __forceinline__ float probe_value(int operands, unsigned h) {
  return operands == 0 ? 0.0f : operands == 1 ? 1.0f : (float)(h & 0xffff) / 32768.0f - 1.0f;
}
typedef float pf32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void mfma_rate_f32(float* out, int iters, int operands) {
  pf32x16 acc[4];
  for (int i = 0; i < 4; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  float a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    const unsigned h = probe_hash(threadIdx.x * 16 + i + blockIdx.x * 7919);
    a[i] = probe_value(operands, h);
    b[i] = probe_value(operands, h >> 16);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[(u + i) & 7], acc[i], 0, 0, 0);
  }
  float s = 0.0f;
  for (int i = 0; i < 4; ++i)
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// 64 independent 16 x 16 blocks per wavefront (a 128 x 128 wavefront tile in GEMM block order: the A
// operand changes every eighth instruction, the B operand every instruction): 64 MFMAs of 16384
// flop per iteration.  (With 16 blocks per wavefront the same loop reaches only three quarters of
// this rate.)
__global__ __launch_bounds__(256) void mfma_rate_bf16_x32(float* out, int iters, int operands) {
  pf32x4 acc[8][8];
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 8; ++j)
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
  pbf16x8 a[8], b[8];
  for (int i = 0; i < 8; ++i)
    for (int e = 0; e < 8; ++e) {
      const unsigned h = probe_hash(threadIdx.x * 64 + i * 8 + e + blockIdx.x * 7919);
      a[i][e] = (__bf16)probe_value(operands, h);
      b[i][e] = (__bf16)probe_value(operands, h >> 16);
    }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
  }
  float s = 0.0f;
  for (int i = 0; i < 8; ++i)
    for (int j = 0; j < 8; ++j)
      for (int r = 0; r < 4; ++r) s += acc[i][j][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void mfma_rate_bf16(float* out, int iters, int operands) {
  pf32x16 acc[4];
  for (int i = 0; i < 4; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  pbf16x8 a[4], b[4];
  for (int i = 0; i < 4; ++i)
    for (int e = 0; e < 8; ++e) {
      const unsigned h = probe_hash(threadIdx.x * 64 + i * 8 + e + blockIdx.x * 7919);
      a[i][e] = (__bf16)probe_value(operands, h);
      b[i][e] = (__bf16)probe_value(operands, h >> 16);
    }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u], b[(u + i) & 3], acc[i], 0, 0, 0);
  }
  float s = 0.0f;
  for (int i = 0; i < 4; ++i)
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// Runs the loop on `s` in batches of three launches for about 0.4 s and returns the average rate
// of the second half in TFLOP/s (the first tens of milliseconds after an idle period run at
// reduced clocks).  The grid is exactly what is resident at once, four workgroups per CU or fewer
// if the register count allows fewer: a grid that needs a second, partly filled round would
// measure that tail, not the MFMA pipes.
hipError_t probe_mfma_rate(bool bf16, int operands, double* tflops, hipStream_t s) {
  constexpr int kThreads = 256, kLaunches = 3;
  const bool x32 = bf16 && operands != 3;    // the instruction of the large bf16 GEMM; operands = 3: 32x32x16 on random values
  const int iters = bf16 ? (x32 ? 4000 : 8000) : 4000;
  const int mfma_per_iter = bf16 ? (x32 ? 64 : 16) : 32;  // per wavefront
  const double flop_per_mfma = bf16 ? (x32 ? 2.0 * 16 * 16 * 32 : 2.0 * 32 * 32 * 16) : 2.0 * 32 * 32 * 2;
  int dev = 0, cus = 0, per_cu = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e == hipSuccess)
    e = x32    ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, mfma_rate_bf16_x32, kThreads, 0)
        : bf16 ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, mfma_rate_bf16, kThreads, 0)
               : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, mfma_rate_f32, kThreads, 0);
  if (e != hipSuccess) return e;
  if (per_cu > 4) per_cu = 4;
  if (per_cu < 1 || cus < 1) return hipErrorInvalidValue;
  const int blocks = cus * per_cu;
  const double flop_per_batch = (double)blocks * (kThreads / 64) * iters * mfma_per_iter * kLaunches * flop_per_mfma;
  float* out = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  e = hipMalloc((void**)&out, (size_t)blocks * kThreads * sizeof(float));
  if (e != hipSuccess) return e;
  double total_ms = 0.0, late_ms = 0.0;
  int late_batches = 0;
  do {
    if ((e = hipEventCreate(&e0)) != hipSuccess) break;
    if ((e = hipEventCreate(&e1)) != hipSuccess) break;
    for (int batch = 0; batch < 400 && total_ms < 400.0 && e == hipSuccess; ++batch) {
      if ((e = hipEventRecord(e0, s)) != hipSuccess) break;
      for (int w = 0; w < kLaunches; ++w) {
        if (x32) hipLaunchKernelGGL(mfma_rate_bf16_x32, dim3(blocks), dim3(kThreads), 0, s, out, iters, operands);
        else if (bf16) hipLaunchKernelGGL(mfma_rate_bf16, dim3(blocks), dim3(kThreads), 0, s, out, iters, operands);
        else hipLaunchKernelGGL(mfma_rate_f32, dim3(blocks), dim3(kThreads), 0, s, out, iters, operands);
      }
      if ((e = hipEventRecord(e1, s)) != hipSuccess) break;
      if ((e = hipEventSynchronize(e1)) != hipSuccess) break;
      if ((e = hipGetLastError()) != hipSuccess) break;
      float ms = 0.0f;
      if ((e = hipEventElapsedTime(&ms, e0, e1)) != hipSuccess) break;
      total_ms += ms;
      if (total_ms > 200.0) {
        late_ms += ms;
        ++late_batches;
      }
    }
  } while (false);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(out);
  if (e != hipSuccess) return e;
  if (late_batches == 0 || late_ms <= 0.0) return hipErrorUnknown;
  *tflops = flop_per_batch * late_batches / (late_ms * 1e-3) / 1e12;
  return hipSuccess;
}

}  // namespace mi
