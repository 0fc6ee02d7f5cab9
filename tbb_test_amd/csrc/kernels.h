// Internal launch interface between the C ABI (capi.hip) and the kernel translation units.
// Every function enqueues work on `s` and returns the launch status; none of them synchronises.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <mutex>

namespace mi {

// Per-launch timing.  While `launch_events` is set (by the timing scope of the C ABI, on the
// calling thread), kernels are launched through hipExtLaunchKernelGGL with a start and a stop
// event attached to the dispatch itself: the pair then measures the kernel's own execution, as a
// profiler's kernel trace does, and not the gap to the previous kernel that a hipEventRecord
// before the launch would add.  The first launch of a scope takes the start event, every launch
// re-records the stop event, so a scope of several kernels is timed from the first kernel's
// start to the last kernel's end.
struct LaunchEvents {
  hipEvent_t start, stop;
  int launches;
};
extern thread_local LaunchEvents* launch_events;

template <typename... KArgs, typename... Args>
inline void launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t s,
                          Args... args) {
  LaunchEvents* ev = launch_events;
  if (ev) {
    hipEvent_t start = ev->launches == 0 ? ev->start : nullptr;
    ev->launches++;
    hipExtLaunchKernelGGL(kernel, grid, block, (std::uint32_t)lds_bytes, s, start, ev->stop, 0, static_cast<KArgs>(args)...);
  } else {
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, s, static_cast<KArgs>(args)...);
  }
}

// Opt-in to more than 64 KiB of dynamic LDS for one kernel, remembered per device (the attribute
// belongs to the kernel's code object on a device) and safe to reach from several host threads.
// One object per kernel (a function-local static of the launcher template).  The attribute call
// is made at most once per device and size, and never during a stream capture as long as the first
// launch of each kernel happens outside one.
struct LdsOptIn {
  static constexpr int kMaxDevices = 64;
  std::atomic<size_t> granted[kMaxDevices];
  std::mutex mutex;
  LdsOptIn() {
    for (auto& g : granted) g.store(0, std::memory_order_relaxed);
  }
  hipError_t ensure(const void* kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return hipSuccess;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    if (granted[dev].load(std::memory_order_acquire) >= bytes) return hipSuccess;
    std::lock_guard<std::mutex> lock(mutex);
    if (granted[dev].load(std::memory_order_relaxed) >= bytes) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return e;
    granted[dev].store(bytes, std::memory_order_release);
    return hipSuccess;
  }
};

// `variant` selects a tile configuration of the MFMA kernel (0 = choose from the shape); it is
// exposed through mi_set_gemm_variant for tuning runs.
hipError_t sgemm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                    int ldc, const float* bias, int relu, hipStream_t s, int variant);
hipError_t sgemm_nn(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                    int ldc, const float* mask, int ldmask, hipStream_t s, int variant);
// colsum (may be null): colsum[r*stride_colsum + m] = sum over replica r's K rows of A[.][m]
hipError_t sgemm_tn(int R, int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                    float* C, int ldc, long long strideC, float* colsum, long long stride_colsum,
                    hipStream_t s, int variant);

// Both backward GEMMs of one dense fp32 layer in one launch, for problems so small that a step is
// bound by the number of launches (the shapes the automatic choice gives to the split-K kernel):
//   dW_r[nout x nin] = dZ_r^T A_r, db_r = colsum dZ_r (r < R, rows / R rows each), dA[rows x nin] = dZ W (masked)
// with dense operands dZ [rows x nout], A [rows x nin], W [nout x nin], mask [rows x nin] or null.
// Same arithmetic, bit for bit, as sgemm_tn + sgemm_nn on those shapes.
bool sgemm_backward_pair_fits(int R, int rows, int nout, int nin);
hipError_t sgemm_backward_pair(int R, int rows, int nout, int nin, const float* dZ, const float* A, const float* W,
                               float* dW, long long strideW, float* db, long long stride_db, float* dA,
                               const float* mask, hipStream_t s);

// gemv_f32.hip: the same three operations for layers whose output width is at most SKINNY_MAX
// (N of the forward GEMM, M of the weight gradient, K of the input gradient), as matrix-vector
// passes at memory speed.  Any alignment; the automatic choice of sgemm_* takes them.
constexpr int SKINNY_MAX = 16;
hipError_t sgemv_nt(int M, int N, int K, const float* X, int ldx, const float* W, int ldw, float* Y, int ldy,
                    const float* bias, int relu, hipStream_t s);
hipError_t sgemv_tn(int R, int M, int N, int K, const float* dZ, int lddz, const float* A, int lda, float* dW,
                    int lddw, long long strideW, float* colsum, long long stride_colsum, hipStream_t s);
hipError_t sgemv_nn(int M, int N, int K, const float* dZ, int lddz, const float* W, int ldw, float* dA, int ldda,
                    const float* mask, int ldmask, hipStream_t s);

// out[r*stride_out + j] = sum_{i in [r*K, (r+1)*K)} A[i*lda + j], j in [0, M)
hipError_t colsum_f32(int R, int M, int K, const float* A, int lda, float* out, long long stride_out,
                      hipStream_t s);

// W[i] = fma(-lr, sum_r G[r*stride + i], W[i]); W16 (bf16 copy of the result) may be null.
// neg_lr_dev (may be null): device address of -lr; when given, the kernel reads the factor from
// there instead of taking `lr` -- a captured graph then follows a changing learning rate.
hipError_t reduce_sgd(float* W, uint16_t* W16, const float* G, size_t n, size_t stride, int R, float lr,
                      hipStream_t s, const float* neg_lr_dev = nullptr);

// Same update for one weight matrix W [rows x cols] (dense) of a bf16 model, writing the bf16 copy
// W16 [rows x cols] and the transposed bf16 copy W16T [cols x rows] in the same pass; the `tail`
// floats that follow the matrix in W, W16 and every replica of G (a layer's bias and padding) are
// updated the flat way by the same launch.  Needs rows and cols multiples of 64, tail a multiple
// of 4 and 16-byte aligned pointers (reduce_sgd_tiled_fits); `stride` = floats between consecutive
// replicas' gradients.  beside_gemm: the launch will run next to a GEMM on another stream (one
// workgroup per CU walks the tiles, see the launcher).
bool reduce_sgd_tiled_fits(const float* W, const uint16_t* W16, const uint16_t* W16T, const float* G, int rows,
                           int cols, size_t stride, size_t tail, int R);
hipError_t reduce_sgd_tiled(float* W, uint16_t* W16, uint16_t* W16T, const float* G, int rows, int cols, size_t stride,
                            size_t tail, int R, float lr, hipStream_t s, const float* neg_lr_dev = nullptr,
                            bool beside_gemm = false);

// bf16: C = A[M,K] * B[N,K]^T with fp32 accumulation, both operands K-contiguous, blockIdx.z
// batches with element strides batchA/B/C.  out_kind: 0 fp32 plain, 1 bf16 with bias + optional
// ReLU, 2 bf16 zeroed where mask (bf16) <= 0, 3 bf16 plain.  Ct (bf16 output kinds, batch 1): the
// result is also written transposed per group of ct_rows rows, Ct[row / ct_rows][col][row % ct_rows];
// *wrote_ct tells whether the kernel that was chosen could do that (else the caller transposes).
// colsum_part (bf16 output kinds, batch 1): the kernel also writes column sums of its output per block
// of 128 rows, colsum_part[row / 128][col] (N floats per block); *wrote_colsum tells whether the
// chosen kernel did.  colsum_fold adds a replica's blocks up: the bias gradient of the layer whose
// dZ the GEMM produced.
hipError_t hgemm_nt(int batch, int M, int N, int K, const uint16_t* A, int lda, long long batchA, const uint16_t* B,
                    int ldb, long long batchB, void* C, int ldc, long long batchC, int out_kind, const float* bias,
                    int relu, const uint16_t* mask, int ldmask, hipStream_t s, int variant, uint16_t* Ct = nullptr,
                    int ct_rows = 0, bool* wrote_ct = nullptr, float* colsum_part = nullptr, bool* wrote_colsum = nullptr);
hipError_t colsum_fold(int R, int N, int blocks_per_replica, const float* part, float* out, long long stride_out,
                       hipStream_t s);
// dst[z][c][r] = src[z][r][c] for 16-bit elements
// mfma_probe.hip: TFLOP/s of a register-resident MFMA loop (operands: 0 zeros, 1 ones, 2 random)
hipError_t probe_mfma_rate(bool bf16, int operands, double* tflops, hipStream_t s);

hipError_t transpose_bf16(int batch, int rows, int cols, const uint16_t* src, int ld_src, long long batch_src,
                          uint16_t* dst, int ld_dst, long long batch_dst, hipStream_t s);
// out[z*stride_out + r] = sum_c src[z][r][c] in fp32
hipError_t rowsum_bf16(int batch, int rows, int cols, const uint16_t* src, int ld, long long batch_src, float* out,
                       long long stride_out, hipStream_t s);

// dst[0..bytes) = src[0..bytes) on the device (16-byte aligned: own kernel; else the runtime's copy)
hipError_t device_copy(void* dst, const void* src, size_t bytes, hipStream_t s);

hipError_t convert_f32_to_bf16(uint16_t* dst, const float* src, size_t n, hipStream_t s);
hipError_t convert_bf16_to_f32(float* dst, const uint16_t* src, size_t n, hipStream_t s);

}  // namespace mi
