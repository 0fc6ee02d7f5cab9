// Internal launch interface between the C ABI (capi.hip) and the kernel translation units.
// Every function enqueues work on `s` and returns the launch status; none of them synchronises.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace mi {

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

// out[r*stride_out + j] = sum_{i in [r*K, (r+1)*K)} A[i*lda + j], j in [0, M)
hipError_t colsum_f32(int R, int M, int K, const float* A, int lda, float* out, long long stride_out,
                      hipStream_t s);

// W[i] = fma(-lr, sum_r G[r*stride + i], W[i]); W16 (bf16 copy of the result) may be null
hipError_t reduce_sgd(float* W, uint16_t* W16, const float* G, size_t n, size_t stride, int R, float lr,
                      hipStream_t s);

hipError_t convert_f32_to_bf16(uint16_t* dst, const float* src, size_t n, hipStream_t s);
hipError_t convert_bf16_to_f32(float* dst, const uint16_t* src, size_t n, hipStream_t s);

}  // namespace mi
