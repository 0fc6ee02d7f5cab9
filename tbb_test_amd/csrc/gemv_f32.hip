// Skinny fp32 layers: the three GEMMs of the MLP step when the layer's output width is at most
// SKINNY_MAX, as in the reference's own default model, whose last layer is 1024 -> 1
// (mlp_bench_common.h:26).  On an MFMA tile such a layer wastes all but one column of the matrix
// cores; as matrix-vector work each GEMM is a single pass over its large operand at memory speed:
//   forward          Y[m][n]  = sum_k X[m][k] W[n][k] + b[n]       N <= SKINNY_MAX  (mlp_omp.cc:474-488)
//   weight gradient  dW_r[m][n] = sum_k dZ_r[k][m] A_r[k][n]       M <= SKINNY_MAX  (mlp_omp.cc:565-580)
//   input gradient   dA[m][n] = sum_k dZ[m][k] W[k][n] (masked)    K <= SKINNY_MAX  (mlp_omp.cc:657-671)
// All sums run in a fixed order (strided partial sums per lane, then a fixed tree), so results do
// not depend on scheduling.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mi {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// ---- forward: one wavefront per row of X -----------------------------------------------------------
// The lane walks its row in float4 pieces (lane, lane + 64, ...) and multiplies each piece with the
// same piece of every row of W (N rows of K floats: they stay in the L1/L2).  VEC = false: element
// by element, for operands whose alignment allows no 16-byte loads.
template <bool VEC>
__global__ __launch_bounds__(256) void gemv_nt_kernel(int M, int N, int K, const float* __restrict__ X, int ldx,
                                                      const float* __restrict__ W, int ldw, float* __restrict__ Y,
                                                      int ldy, const float* __restrict__ bias, int relu) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= M) return;
  const float* x = X + (size_t)row * ldx;
  float acc[SKINNY_MAX];
#pragma unroll
  for (int n = 0; n < SKINNY_MAX; ++n) acc[n] = 0.0f;
  if (VEC) {
    const int k4 = K >> 2;
    for (int c = lane; c < k4; c += 64) {
      const f32x4 xv = *reinterpret_cast<const f32x4*>(x + c * 4);
#pragma unroll
      for (int n = 0; n < SKINNY_MAX; ++n) {
        if (n >= N) break;
        const f32x4 wv = *reinterpret_cast<const f32x4*>(W + (size_t)n * ldw + c * 4);
        acc[n] = fmaf(xv[3], wv[3], fmaf(xv[2], wv[2], fmaf(xv[1], wv[1], fmaf(xv[0], wv[0], acc[n]))));
      }
    }
    for (int k = (k4 << 2) + lane; k < K; k += 64) {
#pragma unroll
      for (int n = 0; n < SKINNY_MAX; ++n) {
        if (n >= N) break;
        acc[n] = fmaf(x[k], W[(size_t)n * ldw + k], acc[n]);
      }
    }
  } else {
    for (int k = lane; k < K; k += 64) {
#pragma unroll
      for (int n = 0; n < SKINNY_MAX; ++n) {
        if (n >= N) break;
        acc[n] = fmaf(x[k], W[(size_t)n * ldw + k], acc[n]);
      }
    }
  }
#pragma unroll
  for (int n = 0; n < SKINNY_MAX; ++n) {
    if (n >= N) break;
    float v = acc[n];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if (lane == 0) {
      if (bias) v += bias[n];
      if (relu) v = v > 0.0f ? v : 0.0f;
      Y[(size_t)row * ldy + n] = v;
    }
  }
}

// ---- weight gradient: a workgroup owns 16 columns of A for one replica ---------------------------
// Thread = (k slot 0..31, column 0..15): a wavefront reads 4 rows x 64 bytes per load, the eight
// wavefronts of the workgroup 32 consecutive rows, and the workgroup strides over the replica's K
// rows, eight loads in flight per thread.  The 32 partial sums of a column are added in slot order.
// The workgroups of column group 0 also produce the column sums of dZ (the bias gradient).
constexpr int TN_SLOTS = 32;
__global__ __launch_bounds__(TN_SLOTS * 16) void gemv_tn_kernel(int M, int N, int K, const float* __restrict__ dZ,
                                                                int lddz, const float* __restrict__ A, int lda,
                                                                float* __restrict__ dW, int lddw, long long strideW,
                                                                float* __restrict__ colsum, long long stride_colsum) {
  __shared__ float part[TN_SLOTS][SKINNY_MAX + 1][16];  // [k slot][m, or the column-sum row][column]
  const int tid = threadIdx.x, col = tid & 15, slot = tid >> 4;
  const int n = blockIdx.x * 16 + col, r = blockIdx.y;
  const float* dz = dZ + (size_t)r * K * lddz;
  const float* a = A + (size_t)r * K * lda + (n < N ? n : 0);
  const bool do_colsum = colsum != nullptr && blockIdx.x == 0;
  float acc[SKINNY_MAX], cs = 0.0f;
#pragma unroll
  for (int m = 0; m < SKINNY_MAX; ++m) acc[m] = 0.0f;
  constexpr int UNROLL = 8;
  int k = slot;
  for (; k + (UNROLL - 1) * TN_SLOTS < K; k += UNROLL * TN_SLOTS) {
    float av[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) av[u] = a[(size_t)(k + u * TN_SLOTS) * lda];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const float* g = dz + (size_t)(k + u * TN_SLOTS) * lddz;
#pragma unroll
      for (int m = 0; m < SKINNY_MAX; ++m) {
        if (m >= M) break;
        acc[m] = fmaf(g[m], av[u], acc[m]);
      }
      if (do_colsum && col < M) cs += g[col];  // thread `col` of every slot sums column `col` of dZ
    }
  }
  for (; k < K; k += TN_SLOTS) {
    const float av = a[(size_t)k * lda];
    const float* g = dz + (size_t)k * lddz;
#pragma unroll
    for (int m = 0; m < SKINNY_MAX; ++m) {
      if (m >= M) break;
      acc[m] = fmaf(g[m], av, acc[m]);
    }
    if (do_colsum && col < M) cs += g[col];
  }
#pragma unroll
  for (int m = 0; m < SKINNY_MAX; ++m)
    if (m < M) part[slot][m][col] = acc[m];
  part[slot][SKINNY_MAX][col] = cs;
  __syncthreads();
  // thread (m = slot, column) folds the partial sums of its (m, column) in slot order
  if (slot < M && n < N) {
    float v = part[0][slot][col];
#pragma unroll
    for (int sl = 1; sl < TN_SLOTS; ++sl) v += part[sl][slot][col];
    dW[(size_t)r * strideW + (size_t)slot * lddw + n] = v;
  }
  if (do_colsum && slot == SKINNY_MAX && col < M) {
    float v = part[0][SKINNY_MAX][col];
#pragma unroll
    for (int sl = 1; sl < TN_SLOTS; ++sl) v += part[sl][SKINNY_MAX][col];
    colsum[(size_t)r * stride_colsum + col] = v;
  }
}

// ---- input gradient: an outer-product-like pass over the output ----------------------------------
// Thread per float4 of dA (VEC) or per element: K <= SKINNY_MAX terms per element, the mask read at
// the output position.
template <bool VEC>
__global__ __launch_bounds__(256) void gemv_nn_kernel(int M, int N, int K, const float* __restrict__ dZ, int lddz,
                                                      const float* __restrict__ W, int ldw, float* __restrict__ dA,
                                                      int ldda, const float* __restrict__ mask, int ldmask) {
  if (VEC) {
    const int n4 = N >> 2;
    const size_t total = (size_t)M * n4;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
      const int row = (int)(i / n4), c = (int)(i % n4) * 4;
      f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
      for (int k = 0; k < K; ++k) {
        const float g = dZ[(size_t)row * lddz + k];
        const f32x4 wv = *reinterpret_cast<const f32x4*>(W + (size_t)k * ldw + c);
        v[0] = fmaf(g, wv[0], v[0]);
        v[1] = fmaf(g, wv[1], v[1]);
        v[2] = fmaf(g, wv[2], v[2]);
        v[3] = fmaf(g, wv[3], v[3]);
      }
      if (mask) {
        const f32x4 mk = *reinterpret_cast<const f32x4*>(mask + (size_t)row * ldmask + c);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (!(mk[e] > 0.0f)) v[e] = 0.0f;
      }
      *reinterpret_cast<f32x4*>(dA + (size_t)row * ldda + c) = v;
    }
  } else {
    const size_t total = (size_t)M * N;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
      const int row = (int)(i / N), c = (int)(i % N);
      float v = 0.0f;
      for (int k = 0; k < K; ++k) v = fmaf(dZ[(size_t)row * lddz + k], W[(size_t)k * ldw + c], v);
      if (mask && !(mask[(size_t)row * ldmask + c] > 0.0f)) v = 0.0f;
      dA[(size_t)row * ldda + c] = v;
    }
  }
}

static inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

hipError_t sgemv_nt(int M, int N, int K, const float* X, int ldx, const float* W, int ldw, float* Y, int ldy,
                    const float* bias, int relu, hipStream_t s) {
  if (M <= 0 || N <= 0) return hipSuccess;
  const bool vec = al16(X) && al16(W) && ldx % 4 == 0 && ldw % 4 == 0;
  const dim3 grid((M + 3) / 4);
  if (vec) launch_kernel(gemv_nt_kernel<true>, grid, dim3(256), 0, s, M, N, K, X, ldx, W, ldw, Y, ldy, bias, relu);
  else launch_kernel(gemv_nt_kernel<false>, grid, dim3(256), 0, s, M, N, K, X, ldx, W, ldw, Y, ldy, bias, relu);
  return hipGetLastError();
}

hipError_t sgemv_tn(int R, int M, int N, int K, const float* dZ, int lddz, const float* A, int lda, float* dW,
                    int lddw, long long strideW, float* colsum, long long stride_colsum, hipStream_t s) {
  if (R <= 0 || M <= 0 || N <= 0) return hipSuccess;
  launch_kernel(gemv_tn_kernel, dim3((N + 15) / 16, R), dim3(TN_SLOTS * 16), 0, s, M, N, K, dZ, lddz, A, lda, dW, lddw, strideW,
                colsum, stride_colsum);
  return hipGetLastError();
}

hipError_t sgemv_nn(int M, int N, int K, const float* dZ, int lddz, const float* W, int ldw, float* dA, int ldda,
                    const float* mask, int ldmask, hipStream_t s) {
  if (M <= 0 || N <= 0) return hipSuccess;
  const bool vec = N % 4 == 0 && al16(W) && al16(dA) && ldw % 4 == 0 && ldda % 4 == 0 &&
                   (!mask || (al16(mask) && ldmask % 4 == 0));
  const size_t items = vec ? (size_t)M * (N / 4) : (size_t)M * N;
  size_t blocks = (items + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  if (vec) launch_kernel(gemv_nn_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s, M, N, K, dZ, lddz, W, ldw, dA, ldda, mask, ldmask);
  else launch_kernel(gemv_nn_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, M, N, K, dZ, lddz, W, ldw, dA, ldda, mask, ldmask);
  return hipGetLastError();
}

}  // namespace mi
