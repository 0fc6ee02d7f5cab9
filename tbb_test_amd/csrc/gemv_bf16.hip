// Skinny bf16 layers: C[M,N] = A[M,K] * B[N,K]^T (both operands bf16 and K-contiguous, fp32 sums)
// when one of the three dimensions is at most SKINNY_MAX -- the bf16 counterpart of gemv_f32.hip.
// In a bf16 model whose last layer is 1024 -> 1, as in the reference's own default model
// (mlp_bench_common.h:26), these are the three GEMMs of that layer:
//   forward          N <= SKINNY_MAX   Y = X W^T + b            (mlp_omp.cc:474-488)
//   weight gradient  M <= SKINNY_MAX   dW_r = dZ_r^T A_r from the K-contiguous copies dZ_r^T, A_r^T  (mlp_omp.cc:565-580)
//   input gradient   K <= SKINNY_MAX   dA = dZ W, masked        (mlp_omp.cc:657-671)
// On a 64 x 64 MFMA tile such a GEMM wastes all but one row or column of the matrix cores; here each
// is one pass over its large operand.  Every sum runs in a fixed order (strided partial sums per
// lane, then a fixed butterfly), so results do not depend on scheduling.  Epilogues as in the MFMA
// kernels (EpilogueH).  The transposed second output and the column-sum partials of the big kernels
// are not produced here; the caller falls back to its transpose / row-sum launches.
#include <hip/hip_runtime.h>

#include "gemm_bf16_common.h"

namespace mi {

namespace {

__device__ __forceinline__ float lo16(unsigned two) { return __uint_as_float(two << 16); }
__device__ __forceinline__ float hi16(unsigned two) { return __uint_as_float(two & 0xffff0000u); }

// acc += dot of the 8 bf16 pairs of two 16-byte pieces, in element order
__device__ __forceinline__ float dot8(const u32x4& a, const u32x4& b, float acc) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    acc = fmaf(lo16(a[e]), lo16(b[e]), acc);
    acc = fmaf(hi16(a[e]), hi16(b[e]), acc);
  }
  return acc;
}

template <int EPI>
__device__ __forceinline__ void store_one(const HGemmArgs& p, int z, int row, int col, float v) {
  if (EPI == EPH_F32) {
    (reinterpret_cast<float*>(p.C) + (size_t)z * p.batchC)[(size_t)row * p.ldc + col] = v;
    return;
  }
  if (EPI == EPH_BIAS_RELU) {
    if (p.bias) v += p.bias[col];
    if (p.relu) v = v > 0.0f ? v : 0.0f;
  } else if (EPI == EPH_MASK) {
    if (!(bf2f(p.mask[(size_t)row * p.ldmask + col]) > 0.0f)) v = 0.0f;
  }
  (reinterpret_cast<u16*>(p.C) + (size_t)z * p.batchC)[(size_t)row * p.ldc + col] = f2bf(v);
}

// ---- one wavefront per row of the long operand -------------------------------------------------------
// LONG_IS_A = true  (N <= SKINNY_MAX): the wavefront owns row m of A and forms its products with the N rows of B;
// LONG_IS_A = false (M <= SKINNY_MAX): it owns row n of B and forms the products with the M rows of A.
// The lane walks the row in 16-byte pieces (lane, lane + 64, ...); the short operand's rows stay in
// the caches.  VEC = false: element by element, for operands that allow no 16-byte loads.
template <int EPI, bool LONG_IS_A, bool VEC>
__global__ __launch_bounds__(256) void gemv_bf16_rows_kernel(HGemmArgs p) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6), z = blockIdx.y;
  const int long_rows = LONG_IS_A ? p.M : p.N, short_rows = LONG_IS_A ? p.N : p.M;
  if (row >= long_rows) return;
  const u16* lng = (LONG_IS_A ? p.A + (size_t)z * p.batchA + (size_t)row * p.lda : p.B + (size_t)z * p.batchB + (size_t)row * p.ldb);
  const u16* sht = LONG_IS_A ? p.B + (size_t)z * p.batchB : p.A + (size_t)z * p.batchA;
  const int ld_short = LONG_IS_A ? p.ldb : p.lda;
  float acc[SKINNY_MAX];
#pragma unroll
  for (int j = 0; j < SKINNY_MAX; ++j) acc[j] = 0.0f;
  int k_done = 0;
  if (VEC) {
    const int k8 = p.K >> 3;
    for (int c = lane; c < k8; c += 64) {
      const u32x4 lv = *reinterpret_cast<const u32x4*>(lng + c * 8);
#pragma unroll
      for (int j = 0; j < SKINNY_MAX; ++j) {
        if (j >= short_rows) break;
        acc[j] = dot8(lv, *reinterpret_cast<const u32x4*>(sht + (size_t)j * ld_short + c * 8), acc[j]);
      }
    }
    k_done = k8 << 3;
  }
  for (int k = k_done + lane; k < p.K; k += 64) {
    const float lv = bf2f(lng[k]);
#pragma unroll
    for (int j = 0; j < SKINNY_MAX; ++j) {
      if (j >= short_rows) break;
      acc[j] = fmaf(lv, bf2f(sht[(size_t)j * ld_short + k]), acc[j]);
    }
  }
#pragma unroll
  for (int j = 0; j < SKINNY_MAX; ++j) {
    if (j >= short_rows) break;
    float v = acc[j];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    if (lane == 0) {
      if (LONG_IS_A) store_one<EPI>(p, z, row, j, v);
      else store_one<EPI>(p, z, j, row, v);
    }
  }
}

// ---- K <= SKINNY_MAX: an outer-product-like pass over the output --------------------------------------
// One thread per output element; the K terms of both operands are a few bytes per row (the rows of
// B, N x K elements in all, stay in the caches).  Consecutive threads write consecutive columns.
template <int EPI>
__global__ __launch_bounds__(256) void gemv_bf16_shortk_kernel(HGemmArgs p) {
  const int z = blockIdx.y;
  const u16* A = p.A + (size_t)z * p.batchA;
  const u16* B = p.B + (size_t)z * p.batchB;
  const size_t total = (size_t)p.M * p.N;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    const int row = (int)(i / p.N), col = (int)(i % p.N);
    const u16* a = A + (size_t)row * p.lda;
    const u16* b = B + (size_t)col * p.ldb;
    float v = 0.0f;
    for (int k = 0; k < p.K; ++k) v = fmaf(bf2f(a[k]), bf2f(b[k]), v);
    store_one<EPI>(p, z, row, col, v);
  }
}

// The same with 8 consecutive columns of one row per thread: 16-byte accesses to C (two for fp32
// results) and to the mask.  The sums run over k in the same order as in the kernel above, so both
// give the same bits.  For N a multiple of 8 and 16-byte aligned rows of C and of the mask.
template <int EPI>
__global__ __launch_bounds__(256) void gemv_bf16_shortk_vec_kernel(HGemmArgs p) {
  const int z = blockIdx.y;
  const u16* A = p.A + (size_t)z * p.batchA;
  const u16* B = p.B + (size_t)z * p.batchB;
  const unsigned groups = (unsigned)p.N >> 3, total = (unsigned)p.M * groups;  // the launcher checks that this fits 32 bits
  for (unsigned i = blockIdx.x * 256u + threadIdx.x; i < total; i += gridDim.x * 256u) {
    const unsigned row = i / groups, col = (i - row * groups) * 8u;
    const u16* a = A + (size_t)row * p.lda;
    float v[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) v[c] = 0.0f;
    for (int k = 0; k < p.K; ++k) {
      const float av = bf2f(a[k]);
#pragma unroll
      for (int c = 0; c < 8; ++c) v[c] = fmaf(av, bf2f(B[(size_t)(col + c) * p.ldb + k]), v[c]);
    }
    if (EPI == EPH_F32) {
      float* out = reinterpret_cast<float*>(p.C) + (size_t)z * p.batchC + (size_t)row * p.ldc + col;
      typedef float f32x4 __attribute__((ext_vector_type(4)));
      *reinterpret_cast<f32x4*>(out) = f32x4{v[0], v[1], v[2], v[3]};
      *reinterpret_cast<f32x4*>(out + 4) = f32x4{v[4], v[5], v[6], v[7]};
      continue;
    }
    if (EPI == EPH_BIAS_RELU) {
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        if (p.bias) v[c] += p.bias[col + c];
        if (p.relu) v[c] = v[c] > 0.0f ? v[c] : 0.0f;
      }
    } else if (EPI == EPH_MASK) {
      const u32x4 m = *reinterpret_cast<const u32x4*>(p.mask + (size_t)row * p.ldmask + col);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (!(lo16(m[e]) > 0.0f)) v[2 * e] = 0.0f;
        if (!(hi16(m[e]) > 0.0f)) v[2 * e + 1] = 0.0f;
      }
    }
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (unsigned)f2bf(v[2 * e]) | ((unsigned)f2bf(v[2 * e + 1]) << 16);
    *reinterpret_cast<u32x4*>(reinterpret_cast<u16*>(p.C) + (size_t)z * p.batchC + (size_t)row * p.ldc + col) = o;
  }
}

template <int EPI>
hipError_t launch_skinny_epi(HGemmArgs& p, int batch, hipStream_t s) {
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec = al16(p.A) && al16(p.B) && p.lda % 8 == 0 && p.ldb % 8 == 0 && p.batchA % 8 == 0 && p.batchB % 8 == 0;
  if (p.K <= SKINNY_MAX) {
    const int per16 = EPI == EPH_F32 ? 4 : 8;  // elements of C in 16 bytes
    const bool wide = p.N % 8 == 0 && al16(p.C) && p.ldc % per16 == 0 && p.batchC % per16 == 0 &&
                      (EPI != EPH_MASK || (al16(p.mask) && p.ldmask % 8 == 0)) &&
                      (size_t)p.M * (size_t)(p.N / 8) <= 0xffffffffu - 16384u * 256u;
    size_t blocks = ((size_t)p.M * (wide ? p.N / 8 : p.N) + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (wide) launch_kernel(gemv_bf16_shortk_vec_kernel<EPI>, dim3((unsigned)blocks, batch), dim3(256), 0, s, p);
    else launch_kernel(gemv_bf16_shortk_kernel<EPI>, dim3((unsigned)blocks, batch), dim3(256), 0, s, p);
  } else if (p.N <= SKINNY_MAX) {
    const dim3 grid((p.M + 3) / 4, batch);
    if (vec) launch_kernel((gemv_bf16_rows_kernel<EPI, true, true>), grid, dim3(256), 0, s, p);
    else launch_kernel((gemv_bf16_rows_kernel<EPI, true, false>), grid, dim3(256), 0, s, p);
  } else {
    const dim3 grid((p.N + 3) / 4, batch);
    if (vec) launch_kernel((gemv_bf16_rows_kernel<EPI, false, true>), grid, dim3(256), 0, s, p);
    else launch_kernel((gemv_bf16_rows_kernel<EPI, false, false>), grid, dim3(256), 0, s, p);
  }
  return hipGetLastError();
}

}  // namespace

bool hgemm_is_skinny(int M, int N, int K) {
  return M > 0 && N > 0 && K > 0 && (M <= SKINNY_MAX || N <= SKINNY_MAX || K <= SKINNY_MAX);
}

hipError_t launch_skinny(HGemmArgs& p, int batch, int epi, hipStream_t s) {
  if (batch <= 0 || batch > 65535) return batch <= 0 ? hipSuccess : hipErrorInvalidValue;
  switch (epi) {
    case EPH_F32: return launch_skinny_epi<EPH_F32>(p, batch, s);
    case EPH_BIAS_RELU: return launch_skinny_epi<EPH_BIAS_RELU>(p, batch, s);
    case EPH_MASK: return launch_skinny_epi<EPH_MASK>(p, batch, s);
    default: return launch_skinny_epi<EPH_BF16>(p, batch, s);
  }
}

}  // namespace mi
