// Bandwidth-bound kernels of the MLP step: the R-way gradient sum with the SGD update fused in,
// the bias gradient (column sums), and fp32 <-> bf16 conversion.
//
// reduce_sgd replaces the reference's ring reduce-scatter + all-gather over sockets
// (mlp_omp.cc:56-169,171-295).  There the R gradient copies sit in R NUMA domains and every chunk
// travels R-1 hops; here all R copies sit in one HBM, so each element is read once from each
// replica's arena, summed in registers in replica order, applied to W with one fused
// multiply-add (the arithmetic of mlp_omp.cc:140-143,242-250), and written once.
// Algorithmic traffic: (R + 2) * 4 bytes per parameter (+2 with the bf16 copy).
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace mi {

thread_local LaunchEvents* launch_events = nullptr;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned short f32_to_bf16_rne(float f) {
  unsigned int u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}

// UNROLL float4 per thread per trip.  Two regimes, chosen by the launcher from the bytes moved:
//   STREAM = true   the arenas exceed the 256 MB Infinity Cache: the gradients are read exactly
//                   once, so they are loaded non-temporally; one float4 per thread, one trip.
//   STREAM = false  everything fits the Infinity Cache, where the gradient GEMMs have just left
//                   their output: ordinary loads (non-temporal ones would bypass that cache), two
//                   float4 per thread in flight.
template <int R_FIXED, bool WRITE_BF16, int UNROLL, bool STREAM>
__global__ __launch_bounds__(256) void reduce_sgd_vec4(float* __restrict__ W, unsigned short* __restrict__ W16,
                                                       const float* __restrict__ G, size_t nvec,
                                                       size_t stride_vec, int R_dyn, float neg_lr_arg,
                                                       const float* __restrict__ neg_lr_dev) {
  const int R = R_FIXED > 0 ? R_FIXED : R_dyn;
  const float neg_lr = neg_lr_dev ? *neg_lr_dev : neg_lr_arg;  // uniform: one scalar load
  const f32x4* __restrict__ g4 = reinterpret_cast<const f32x4*>(G);
  f32x4* __restrict__ w4 = reinterpret_cast<f32x4*>(W);
  auto ld = [&](const f32x4* ptr) { return STREAM ? __builtin_nontemporal_load(ptr) : *ptr; };
  const size_t step = (size_t)gridDim.x * blockDim.x * UNROLL;
  for (size_t base = (size_t)blockIdx.x * blockDim.x * UNROLL + threadIdx.x; base < nvec; base += step) {
    f32x4 s[UNROLL], w[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const size_t i = base + (size_t)u * blockDim.x;
      if (i < nvec) {
        s[u] = ld(g4 + i);
        w[u] = w4[i];
      }
    }
    if (R_FIXED > 0) {
#pragma unroll
      for (int r = 1; r < R_FIXED; ++r)
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const size_t i = base + (size_t)u * blockDim.x;
          if (i < nvec) s[u] += ld(g4 + (size_t)r * stride_vec + i);
        }
    } else {
      for (int r = 1; r < R; ++r)
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const size_t i = base + (size_t)u * blockDim.x;
          if (i < nvec) s[u] += ld(g4 + (size_t)r * stride_vec + i);
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const size_t i = base + (size_t)u * blockDim.x;
      if (i >= nvec) continue;
      f32x4 o;
      o[0] = fmaf(neg_lr, s[u][0], w[u][0]);
      o[1] = fmaf(neg_lr, s[u][1], w[u][1]);
      o[2] = fmaf(neg_lr, s[u][2], w[u][2]);
      o[3] = fmaf(neg_lr, s[u][3], w[u][3]);
      w4[i] = o;
      if (WRITE_BF16) {
        u16x4 h = {f32_to_bf16_rne(o[0]), f32_to_bf16_rne(o[1]), f32_to_bf16_rne(o[2]), f32_to_bf16_rne(o[3])};
        reinterpret_cast<u16x4*>(W16)[i] = h;
      }
    }
  }
}

// scalar version for unaligned arenas and for the tail that does not fill a float4
__global__ __launch_bounds__(256) void reduce_sgd_scalar(float* __restrict__ W, unsigned short* __restrict__ W16,
                                                         const float* __restrict__ G, size_t begin, size_t n,
                                                         size_t stride, int R, float neg_lr_arg,
                                                         const float* __restrict__ neg_lr_dev) {
  const float neg_lr = neg_lr_dev ? *neg_lr_dev : neg_lr_arg;
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = begin + (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step) {
    float s = G[i];
    for (int r = 1; r < R; ++r) s += G[(size_t)r * stride + i];
    float w = fmaf(neg_lr, s, W[i]);
    W[i] = w;
    if (W16) W16[i] = f32_to_bf16_rne(w);
  }
}

static int grid_for(size_t work_items, int per_block, int max_blocks) {
  size_t b = (work_items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > (size_t)max_blocks) b = max_blocks;
  return (int)b;
}

hipError_t reduce_sgd(float* W, uint16_t* W16, const float* G, size_t n, size_t stride, int R, float lr,
                      hipStream_t s, const float* neg_lr_dev) {
  if (n == 0 || R <= 0) return hipSuccess;
  const float neg_lr = -lr;
  const bool vec = ((reinterpret_cast<uintptr_t>(W) | reinterpret_cast<uintptr_t>(G)) & 15) == 0 &&
                   (stride % 4 == 0 || R == 1) && (!W16 || (reinterpret_cast<uintptr_t>(W16) & 7) == 0);
  size_t done = 0;
  if (vec && n >= 4) {
    const size_t nvec = n / 4;
    const bool stream = (double)(R + 1) * (double)n * 4.0 > 192e6;  // beyond what the Infinity Cache holds
    // cached regime: about a thousand blocks for a launch over a whole arena (2048 float4 each;
    // measured 32.4 us against 33.3 us with 512 at config 2), 512 float4 per block below that, so
    // that a single layer's launch still covers the CUs
    const size_t per_block = stream ? 256 : (nvec >= ((size_t)1 << 21) ? 2048 : 512);
    const int blocks = grid_for(nvec, (int)per_block, stream ? (1 << 30) : 8192);
#define MI_LAUNCH_REDUCE2(RF, BF)                                                                          \
  do {                                                                                                     \
    if (stream)                                                                                            \
      launch_kernel((reduce_sgd_vec4<RF, BF, 1, true>), dim3(blocks), dim3(256), 0, s, W, W16, G, nvec, \
                         stride / 4, R, neg_lr, neg_lr_dev);                                               \
    else                                                                                                   \
      launch_kernel((reduce_sgd_vec4<RF, BF, 2, false>), dim3(blocks), dim3(256), 0, s, W, W16, G, nvec, \
                         stride / 4, R, neg_lr, neg_lr_dev);                                               \
  } while (0)
#define MI_LAUNCH_REDUCE(RF, BF) MI_LAUNCH_REDUCE2(RF, BF)
    if (W16) {
      switch (R) {
        case 1: MI_LAUNCH_REDUCE(1, true); break;
        case 2: MI_LAUNCH_REDUCE(2, true); break;
        case 4: MI_LAUNCH_REDUCE(4, true); break;
        case 8: MI_LAUNCH_REDUCE(8, true); break;
        default: MI_LAUNCH_REDUCE(0, true); break;
      }
    } else {
      switch (R) {
        case 1: MI_LAUNCH_REDUCE(1, false); break;
        case 2: MI_LAUNCH_REDUCE(2, false); break;
        case 4: MI_LAUNCH_REDUCE(4, false); break;
        case 8: MI_LAUNCH_REDUCE(8, false); break;
        default: MI_LAUNCH_REDUCE(0, false); break;
      }
    }
#undef MI_LAUNCH_REDUCE2
#undef MI_LAUNCH_REDUCE
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    done = nvec * 4;
  }
  if (done < n) {
    const int blocks = grid_for(n - done, 256, 2048);
    launch_kernel(reduce_sgd_scalar, dim3(blocks), dim3(256), 0, s, W, W16, G, done, n, stride, R, neg_lr, neg_lr_dev);
  }
  return hipGetLastError();
}

// ---- bias gradient: column sums of the K rows of each replica ----------------------------------
// One workgroup owns 64 columns of one replica; its 4 wavefronts stride over the rows (coalesced
// 256-byte row segments), then the 4 partial sums are combined through LDS in a fixed order, so
// the result does not depend on scheduling.
__global__ __launch_bounds__(256) void colsum_kernel(int M, int K, const float* __restrict__ A, int lda,
                                                     float* __restrict__ out, long long stride_out) {
  __shared__ float part[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + lane;
  const float* a = A + (size_t)blockIdx.y * K * lda;
  float s = 0.0f;
  if (col < M) {
    for (int k = wave; k < K; k += 4) s += a[(size_t)k * lda + col];
  }
  part[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && col < M) {
    out[(size_t)blockIdx.y * stride_out + col] = ((part[0][lane] + part[1][lane]) + part[2][lane]) + part[3][lane];
  }
}

hipError_t colsum_f32(int R, int M, int K, const float* A, int lda, float* out, long long stride_out,
                      hipStream_t s) {
  if (R <= 0 || M <= 0) return hipSuccess;
  launch_kernel(colsum_kernel, dim3((M + 63) / 64, R), dim3(256), 0, s, M, K, A, lda, out, stride_out);
  return hipGetLastError();
}

// ---- dtype conversion --------------------------------------------------------------------------
__global__ __launch_bounds__(256) void f32_to_bf16_kernel(unsigned short* __restrict__ dst,
                                                          const float* __restrict__ src, size_t n) {
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step) dst[i] = f32_to_bf16_rne(src[i]);
}

__global__ __launch_bounds__(256) void bf16_to_f32_kernel(float* __restrict__ dst,
                                                          const unsigned short* __restrict__ src, size_t n) {
  const size_t step = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += step)
    dst[i] = __uint_as_float((unsigned int)src[i] << 16);
}

hipError_t convert_f32_to_bf16(uint16_t* dst, const float* src, size_t n, hipStream_t s) {
  if (n == 0) return hipSuccess;
  launch_kernel(f32_to_bf16_kernel, dim3(grid_for(n, 256, 4096)), dim3(256), 0, s, dst, src, n);
  return hipGetLastError();
}

hipError_t convert_bf16_to_f32(float* dst, const uint16_t* src, size_t n, hipStream_t s) {
  if (n == 0) return hipSuccess;
  launch_kernel(bf16_to_f32_kernel, dim3(grid_for(n, 256, 4096)), dim3(256), 0, s, dst, src, n);
  return hipGetLastError();
}

}  // namespace mi
