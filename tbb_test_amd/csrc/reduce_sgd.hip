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
//                   once, so they are loaded non-temporally; four float4 per thread in flight, one
//                   trip (R = 8, 3.36 GB: 5.70 TB/s with one, 5.98 with two, 6.09 with four, 3.98
//                   with eight; R = 2, 1.07 GB: 6.64 / 6.67 / 6.73 / 5.76).
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
        // The bf16 copy is read next by a GEMM of a later step: stored non-temporally it does not push
        // W out of the Infinity Cache (8192 x 8192, R = 4, one matrix updated over and over: 225 us
        // without the copy, 300 us with it as ordinary stores, 241 us non-temporal; on cold data, eight
        // such matrices taken in turn, 268 us without the copy and 289 us with it).
        if (STREAM) __builtin_nontemporal_store(h, reinterpret_cast<u16x4*>(W16) + i);
        else reinterpret_cast<u16x4*>(W16)[i] = h;
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
    const size_t per_block = stream ? 1024 : (nvec >= ((size_t)1 << 21) ? 2048 : 512);
    const int blocks = grid_for(nvec, (int)per_block, stream ? (1 << 30) : 8192);
#define MI_LAUNCH_REDUCE2(RF, BF)                                                                          \
  do {                                                                                                     \
    if (stream)                                                                                            \
      launch_kernel((reduce_sgd_vec4<RF, BF, 4, true>), dim3(blocks), dim3(256), 0, s, W, W16, G, nvec, \
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

// ---- reduce + SGD of one layer of a bf16 model, writing both bf16 operand copies ------------------
// The bf16 GEMMs read W (forward) and W^T (input gradient) as K-contiguous bf16 matrices.  The
// reference forwards the updated chunk to its consumers in the same pass that applies the SGD
// update (mlp_omp.cc:240-252); here that pass writes, from registers, the fp32 master weights, the
// bf16 copy, and -- through an LDS tile -- the transposed bf16 copy, so that no separate transpose
// launch re-reads what the update just produced.  A workgroup takes the TR x TC tiles blockIdx.x,
// blockIdx.x + gridDim.x, ... of W (one each when the grid covers them all); a pass of
// the 256 threads covers 1024 / (TC/4) whole tile rows (TC = 256: four rows of 1 KB each, the
// contiguous runs the memory likes), the arithmetic per element is that of reduce_sgd_vec4.  The
// transposed copy leaves as runs of 128 bytes (64 rows of one column).  The tiles of one extra
// tile row (tile_y == rows / TR) stand for the `tail` floats that follow the matrix in the
// arena (the layer's bias and padding), updated the flat way, so that a layer is one launch.
// GROUP = passes whose loads are in flight together.
// STREAM (the layer exceeds the caches): the two bf16 copies are stored non-temporally and the tiles
// are walked in bands of 16 tile rows, column by column inside a band, so that the workgroups
// running at the same time write runs of 2 KB of the transposed copy where row-major order gives
// 128-byte pieces 16 KB apart.  8192 x 8192, R = 4, on cold data (eight such layers taken in turn,
// as a step does): 365 us = 5.15 TB/s with 64 x 64 tiles, ordinary stores and row-major order,
// 333 us = 5.64 TB/s = 0.705 of the HBM peak with 64 x 128 tiles, non-temporal stores and bands;
// the flat fp32 update of the same matrices (no bf16 copies) reaches 0.75 on the same data.
// Algorithmic traffic per weight: (R + 2) * 4 + 2 + 2 bytes.
template <int R_FIXED, bool STREAM, int TR, int TC, int GROUP>
__global__ __launch_bounds__(256) void reduce_sgd_tile(float* __restrict__ W, unsigned short* __restrict__ W16,
                                                       unsigned short* __restrict__ W16T,
                                                       const float* __restrict__ G, int rows, int cols,
                                                       size_t stride, size_t tail, int R_dyn, float neg_lr_arg,
                                                       const float* __restrict__ neg_lr_dev, int tiles_x,
                                                       int total_tiles) {
  constexpr int NT = 256;  // threads of a workgroup
  // bf16 pairs; an odd number of words per row keeps the column gather below free of bank conflicts
  __shared__ unsigned int tile[TR][TC / 2 + 1];
  const int R = R_FIXED > 0 ? R_FIXED : R_dyn;
  const float neg_lr = neg_lr_dev ? *neg_lr_dev : neg_lr_arg;
  const int tid = threadIdx.x;
  auto ld = [&](const float* ptr) {
    const f32x4* q = reinterpret_cast<const f32x4*>(ptr);
    return STREAM ? __builtin_nontemporal_load(q) : *q;
  };
  auto update4 = [&](f32x4 sum, f32x4 w) {
    f32x4 o;
    o[0] = fmaf(neg_lr, sum[0], w[0]);
    o[1] = fmaf(neg_lr, sum[1], w[1]);
    o[2] = fmaf(neg_lr, sum[2], w[2]);
    o[3] = fmaf(neg_lr, sum[3], w[3]);
    return o;
  };
  const int tiles_y = rows / TR, matrix_tiles = tiles_x * tiles_y;
  for (int t = blockIdx.x; t < total_tiles; t += gridDim.x) {
    int tile_x = t % tiles_x, tile_y = t / tiles_x;
    if (STREAM && t < matrix_tiles) {  // bands of BAND tile rows, walked column by column
      constexpr int BAND = 16;
      const int per_band = BAND * tiles_x, band = t / per_band, within = t - band * per_band;
      const int band_rows = tiles_y - band * BAND < BAND ? tiles_y - band * BAND : BAND;
      tile_x = within / band_rows;
      tile_y = band * BAND + within - tile_x * band_rows;
    }
    if (tile_y * TR >= rows) {  // the floats behind the matrix: bias and padding
      const size_t base = (size_t)rows * cols, nvec = tail / 4;
      for (size_t i = (size_t)tile_x * NT + tid; i < nvec; i += (size_t)tiles_x * NT) {
        const size_t off = base + i * 4;
        f32x4 sum = ld(G + off);
        for (int r = 1; r < R; ++r) sum += ld(G + (size_t)r * stride + off);
        const f32x4 o = update4(sum, *reinterpret_cast<const f32x4*>(W + off));
        *reinterpret_cast<f32x4*>(W + off) = o;
        const u16x4 h = {f32_to_bf16_rne(o[0]), f32_to_bf16_rne(o[1]), f32_to_bf16_rne(o[2]), f32_to_bf16_rne(o[3])};
        *reinterpret_cast<u16x4*>(W16 + off) = h;
      }
      continue;
    }
    const int r0 = tile_y * TR, c0 = tile_x * TC;
    constexpr int VPR = TC / 4;            // float4 per tile row
    constexpr int PASSES = TR * VPR / NT;  // NT float4 per pass; GROUP = passes whose loads are in flight together
    static_assert(PASSES % GROUP == 0, "tile shape");
#pragma unroll 1
    for (int g = 0; g < PASSES / GROUP; ++g) {
      size_t off[GROUP];
      f32x4 sum[GROUP], w[GROUP];
#pragma unroll
      for (int i = 0; i < GROUP; ++i) {
        const int idx = tid + NT * (g * GROUP + i), row = idx / VPR, c4 = idx % VPR;
        off[i] = (size_t)(r0 + row) * cols + c0 + c4 * 4;
        sum[i] = ld(G + off[i]);
        w[i] = *reinterpret_cast<const f32x4*>(W + off[i]);
      }
      if (R_FIXED > 0) {
#pragma unroll
        for (int r = 1; r < R_FIXED; ++r)
#pragma unroll
          for (int i = 0; i < GROUP; ++i) sum[i] += ld(G + (size_t)r * stride + off[i]);
      } else {
        for (int r = 1; r < R; ++r)
#pragma unroll
          for (int i = 0; i < GROUP; ++i) sum[i] += ld(G + (size_t)r * stride + off[i]);
      }
#pragma unroll
      for (int i = 0; i < GROUP; ++i) {
        const int idx = tid + NT * (g * GROUP + i), row = idx / VPR, c4 = idx % VPR;
        const f32x4 o = update4(sum[i], w[i]);
        const u16x4 h = {f32_to_bf16_rne(o[0]), f32_to_bf16_rne(o[1]), f32_to_bf16_rne(o[2]), f32_to_bf16_rne(o[3])};
        *reinterpret_cast<f32x4*>(W + off[i]) = o;
        if (STREAM) __builtin_nontemporal_store(h, reinterpret_cast<u16x4*>(W16 + off[i]));
        else *reinterpret_cast<u16x4*>(W16 + off[i]) = h;
        tile[row][c4 * 2] = (unsigned)h[0] | ((unsigned)h[1] << 16);
        tile[row][c4 * 2 + 1] = (unsigned)h[2] | ((unsigned)h[3] << 16);
      }
    }
    __syncthreads();
    // transposed copy: output row c0 + c holds the tile's TR rows = 2 TR contiguous bytes, 16 per thread
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    constexpr int CP = TR / 8;  // 16-byte chunks per output row
#pragma unroll
    for (int i = 0; i < TC * CP / NT; ++i) {
      const int q = tid + NT * i, c = q / CP, part = q % CP;
      unsigned e[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) e[k] = (tile[part * 8 + k][c >> 1] >> ((c & 1) * 16)) & 0xffffu;
      const u32x4 v = {e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
      u32x4* dst = reinterpret_cast<u32x4*>(W16T + (size_t)(c0 + c) * rows + r0 + part * 8);
      if (STREAM) __builtin_nontemporal_store(v, dst);
      else *dst = v;
    }
    __syncthreads();  // the tile is read out before the next one is written
  }
}

bool reduce_sgd_tiled_fits(const float* W, const uint16_t* W16, const uint16_t* W16T, const float* G, int rows,
                           int cols, size_t stride, size_t tail, int R) {
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  return rows > 0 && cols > 0 && rows % 64 == 0 && cols % 64 == 0 && al16(W) && al16(G) && al16(W16T) &&
         (reinterpret_cast<uintptr_t>(W16) & 7) == 0 && (stride % 4 == 0 || R == 1) && tail % 4 == 0 &&
         (long long)(rows / 64 + 1) * (cols / 64) < (1ll << 31);
}

hipError_t reduce_sgd_tiled(float* W, uint16_t* W16, uint16_t* W16T, const float* G, int rows, int cols, size_t stride,
                            size_t tail, int R, float lr, hipStream_t s, const float* neg_lr_dev, bool beside_gemm) {
  if (!reduce_sgd_tiled_fits(W, W16, W16T, G, rows, cols, stride, tail, R) || R <= 0) return hipErrorInvalidValue;
  const float neg_lr = -lr;
  const bool stream = (double)(R + 1) * (double)rows * (double)cols * 4.0 > 192e6;  // beyond the Infinity Cache
  // 64 x 64 tiles in the cached regime.  Streaming regime, cold 8192 x 8192 layers with R = 4 (the
  // kernel body in a stand-alone loop over four such layers): 64 x 128 tiles in bands 330 us,
  // 256 x 128 row-major 333 us, 128 x 128 row-major 339 us, 128 x 128 in bands 354 us, 64 x 64 in
  // bands 361 us, 256 x 64 row-major 376 us, 64 x 64 row-major 380 us, 64 x 64 column-major 467 us;
  // without the transposed copy 306 us.
  // streaming regime: 64 x 128 tiles where the width allows
  const bool wide = stream && cols % 128 == 0;
  const int tiles_x = cols / (wide ? 128 : 64), total_tiles = tiles_x * (rows / 64 + (tail ? 1 : 0));
  // A launch that runs beside a GEMM on another stream (the per-layer update of a bf16 model under
  // the input-gradient GEMM of the next layer) is one workgroup per CU walking the tiles, with half
  // the loads in flight (65 instead of 120 registers at R = 4): that leaves the registers and the
  // LDS a 256 x 256 GEMM workgroup needs on the same CU, where thousands of short workgroups take
  // whole CUs in turns with the GEMM.  Alone such a grid is as fast as the full one (2.90 against
  // 2.86 ms for eight 8192 x 8192 layers, R = 4); beside the GEMMs the step of that model takes
  // 40.2-40.3 ms instead of 40.8-40.9.  Twice or half as many workgroups, or workgroups of 64 or
  // 128 threads that stay longer, lose the gain or more: a GEMM runs slower for as long as an
  // update runs on its CUs, so the update has to be short.
  int grid_x = total_tiles;
  if (beside_gemm && stream) {
    int dev = 0, cus = 0;
    if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
    if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev); e != hipSuccess) return e;
    if (cus > 0 && cus < grid_x) grid_x = cus;
  }
  const bool lean = grid_x < total_tiles;
  const dim3 grid(grid_x);
#define MI_LAUNCH_TILE3(RF, ST, TR, TC, GR)                                                                          \
  launch_kernel((reduce_sgd_tile<RF, ST, TR, TC, GR>), grid, dim3(256), 0, s, W, W16, W16T, G, rows, cols, stride, tail, \
                R, neg_lr, neg_lr_dev, tiles_x, total_tiles)
#define MI_LAUNCH_TILE(RF)                     \
  do {                                         \
    if (lean && wide) MI_LAUNCH_TILE3(RF, true, 64, 128, 2);    \
    else if (lean) MI_LAUNCH_TILE3(RF, true, 64, 64, 2);        \
    else if (wide) MI_LAUNCH_TILE3(RF, true, 64, 128, 4);       \
    else if (stream) MI_LAUNCH_TILE3(RF, true, 64, 64, 4);      \
    else MI_LAUNCH_TILE3(RF, false, 64, 64, 4);                 \
  } while (0)
  switch (R) {
    case 1: MI_LAUNCH_TILE(1); break;
    case 2: MI_LAUNCH_TILE(2); break;
    case 4: MI_LAUNCH_TILE(4); break;
    case 8: MI_LAUNCH_TILE(8); break;
    default: MI_LAUNCH_TILE(0); break;
  }
#undef MI_LAUNCH_TILE
#undef MI_LAUNCH_TILE3
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

// ---- device copy -------------------------------------------------------------------------------
// The weight snapshot / restore of a benchmark loop.  The runtime's own device-to-device copy runs
// at about 1.2 TB/s (read + write) on this GPU; a plain grid of 16-byte loads and stores moves the
// same bytes four times as fast.
__global__ __launch_bounds__(256) void copy_kernel(f32x4* __restrict__ dst, const f32x4* __restrict__ src, size_t nvec) {
  const size_t step = (size_t)gridDim.x * 256 * 4;
  for (size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x; base < nvec; base += step) {
    f32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (base + u * 256 < nvec) v[u] = __builtin_nontemporal_load(src + base + u * 256);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (base + u * 256 < nvec) dst[base + u * 256] = v[u];
  }
}

hipError_t device_copy(void* dst, const void* src, size_t bytes, hipStream_t s) {
  if (bytes == 0) return hipSuccess;
  if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | bytes) & 15) != 0)
    return hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, s);
  const size_t nvec = bytes / 16;
  launch_kernel(copy_kernel, dim3(grid_for(nvec, 1024, 1 << 20)), dim3(256), 0, s, reinterpret_cast<f32x4*>(dst),
                reinterpret_cast<const f32x4*>(src), nvec);
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
