// fp32 GEMM kernels for gfx950 on v_mfma_f32_32x32x2_f32, templates over the three operand
// layouts of the MLP step:
//   NT  C = A[M,K] * B[N,K]^T   forward        (reference call site mlp_omp.cc:474-488)
//   NN  C = A[M,K] * B[K,N]     input gradient (mlp_omp.cc:657-671)
//   TN  C = A[K,M]^T * B[K,N]   weight gradient, batched over replicas (mlp_omp.cc:565-580)
//
// Structure of one workgroup (WM x WN wavefronts of 64 lanes):
//   - owns a BM x BN tile of C; walks K in steps of BK;
//   - operand tiles travel global -> LDS either directly (gemm_f32_dma: global_load_lds into a
//     ring of LDS buffers; the kernel of all large GEMMs) or through registers (gemm_f32_mfma:
//     small tilings, and the guarded instances for ragged or unaligned shapes);
//   - each wavefront owns a (BM/WM) x (BN/WN) sub-tile as TM x TN blocks of 32 x 32 held in
//     accumulator registers.
//
// Operand fragments.  One MFMA consumes, per lane, one A value A[i = lane%32][k = lane/32] and
// one B value B[k = lane/32][j = lane%32].  A lane fetches four values with one 16-byte LDS
// read, and what the four values are depends on how the operand lies in memory:
//   * "K-major" operand (k contiguous: A of NT/NN, B of NT): the tile is stored [row][k] (with
//     a 4-float pad per row in gemm_f32_mfma, XOR-swizzled chunks in gemm_f32_dma); the lane reads k = kk*8 + 4*(lane/32) + {0,1,2,3} of its row and
//     feeds them to four consecutive MFMAs of the same 32 x 32 block.
//   * "M-major" operand (rows contiguous: A of TN, B of NN/TN): the tile is stored [k][row];
//     the lane reads rows TM*(lane%32) + {0..TM-1} of one k and feeds them to the TM blocks of
//     one MFMA step, i.e. block b of the wavefront owns the interleaved rows TM*i + b.
// Both choices walk k in the same order (MFMA step q of chunk kk multiplies k = kk*8 + q on
// lanes 0-31 and kk*8 + 4 + q on lanes 32-63), so any pairing of the two is consistent.
//
// Result layout of a 32 x 32 block: lane holds column (lane%32), rows 8*(r/4) + 4*(lane/32) + r%4
// for accumulator register r = 0..15.
#include <hip/hip_runtime.h>

#include <type_traits>
#include <utility>

#include "kernels.h"

namespace mi {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

enum Epilogue { EPI_NONE = 0, EPI_BIAS_RELU = 1, EPI_MASK = 2 };

struct GemmArgs {
  int M, N, K;
  const float* A;
  const float* B;
  float* C;
  int lda, ldb, ldc;
  // batch: element offsets added per batch index
  long long batchA, batchB, batchC;
  // epilogue
  const float* bias;  // EPI_BIAS_RELU: [N] or null
  int relu;           // EPI_BIAS_RELU
  const float* mask;  // EPI_MASK: [M x N], result zeroed where mask <= 0
  int ldmask;
  // fused column sums of the A operand (TN only): colsum[z*batchColsum + m] = sum_k A[k][m]
  float* colsum;
  long long batchColsum;
  // GUARD kernels: which 16-byte vector accesses the alignment of pointers and leading dimensions
  // allows (bit 0: A loads, bit 1: B loads, bit 2: C stores and mask loads)
  int vec_flags;
  // tile rasterisation (flat grid of tiles_m * tiles_n * batch workgroups)
  int tiles_m, tiles_n, batch;
  int raster, per_xcd, total_shift, tiles_n_shift;  // see tile_of_block / set_raster
  // CHAIN instances of gemm_f32_dma: number of batch entries a workgroup walks through
  int chain;
};

// Maps the flat workgroup index to a batch entry and a C tile.  Workgroups are handed to the 8
// XCDs round-robin (id % 8), each XCD has a private 4 MB L2, and about 32 workgroups (one per CU)
// of an XCD run at the same time.
//   * raster 2, large grids (tile counts divisible as needed): the grid of one batch entry is cut
//     into super-tiles of 4 x 8 tiles; XCD x owns super-tiles x, x+8, ... and walks each row by
//     row, so the 32 tiles it runs together share 4 A panels and 8 B panels.
//   * raster 1, otherwise, if the tile count of the whole batch is a multiple of 8: XCD x gets the
//     contiguous range [x*T/8, (x+1)*T/8) of the (batch entry, row, column) order, so that the
//     tiles it runs together belong to as few batch entries and rows as possible (tiles of one row
//     share their A panel, tiles of one batch entry their B panels).
//   * raster 0, otherwise the identity.
// The host chooses (set_raster) and passes the divisors' logarithms where they are powers of two:
// every wavefront runs this before its first load, and an integer division is about 25 scalar
// instructions.
__device__ __forceinline__ int div_tiles(int x, int d, int shift) { return shift >= 0 ? x >> shift : x / d; }

__device__ __forceinline__ void tile_of_block(const GemmArgs& p, int& tm, int& tn, int& z) {
  int id = blockIdx.x;
  const int total = p.tiles_m * p.tiles_n;
  if (p.raster == 2) {
    z = div_tiles(id, total, p.total_shift);  // total is a multiple of 8, so id % 8 is still the XCD
    id -= z * total;
    const int xcd = id & 7, j = id >> 3;
    const int super = (j >> 5) * 8 + xcd, within = j & 31;
    const int super_cols = p.tiles_n >> 3;
    const int sr = div_tiles(super, super_cols, p.tiles_n_shift >= 3 ? p.tiles_n_shift - 3 : -1);
    tm = sr * 4 + (within >> 3);
    tn = (super - sr * super_cols) * 8 + (within & 7);
    return;
  }
  if (p.raster == 1) id = (id & 7) * p.per_xcd + (id >> 3);
  z = div_tiles(id, total, p.total_shift);
  id -= z * total;
  tm = div_tiles(id, p.tiles_n, p.tiles_n_shift);
  tn = id - tm * p.tiles_n;
}

// Host side of tile_of_block; tiles_m and tiles_n are set.
static inline int log2_if_pow2(int v) {
  if (v <= 0 || (v & (v - 1)) != 0) return -1;
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}
static inline void set_raster(GemmArgs& p, int batch) {
  const int total = p.tiles_m * p.tiles_n;
  p.batch = batch;
  p.total_shift = log2_if_pow2(total);
  p.tiles_n_shift = log2_if_pow2(p.tiles_n);
  p.per_xcd = 0;
  if ((p.tiles_m & 3) == 0 && (p.tiles_n & 7) == 0 && (total & 255) == 0 && total >= 512) {
    p.raster = 2;
  } else if ((((long long)total * batch) & 7) == 0) {
    p.raster = 1;
    p.per_xcd = (int)(((long long)total * batch) >> 3);
  } else {
    p.raster = 0;
  }
}

// Workgroup barrier that orders LDS traffic only: unlike __syncthreads() it does not wait for
// global loads still in flight, so prefetches may cross it.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int ROWS, int BK, bool KMAJOR>
struct TileShape {
  // K-major: [ROWS][BK + 4]; M-major: [BK][ROWS]
  static constexpr int kStride = KMAJOR ? (BK + 4) : ROWS;
  static constexpr int kFloats = KMAJOR ? ROWS * (BK + 4) : BK * ROWS;
  static constexpr int kVecs = ROWS * BK / 4;  // float4 per tile
};

// Global -> registers for one operand tile.  `base` points at the tile's first element for this
// K step.  NV = float4 per thread.
template <int ROWS, int BK, bool KMAJOR, int NT, int NV>
__device__ __forceinline__ void load_tile(f32x4 (&v)[NV], const float* __restrict__ base, int ld,
                                          int tid) {
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * NT;
    if (KMAJOR) {
      const int row = idx / (BK / 4), c4 = idx % (BK / 4);
      v[i] = *reinterpret_cast<const f32x4*>(base + (size_t)row * ld + c4 * 4);
    } else {
      const int k = idx / (ROWS / 4), c4 = idx % (ROWS / 4);
      v[i] = *reinterpret_cast<const f32x4*>(base + (size_t)k * ld + c4 * 4);
    }
  }
}

// Same for a tile that may stick out of the matrix (GUARD kernels): `op` points at the operand,
// the tile covers rows [row0, row0 + ROWS) of `rows_total` and k in [k0, k0 + BK) of K; whatever
// lies outside is read as zero, so the MFMAs need no special cases.
template <int ROWS, int BK, bool KMAJOR, int NT, int NV>
__device__ __forceinline__ void load_tile_guard(f32x4 (&v)[NV], const float* __restrict__ op, int ld, int row0,
                                                int rows_total, int k0, int K, int tid, bool vec) {
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * NT;
    f32x4 t = {0.0f, 0.0f, 0.0f, 0.0f};
    if (KMAJOR) {
      const int row = row0 + idx / (BK / 4), k = k0 + (idx % (BK / 4)) * 4;
      if (row < rows_total && k < K) {
        const float* src = op + (size_t)row * ld + k;
        if (vec && k + 3 < K) {
          t = *reinterpret_cast<const f32x4*>(src);
        } else if (k + 3 < K) {
          t[0] = src[0]; t[1] = src[1]; t[2] = src[2]; t[3] = src[3];
        } else {
          t[0] = src[0];
          if (k + 1 < K) t[1] = src[1];
          if (k + 2 < K) t[2] = src[2];
        }
      }
    } else {
      const int k = k0 + idx / (ROWS / 4), row = row0 + (idx % (ROWS / 4)) * 4;
      if (k < K && row < rows_total) {
        const float* src = op + (size_t)k * ld + row;
        if (vec && row + 3 < rows_total) {
          t = *reinterpret_cast<const f32x4*>(src);
        } else if (row + 3 < rows_total) {
          t[0] = src[0]; t[1] = src[1]; t[2] = src[2]; t[3] = src[3];
        } else {
          t[0] = src[0];
          if (row + 1 < rows_total) t[1] = src[1];
          if (row + 2 < rows_total) t[2] = src[2];
        }
      }
    }
    v[i] = t;
  }
}

template <int ROWS, int BK, bool KMAJOR, int NT, int NV>
__device__ __forceinline__ void store_tile(float* lds, const f32x4 (&v)[NV], int tid) {
  using TS = TileShape<ROWS, BK, KMAJOR>;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int idx = tid + i * NT;
    if (KMAJOR) {
      const int row = idx / (BK / 4), c4 = idx % (BK / 4);
      *reinterpret_cast<f32x4*>(lds + row * TS::kStride + c4 * 4) = v[i];
    } else {
      const int k = idx / (ROWS / 4), c4 = idx % (ROWS / 4);
      *reinterpret_cast<f32x4*>(lds + k * TS::kStride + c4 * 4) = v[i];
    }
  }
}

// LDS -> fragment registers for one 8-wide K chunk.  frag[b][q]: value for block b, MFMA step q.
template <int ROWS, int BK, bool KMAJOR, int TB>
__device__ __forceinline__ void load_frag(float (&frag)[TB][4], const float* lds, int wave_row0,
                                          int kk, int lane) {
  using TS = TileShape<ROWS, BK, KMAJOR>;
  const int l32 = lane & 31, hi = lane >> 5;
  if (KMAJOR) {
#pragma unroll
    for (int b = 0; b < TB; ++b) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(lds + (wave_row0 + b * 32 + l32) * TS::kStride +
                                                      kk * 8 + hi * 4);
      frag[b][0] = t[0];
      frag[b][1] = t[1];
      frag[b][2] = t[2];
      frag[b][3] = t[3];
    }
  } else {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float* src = lds + (kk * 8 + hi * 4 + q) * TS::kStride + wave_row0 + TB * l32;
      if (TB == 4) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(src);
        frag[0][q] = t[0];
        frag[1 % TB][q] = t[1];
        frag[2 % TB][q] = t[2];
        frag[3 % TB][q] = t[3];
      } else if (TB == 2) {
        const f32x2 t = *reinterpret_cast<const f32x2*>(src);
        frag[0][q] = t[0];
        frag[1 % TB][q] = t[1];
      } else {
        frag[0][q] = src[0];
      }
    }
  }
}

// ---- epilogue: registers -> global, fused bias/ReLU or ReLU mask ------------------------------
// Writes the TM x TN accumulator blocks of one wavefront; (m0w, n0w) is the wavefront's first
// row / column in C.
template <int TM, int TN, bool A_KMAJOR, bool B_KMAJOR, int EPI, bool GUARD>
__device__ __forceinline__ void write_tile(const GemmArgs& p, float* __restrict__ C, f32x16 (&acc)[TM][TN], int m0w,
                                           int n0w, int lane) {
  // Column of (block j, value e) held by this lane: K-major B keeps the blocks side by side,
  // N-major B interleaves them so that the lane owns TN consecutive columns (one vector store).
  const int l32 = lane & 31, hi = lane >> 5;
  const int col0 = n0w + (B_KMAJOR ? l32 : TN * l32);
  constexpr int CSTEP = B_KMAJOR ? 32 : 1;
  const float* __restrict__ mask = p.mask;

  // GUARD: element (row, column j of this lane) exists
  auto col_ok = [&](int j) { return !GUARD || col0 + j * CSTEP < p.N; };
  constexpr bool VEC_STORE = !B_KMAJOR && (TN == 2 || TN == 4);
  // a vector access covers TN consecutive columns starting at col0; with GUARD it needs all of them
  const bool vec_ok = VEC_STORE && (!GUARD || ((p.vec_flags & 4) && col0 + TN - 1 < p.N));

  float bias_v[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
    bias_v[j] = (EPI == EPI_BIAS_RELU && p.bias && col_ok(j)) ? p.bias[col0 + j * CSTEP] : 0.0f;

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    // rows of accumulator registers r = 0..15 of block row i
    auto row_of = [&](int r) {
      const int rb32 = 8 * (r >> 2) + 4 * hi + (r & 3);
      return m0w + (A_KMAJOR ? i * 32 + rb32 : TM * rb32 + i);
    };
    // all mask reads of this block row first, so that they are in flight together
    float mk[16][TN];
    if (EPI == EPI_MASK) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = row_of(r);
        const float* mrow = mask + (size_t)row * p.ldmask + col0;
        const bool row_ok = !GUARD || row < p.M;
        if (VEC_STORE && TN == 4 && vec_ok && row_ok) {
          const f32x4 t = *reinterpret_cast<const f32x4*>(mrow);
          mk[r][0] = t[0]; mk[r][1 % TN] = t[1]; mk[r][2 % TN] = t[2]; mk[r][3 % TN] = t[3];
        } else if (VEC_STORE && TN == 2 && vec_ok && row_ok) {
          const f32x2 t = *reinterpret_cast<const f32x2*>(mrow);
          mk[r][0] = t[0]; mk[r][1 % TN] = t[1];
        } else {
#pragma unroll
          for (int j = 0; j < TN; ++j) mk[r][j] = (row_ok && col_ok(j)) ? mrow[j * CSTEP] : 0.0f;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = row_of(r);
      if (GUARD && row >= p.M) continue;
      float* crow = C + (size_t)row * p.ldc + col0;
      float v[TN];
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        v[j] = acc[i][j][r];
        if (EPI == EPI_BIAS_RELU) {
          v[j] += bias_v[j];
          if (p.relu) v[j] = v[j] > 0.0f ? v[j] : 0.0f;
        } else if (EPI == EPI_MASK) {
          if (!(mk[r][j] > 0.0f)) v[j] = 0.0f;
        }
      }
      if (VEC_STORE && TN == 4 && vec_ok) {
        const f32x4 o = {v[0], v[1 % TN], v[2 % TN], v[3 % TN]};
        *reinterpret_cast<f32x4*>(crow) = o;
      } else if (VEC_STORE && TN == 2 && vec_ok) {
        const f32x2 o = {v[0], v[1 % TN]};
        *reinterpret_cast<f32x2*>(crow) = o;
      } else {
#pragma unroll
        for (int j = 0; j < TN; ++j)
          if (col_ok(j)) crow[j * CSTEP] = v[j];
      }
    }
  }
}

// COLSUM (weight gradient only, A stored [k][m]): the workgroups of tile column 0 also add up the
// columns of their A tile while it sits in LDS.  Every thread takes part so that no wavefront
// falls behind: thread t owns column t % BM and the k rows of slice t / BM of every K step; the
// NT / BM partial sums of a column are combined through LDS in slice order at the end, so the
// result does not depend on scheduling.  The extra LDS reads and adds run in the shadow of the
// MFMAs.
//
// STAGES selects the software pipeline:
//   2  two LDS buffers; loads of step t+1 are issued at the top of step t, written to LDS at its
//      end, one barrier per step at the step boundary.
//   3  three LDS buffers; the tile of step t+1 (loaded during step t-1) is written to LDS at the
//      top of step t, the loads of step t+2 are issued right after, and the one barrier per step
//      sits in the middle of the step, where it only has to absorb the skew between wavefronts.
//      Step boundaries carry no synchronisation at all, and the operand fragments of the next
//      8-wide K chunk are always fetched from LDS while the current chunk is multiplied.
//      PF (1 or 2) is the distance, in K steps, between issuing a tile's global loads and
//      writing it to LDS; 2 covers an L2 miss without stalling the step that needs the data.
//
// GUARD = true: M, N and K need not be multiples of the tile; loads outside the matrices read zero
// and the epilogue skips what lies outside C.  (Leading dimensions and base pointers must still be
// 16-byte aligned; anything else goes to the any-shape kernel below.)
template <int BM, int BN, int BK, int WM, int WN, bool A_KMAJOR, bool B_KMAJOR, int EPI, bool COLSUM = false,
          int STAGES = 2, int PF = 1, bool GUARD = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_f32_mfma(GemmArgs p) {
  static_assert(STAGES == 2 || STAGES == 3, "two or three LDS buffers");
  static_assert(!GUARD || (STAGES == 3 && PF == 1), "the guarded loads are written for the 3-stage loop");
  static_assert(STAGES == 2 || (BK / 8) % 2 == 0, "the 3-stage loop alternates two fragment sets per chunk");
  static_assert(!COLSUM || (!A_KMAJOR && (WM * WN * 64) % BM == 0 && BK % ((WM * WN * 64) / BM) == 0),
                "fused column sums need A stored [k][m] and a whole number of k slices");
  constexpr int NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN;  // wavefront sub-tile
  constexpr int TM = WTM / 32, TN = WTN / 32;  // 32x32 blocks per wavefront
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wavefront tile must be whole 32x32 blocks");
  static_assert(BK % 8 == 0, "BK must be a multiple of 8");
  static_assert(A_KMAJOR || TM == 1 || TM == 2 || TM == 4, "interleaved A needs TM in {1,2,4}");
  static_assert(B_KMAJOR || TN == 1 || TN == 2 || TN == 4, "interleaved B needs TN in {1,2,4}");
  using TA = TileShape<BM, BK, A_KMAJOR>;
  using TB = TileShape<BN, BK, B_KMAJOR>;
  static_assert(TA::kVecs % NT == 0 && TB::kVecs % NT == 0, "tile must divide over the threads");
  constexpr int NVA = TA::kVecs / NT, NVB = TB::kVecs / NT;

  extern __shared__ __attribute__((aligned(16))) float smem[];
  // LDS layout: [A buffers 0..STAGES-1][B buffers 0..STAGES-1]
  auto As = [&](int buf) { return smem + buf * TA::kFloats; };
  auto Bs = [&](int buf) { return smem + STAGES * TA::kFloats + buf * TB::kFloats; };

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WN) * WTM, wn0 = (wave % WN) * WTN;

  int tile_m, tile_n, bz;
  tile_of_block(p, tile_m, tile_n, bz);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const float* __restrict__ A = p.A + (size_t)bz * p.batchA;
  const float* __restrict__ B = p.B + (size_t)bz * p.batchB;
  float* __restrict__ C = p.C + (size_t)bz * p.batchC;

  // first element of this workgroup's panel, and the pointer advance per K step
  const float* a_ptr = A_KMAJOR ? A + (size_t)m0 * p.lda : A + m0;
  const float* b_ptr = B_KMAJOR ? B + (size_t)n0 * p.ldb : B + n0;
  const size_t a_step = A_KMAJOR ? (size_t)BK : (size_t)BK * p.lda;
  const size_t b_step = B_KMAJOR ? (size_t)BK : (size_t)BK * p.ldb;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  constexpr int CS_SLICES = COLSUM ? NT / BM : 1;  // k slices per step, one per group of BM threads
  constexpr int CS_ROWS = BK / CS_SLICES;
  const bool do_colsum = COLSUM && p.colsum != nullptr && tile_n == 0;  // uniform over the workgroup
  float csum = 0.0f;

  f32x4 ra[NVA], rb[NVB];
  const int nk = GUARD ? (p.K + BK - 1) / BK : p.K / BK;
  int kt = 0;  // index of the next K tile to request (GUARD loads address from scratch)
  const float* __restrict__ a_op = p.A + (size_t)bz * p.batchA;
  const float* __restrict__ b_op = p.B + (size_t)bz * p.batchB;
  auto mfma_chunk = [&](const float (&fa)[TM][4], const float (&fb)[TN][4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][q], fb[j][q], acc[i][j], 0, 0, 0);
  };
  auto colsum_step = [&](const float* a_tile) {
    const float* col = a_tile + (tid / BM) * CS_ROWS * TA::kStride + (tid % BM);
#pragma unroll
    for (int k = 0; k < CS_ROWS; ++k) csum += col[k * TA::kStride];
  };

  if constexpr (GUARD) {
    load_tile_guard<BM, BK, A_KMAJOR, NT, NVA>(ra, a_op, p.lda, m0, p.M, 0, p.K, tid, p.vec_flags & 1);
    load_tile_guard<BN, BK, B_KMAJOR, NT, NVB>(rb, b_op, p.ldb, n0, p.N, 0, p.K, tid, p.vec_flags & 2);
    kt = 1;
  } else {
    load_tile<BM, BK, A_KMAJOR, NT, NVA>(ra, a_ptr, p.lda, tid);
    load_tile<BN, BK, B_KMAJOR, NT, NVB>(rb, b_ptr, p.ldb, tid);
  }
  store_tile<BM, BK, A_KMAJOR, NT, NVA>(As(0), ra, tid);
  store_tile<BN, BK, B_KMAJOR, NT, NVB>(Bs(0), rb, tid);

  if constexpr (STAGES == 2) {
    __syncthreads();
    for (int t = 0; t < nk; ++t) {
      const int cur = t & 1;
      if (t + 1 < nk) {
        a_ptr += a_step;
        b_ptr += b_step;
        load_tile<BM, BK, A_KMAJOR, NT, NVA>(ra, a_ptr, p.lda, tid);
        load_tile<BN, BK, B_KMAJOR, NT, NVB>(rb, b_ptr, p.ldb, tid);
      }
#pragma unroll
      for (int kk = 0; kk < BK / 8; ++kk) {
        float fa[TM][4], fb[TN][4];
        load_frag<BM, BK, A_KMAJOR, TM>(fa, As(cur), wm0, kk, lane);
        load_frag<BN, BK, B_KMAJOR, TN>(fb, Bs(cur), wn0, kk, lane);
        mfma_chunk(fa, fb);
      }
      if (COLSUM && do_colsum) colsum_step(As(cur));
      if (t + 1 < nk) {
        store_tile<BM, BK, A_KMAJOR, NT, NVA>(As(cur ^ 1), ra, tid);
        store_tile<BN, BK, B_KMAJOR, NT, NVB>(Bs(cur ^ 1), rb, tid);
      }
      __syncthreads();
    }
  } else {
    constexpr int CH = BK / 8;  // 8-wide K chunks per step
    // Global loads run PF steps ahead of their use.  With PF == 2 two register sets alternate:
    // tiles with an odd index travel through (ra2, rb2), even ones through (ra, rb).
    f32x4 ra2[PF == 2 ? NVA : 1], rb2[PF == 2 ? NVB : 1];
    auto fetch = [&](auto& sa, auto& sb) {
      if constexpr (GUARD) {
        load_tile_guard<BM, BK, A_KMAJOR, NT, NVA>(sa, a_op, p.lda, m0, p.M, kt * BK, p.K, tid, p.vec_flags & 1);
        load_tile_guard<BN, BK, B_KMAJOR, NT, NVB>(sb, b_op, p.ldb, n0, p.N, kt * BK, p.K, tid, p.vec_flags & 2);
        ++kt;
      } else {
        a_ptr += a_step;
        b_ptr += b_step;
        load_tile<BM, BK, A_KMAJOR, NT, NVA>(sa, a_ptr, p.lda, tid);
        load_tile<BN, BK, B_KMAJOR, NT, NVB>(sb, b_ptr, p.ldb, tid);
      }
    };
    if constexpr (PF == 2) {
      if (nk > 1) fetch(ra2, rb2);
      if (nk > 2) fetch(ra, rb);
    } else {
      if (nk > 1) fetch(ra, rb);
    }
    lds_barrier();
    float fa[2][TM][4], fb[2][TN][4];
    load_frag<BM, BK, A_KMAJOR, TM>(fa[0], As(0), wm0, 0, lane);
    load_frag<BN, BK, B_KMAJOR, TN>(fb[0], Bs(0), wn0, 0, lane);
    int cur = 0;
    // One K step; (sa, sb) hold tile t+1 on entry and receive tile t+1+PF.  STEADY = true is the
    // body of the main loop, where a next tile and a tile to request always exist: without the
    // conditionals the compiler counts the outstanding LDS operations exactly, so the MFMAs of a
    // chunk wait for their own fragments only (with the conditional version the waits collapse
    // towards "all LDS operations done").  Measured: +2..5 % on every shape.  Pinning the
    // instruction order on top of that with sched_barriers was measured too and loses 1..3 %
    // (up to 13 % with two workgroups per CU): the scheduler's own interleaving is kept.
    auto step = [&](int t, auto& sa, auto& sb, auto steady) {
      constexpr bool STEADY = decltype(steady)::value;
      const int nxt = cur == 2 ? 0 : cur + 1;
#pragma unroll
      for (int kk = 0; kk < CH; ++kk) {
        const int fc = kk & 1, fn = fc ^ 1;
        // fragments of the next chunk: same buffer, or chunk 0 of the next step's buffer (made
        // visible by this step's barrier, which lies before the last chunk)
        if (kk + 1 < CH) {
          load_frag<BM, BK, A_KMAJOR, TM>(fa[fn], As(cur), wm0, kk + 1, lane);
          load_frag<BN, BK, B_KMAJOR, TN>(fb[fn], Bs(cur), wn0, kk + 1, lane);
        } else if (STEADY || t + 1 < nk) {
          load_frag<BM, BK, A_KMAJOR, TM>(fa[fn], As(nxt), wm0, 0, lane);
          load_frag<BN, BK, B_KMAJOR, TN>(fb[fn], Bs(nxt), wn0, 0, lane);
        }
        if (kk == 0) {
          if (STEADY || t + 1 < nk) {  // tile t+1 was requested PF whole steps ago
            store_tile<BM, BK, A_KMAJOR, NT, NVA>(As(nxt), sa, tid);
            store_tile<BN, BK, B_KMAJOR, NT, NVB>(Bs(nxt), sb, tid);
          }
          if (STEADY || t + 1 + PF < nk) fetch(sa, sb);
        }
        mfma_chunk(fa[fc], fb[fc]);
        if (kk == CH - 2) lds_barrier();
        if (kk == CH - 1 && COLSUM && do_colsum) colsum_step(As(cur));
      }
      cur = nxt;
    };
    const std::true_type steady_step;
    const std::false_type edge_step;
    if constexpr (PF == 2) {
      int t = 0;
      for (; t + 4 < nk; t += 2) {  // both steps of the pair have t + 1 + PF < nk
        step(t, ra2, rb2, steady_step);
        step(t + 1, ra, rb, steady_step);
      }
      for (; t < nk; t += 2) {
        step(t, ra2, rb2, edge_step);
        if (t + 1 < nk) step(t + 1, ra, rb, edge_step);
      }
    } else {
      int t = 0;
      for (; t + 2 < nk; ++t) step(t, ra, rb, steady_step);
      for (; t < nk; ++t) step(t, ra, rb, edge_step);
    }
  }

  if (COLSUM && do_colsum) {
    __syncthreads();  // every wavefront is done with the operand tiles: reuse LDS for the partials
    smem[tid] = csum;
    __syncthreads();
    if (tid < BM) {
      float total = smem[tid];
#pragma unroll
      for (int sl = 1; sl < CS_SLICES; ++sl) total += smem[sl * BM + tid];
      if (!GUARD || m0 + tid < p.M) p.colsum[(size_t)bz * p.batchColsum + m0 + tid] = total;
    }
  }

  write_tile<TM, TN, A_KMAJOR, B_KMAJOR, EPI, GUARD>(p, C, acc, m0 + wm0, n0 + wn0, lane);
}

// ---- the same GEMM with direct global -> LDS loads ----------------------------------------------
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight into the LDS: the 64
// lanes of one instruction fill 1 KB of consecutive LDS bytes from a wave-uniform base (lane i
// lands at base + 16 i) while every lane names its own global address.  The tile no longer passes
// through VGPRs: the ds_write of the next tile and the wait for its global loads at the top of
// every K step -- measured at 7 % of the register-staged kernel's time -- disappear.
//
// LDS layouts (no padding, an instruction's 1 KB must be contiguous):
//   K-major operand  [row][BK]; the 16-byte chunk c of row r sits at chunk position c ^ swz(r),
//                    swz(r) = (r / rows per 256 bytes) mod chunks per row.  The swizzle is produced
//                    on the global side (the lane that fills position pc of row r fetches chunk
//                    pc ^ swz(r)); the 16 lanes the LDS serves together on a fragment read (same
//                    chunk, 16 consecutive rows) then touch all 64 banks once.
//   M-major operand  [k][ROWS], as in the register-staged kernel.
//
// Ring of STAGES buffers; in the middle of step t every wave waits (vmcnt) until its own loads of
// tile t+1 have landed, all waves meet at one barrier, and the loads of tile t+STAGES-1 are issued
// into the buffer step t-1 read.  The load is inline assembly on purpose: the compiler models the
// builtin as a FLAT access that may touch both memories and then turns every later LDS-counter
// wait into lgkmcnt(0) while such a load is pending; written this way it does not track the load
// at all and the kernel counts vmcnt itself (compiler-inserted vmcnt waits can only get longer
// through the extra loads in flight, never shorter: vmcnt retires in order).
// The order of fragment reads and MFMAs inside a chunk is left to the compiler: pinning "reads of
// the next chunk first" with sched_barrier was measured 2-4 % slower, interleaving reads between
// MFMAs with sched_group_barrier within +-1 %.  The one pinned point is the fence in front of the
// ring barrier (see the step below).  Also measured without gain: issuing the loads after the last
// chunk's MFMAs instead of right after the barrier, rings of four and five buffers at BK = 16,
// 128 x 64 tiles with two workgroups per CU, 4 and 16 wavefronts per workgroup, non-temporal
// stores in the epilogue.  Timestamps taken inside the kernel: 1.3 us from the start of a
// workgroup to its first tile in the LDS, 1.6 us from the last K step to the last store issued.
__device__ __forceinline__ void load_to_lds_f32(const float* uniform_base, unsigned lane_byte_offset,
                                                unsigned lds_byte_addr) {
  const unsigned lds_addr = __builtin_amdgcn_readfirstlane(lds_byte_addr);
  const unsigned long long b = reinterpret_cast<unsigned long long>(uniform_base);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b), hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  const unsigned long long sbase = ((unsigned long long)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(lane_byte_offset), "s"(sbase)
               : "memory", "m0");
}

template <int... S, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, S...>, F&& f) {
  (f(std::integral_constant<int, S>{}), ...);
}
// f(integral_constant<int, 0>), ..., f(integral_constant<int, N-1>)
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14,
// expcnt 6:4, lgkmcnt 11:8; the other counters at their maximum = no wait).
constexpr int vmcnt_only(int n) { return (n & 15) | ((n >> 4) << 14) | 0x70 | 0xf00; }

template <int ROWS, int BK>
struct SwizzledTile {
  static constexpr int kChunks = BK / 4;                                   // 16-byte chunks per row
  static constexpr int kRowsPerLine = 256 / (BK * 4) > 0 ? 256 / (BK * 4) : 1;
  static __device__ __forceinline__ int swz(int row) { return (row / kRowsPerLine) % kChunks; }
};

// K-major fragment read from the swizzled layout: same values as load_frag<.., true, ..>.
template <int ROWS, int BK, int TB>
__device__ __forceinline__ void load_frag_swz(float (&frag)[TB][4], const float* lds, int wave_row0, int kk, int lane) {
  using ST = SwizzledTile<ROWS, BK>;
  const int l32 = lane & 31, hi = lane >> 5;
#pragma unroll
  for (int b = 0; b < TB; ++b) {
    const int row = wave_row0 + b * 32 + l32;
    const f32x4 t = *reinterpret_cast<const f32x4*>(lds + row * BK + ((kk * 2 + hi) ^ ST::swz(row)) * 4);
    frag[b][0] = t[0];
    frag[b][1] = t[1];
    frag[b][2] = t[2];
    frag[b][3] = t[3];
  }
}

// CHAIN = true (weight gradient with a short K per replica): the replicas of one launch are
// consecutive ranges of K rows of both operands (batchA = K * lda, batchB = K * ldb), so a
// workgroup that keeps its (m, n) tile and walks through all p.chain replicas sees one long K loop
// whose ring of tile loads never drains; every p.K / BK steps it stores the accumulators as that
// replica's C tile (and the column sums as its bias gradient), clears them and goes on.  Prologue
// and epilogue are paid once per workgroup instead of once per replica, and the stores of a replica
// drain under the next replica's MFMAs: the wait in front of the next ring barrier lets them stay
// in flight (vmcnt retires in order, and the tile that barrier needs was requested before them).
// Measured on 20 layers of 2048 x 2048 with 8 replicas of 256 rows: 127-129 us per launch against
// 139 us for one workgroup per (replica, tile).  How many replicas a workgroup should walk is a
// matter of the whole step, see dispatch(): all 8 make the step slower, groups of 4 faster.
template <int BM, int BN, int BK, int WM, int WN, bool A_KMAJOR, bool B_KMAJOR, int EPI, bool COLSUM, int STAGES,
          bool CHAIN = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_f32_dma(GemmArgs p) {
  static_assert(!CHAIN || (!A_KMAJOR && !B_KMAJOR && EPI == EPI_NONE), "chained replicas: weight gradient only");
  constexpr int NW = WM * WN, NT = NW * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int CH = BK / 8;
  constexpr int A_FLOATS = BM * BK, B_FLOATS = BN * BK;
  // load instructions per wave and tile: an instruction covers 1 KB = 256 floats of the tile
  constexpr int NIA = A_FLOATS / 256 / NW, NIB = B_FLOATS / 256 / NW, INSTR = NIA + NIB;
  static_assert(STAGES >= 3 && STAGES <= 5, "ring depth");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && CH % 2 == 0, "tile shape");
  static_assert(A_FLOATS % (256 * NW) == 0 && B_FLOATS % (256 * NW) == 0, "tile must divide over the waves");
  static_assert((STAGES - 2) * INSTR <= 63, "vmcnt is a 6-bit counter");
  static_assert(A_KMAJOR || TM == 1 || TM == 2 || TM == 4, "interleaved A needs TM in {1,2,4}");
  static_assert(B_KMAJOR || TN == 1 || TN == 2 || TN == 4, "interleaved B needs TN in {1,2,4}");
  static_assert(!COLSUM || (!A_KMAJOR && NT % BM == 0 && BK % (NT / BM) == 0),
                "fused column sums need A stored [k][m] and a whole number of k slices");

  extern __shared__ __attribute__((aligned(16))) float smem[];
  auto As = [&](int buf) { return smem + buf * A_FLOATS; };
  auto Bs = [&](int buf) { return smem + STAGES * A_FLOATS + buf * B_FLOATS; };
  const unsigned lds_base = (unsigned)(size_t)((__attribute__((address_space(3))) const void*)smem);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WN) * WTM, wn0 = (wave % WN) * WTN;

  int tile_m, tile_n, bz;
  tile_of_block(p, tile_m, tile_n, bz);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  if (CHAIN) bz *= p.chain;  // the grid's batch index counts groups of p.chain consecutive entries
  float* __restrict__ C = p.C + (size_t)bz * p.batchC;
  float* __restrict__ colsum_out = COLSUM && p.colsum ? p.colsum + (size_t)bz * p.batchColsum + m0 : nullptr;

  // Global source of the load instructions: a wave-uniform base pointer per operand (the tile's
  // first element for the current K step, advanced with scalar adds) plus a constant 32-bit byte
  // offset per lane and instruction -- no vector arithmetic in the K loop.
  unsigned offa[NIA], offb[NIB];
  auto offsets = [&](auto& off, auto kmajor, auto rows_c, int ld, int ni) {
    constexpr bool KM = decltype(kmajor)::value;
    constexpr int ROWS = decltype(rows_c)::value;
    for (int j = 0; j < ni; ++j) {
      const int unit = j * NW + wave;  // which 1 KB piece of the tile
      if (KM) {
        using ST = SwizzledTile<ROWS, BK>;
        constexpr int RPI = 64 / ST::kChunks;
        const int row = unit * RPI + lane / ST::kChunks, pc = lane % ST::kChunks;
        off[j] = 4u * ((unsigned)row * (unsigned)ld + (unsigned)(pc ^ ST::swz(row)) * 4u);
      } else {
        constexpr int CPR = ROWS / 4, KPI = 64 / CPR > 0 ? 64 / CPR : 1;
        static_assert(CPR <= 64, "a tile row must fit one load instruction");
        const int k = unit * KPI + lane / CPR, c = lane % CPR;
        off[j] = 4u * ((unsigned)k * (unsigned)ld + (unsigned)c * 4u);
      }
    }
  };
  offsets(offa, std::integral_constant<bool, A_KMAJOR>{}, std::integral_constant<int, BM>{}, p.lda, NIA);
  offsets(offb, std::integral_constant<bool, B_KMAJOR>{}, std::integral_constant<int, BN>{}, p.ldb, NIB);
  const float* a_base = p.A + (size_t)bz * p.batchA + (A_KMAJOR ? (size_t)m0 * p.lda : (size_t)m0);
  const float* b_base = p.B + (size_t)bz * p.batchB + (B_KMAJOR ? (size_t)n0 * p.ldb : (size_t)n0);
  const size_t a_step = A_KMAJOR ? (size_t)BK : (size_t)BK * p.lda;
  const size_t b_step = B_KMAJOR ? (size_t)BK : (size_t)BK * p.ldb;
  auto issue = [&](int buf) {
#pragma unroll
    for (int j = 0; j < NIA; ++j)
      load_to_lds_f32(a_base, offa[j], lds_base + 4u * (unsigned)(buf * A_FLOATS + (j * NW + wave) * 256));
#pragma unroll
    for (int j = 0; j < NIB; ++j)
      load_to_lds_f32(b_base, offb[j], lds_base + 4u * (unsigned)(STAGES * A_FLOATS + buf * B_FLOATS + (j * NW + wave) * 256));
    a_base += a_step;
    b_base += b_step;
  };
  auto frags = [&](float (&fa)[TM][4], float (&fb)[TN][4], int buf, int kk) {
    if constexpr (A_KMAJOR) load_frag_swz<BM, BK, TM>(fa, As(buf), wm0, kk, lane);
    else load_frag<BM, BK, false, TM>(fa, As(buf), wm0, kk, lane);
    if constexpr (B_KMAJOR) load_frag_swz<BN, BK, TN>(fb, Bs(buf), wn0, kk, lane);
    else load_frag<BN, BK, false, TN>(fb, Bs(buf), wn0, kk, lane);
  };
  // Barrier of the ring.  Nothing is written with ds_write, so no LDS-counter wait is needed for
  // visibility; a buffer is refilled only after the MFMAs that consumed its last fragments.  The
  // fused column sums read the tile with plain LDS loads whose consumers the compiler may delay,
  // so that instantiation drains the LDS counter first.
  auto ring_barrier = [&]() {
    if constexpr (COLSUM) __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0) only
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  constexpr int CS_SLICES = COLSUM ? NT / BM : 1;
  constexpr int CS_ROWS = BK / CS_SLICES;
  const bool do_colsum = COLSUM && p.colsum != nullptr && tile_n == 0;
  float csum = 0.0f;

  const int steps_per_entry = p.K / BK;                       // CHAIN: K steps per replica
  const int nk = CHAIN ? steps_per_entry * p.chain : steps_per_entry;
  int steps_left = steps_per_entry;                           // CHAIN: steps until the accumulators are stored
  bool stores_in_flight = false;                              // CHAIN: the previous step ended with a store burst
  // one float per thread behind the ring: partial column sums of a replica (CHAIN; the ring itself is never idle)
  float* cs_smem = smem + STAGES * (A_FLOATS + B_FLOATS);
  constexpr int TILE_STORES = TM * TN * 16 / ((!B_KMAJOR && (TN == 2 || TN == 4)) ? TN : 1);  // store instructions of write_tile per wave
#pragma unroll
  for (int st = 0; st < STAGES - 1; ++st)
    if (st < nk) issue(st);
  if (nk >= STAGES - 1) __builtin_amdgcn_s_waitcnt(vmcnt_only((STAGES - 2) * INSTR));
  else __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
  ring_barrier();

  float fa[2][TM][4], fb[2][TN][4];
  frags(fa[0], fb[0], 0, 0);
  // One K step at ring position `cur`.  The position is a compile-time constant (the loop below
  // is unrolled over the ring) so that every LDS address of the step is a register plus an
  // immediate offset.
  auto step = [&](int t, auto cur_c, auto steady_c) {
    constexpr int cur = decltype(cur_c)::value;
    constexpr bool steady = decltype(steady_c)::value;  // tiles t+1 .. t+STAGES-1 all exist
    constexpr int nxt = cur + 1 == STAGES ? 0 : cur + 1;
    constexpr int fill = cur == 0 ? STAGES - 1 : cur - 1;
#pragma unroll
    for (int kk = 0; kk < CH; ++kk) {
      const int fc = kk & 1, fn = fc ^ 1;
      if (kk + 1 < CH) frags(fa[fn], fb[fn], cur, kk + 1);
      else frags(fa[fn], fb[fn], nxt, 0);  // after the last tile: a harmless read of ring memory, keeps one code path
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[fc][i][q], fb[fc][j][q], acc[i][j], 0, 0, 0);
      if (kk == CH - 2) {
        // The barrier does not order register-only instructions, and the scheduler otherwise sinks
        // this chunk's MFMAs below it in some steps: the wavefronts then meet at the barrier with an
        // empty MFMA pipe (measured: every such step 12 % longer).
        __builtin_amdgcn_sched_barrier(0);
        // tiles t+1 .. t+STAGES-2 are in flight; tile t+1 must have landed
        if (CHAIN && stores_in_flight) {
          // the stores of the replica that ended with the previous step are younger than every load
          // that has to be complete here: they may stay outstanding
          if (steady || t + STAGES - 2 < nk) __builtin_amdgcn_s_waitcnt(vmcnt_only((STAGES - 3) * INSTR + TILE_STORES));
          else __builtin_amdgcn_s_waitcnt(vmcnt_only(TILE_STORES));
        } else {
          if (steady || t + STAGES - 2 < nk) __builtin_amdgcn_s_waitcnt(vmcnt_only((STAGES - 3) * INSTR));
          else __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
        }
        ring_barrier();
        if (steady || t + STAGES - 1 < nk) issue(fill);
      }
      if (kk == CH - 1 && COLSUM && do_colsum) {
        const float* col = As(cur) + (tid / BM) * CS_ROWS * BM + (tid % BM);
#pragma unroll
        for (int k = 0; k < CS_ROWS; ++k) csum += col[k * BM];
      }
    }
    if constexpr (CHAIN) {
      stores_in_flight = false;
      if (--steps_left == 0 && t + 1 < nk) {  // a replica is complete (the last one leaves through the epilogue below)
        steps_left = steps_per_entry;
        if (COLSUM && do_colsum) {  // uniform over the workgroup
          cs_smem[tid] = csum;
          csum = 0.0f;
          lds_barrier();
          if (tid < BM) {
            float total = cs_smem[tid];
#pragma unroll
            for (int sl = 1; sl < CS_SLICES; ++sl) total += cs_smem[sl * BM + tid];
            colsum_out[tid] = total;
          }
          colsum_out += p.batchColsum;
          // cs_smem is written again one replica later at the earliest, i.e. behind a ring barrier
        }
        write_tile<TM, TN, A_KMAJOR, B_KMAJOR, EPI, false>(p, C, acc, m0 + wm0, n0 + wn0, lane);
        C += p.batchC;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        stores_in_flight = true;
      }
    }
  };
  // Steady part: whole turns of the ring whose steps all refill a buffer -- straight-line code
  // with no branch for the scheduler to stop at.
  int t = 0;
  for (; t + 2 * STAGES - 1 <= nk; t += STAGES)
    static_for<STAGES>([&](auto sc) { step(t + decltype(sc)::value, sc, std::true_type{}); });
  // fewer than 2 * STAGES - 1 steps are left; the ring is back at position 0
  static_for<2 * STAGES - 2>([&](auto sc) {
    constexpr int s = decltype(sc)::value;
    if (t + s < nk) step(t + s, std::integral_constant<int, s % STAGES>{}, std::false_type{});
  });

  if (COLSUM && do_colsum) {
    __syncthreads();  // every wavefront is done with the operand tiles: reuse LDS for the partials
    smem[tid] = csum;
    __syncthreads();
    if (tid < BM) {
      float total = smem[tid];
#pragma unroll
      for (int sl = 1; sl < CS_SLICES; ++sl) total += smem[sl * BM + tid];
      colsum_out[tid] = total;
    }
  }
  write_tile<TM, TN, A_KMAJOR, B_KMAJOR, EPI, false>(p, C, acc, m0 + wm0, n0 + wn0, lane);
}

// ---- small problems: 32 x 32 tiles, K split over the four wavefronts of a workgroup --------------
// With fewer 64 x 64 tiles than CUs (config 1: 512 x 512 outputs) the tiled kernels leave most
// SIMDs idle and every wavefront walks the whole K on its own: 256 dependent 64-cycle MFMAs.  Here
// a workgroup owns one 32 x 32 block of C and each of its four wavefronts (one per SIMD)
// multiplies a quarter of K, so a 512 x 512 x 512 GEMM puts 64 MFMAs on each of the 1024 SIMDs.
// The wavefronts share no operand data, so fragments are loaded from global memory straight into
// the registers the MFMAs read -- no LDS tile, no barrier in the loop (the operands of such small
// problems sit in the L2).  The four partial blocks are added through the LDS in wavefront order
// (deterministic), wavefront w finishing rows 8w .. 8w+7 of the block.
// NW = 8 (the forward GEMM from K = 512 on, see splitk_eight_waves): eight wavefronts, two per SIMD,
// with an eighth of K each -- half the chain of dependent MFMAs per wavefront, which is what a
// launch of one workgroup per CU waits for; wavefront w then finishes the accumulator registers
// 2w and 2w+1.
// `tile` = index of the 32 x 32 block in row-major order, `z` = batch entry, `lds` = the
// workgroup's SPLITK_LDS_FLOATS(NW) floats of LDS.
#define SPLITK_LDS_FLOATS(NW) ((NW) * 16 * 64 + (NW) * 32)
template <bool A_KMAJOR, bool B_KMAJOR, int EPI, bool COLSUM, int NW = 4, int DEPTH = 4>
__device__ __forceinline__ void splitk_block(const GemmArgs& p, int tile, int z, float* lds) {
  static_assert(NW == 4 || NW == 8, "split of K over the wavefronts");
  float(*part)[16][64] = reinterpret_cast<float(*)[16][64]>(lds);             // [NW][16][64]
  float(*cs_part)[32] = reinterpret_cast<float(*)[32]>(lds + NW * 16 * 64);  // [NW][32]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hi = lane >> 5;
  const int tile_m = tile / p.tiles_n, tile_n = tile - tile_m * p.tiles_n;
  const int m0 = tile_m * 32, n0 = tile_n * 32;
  const float* __restrict__ A = p.A + (size_t)z * p.batchA;
  const float* __restrict__ B = p.B + (size_t)z * p.batchB;
  float* __restrict__ C = p.C + (size_t)z * p.batchC;
  const int kq = p.K / NW, k_begin = wave * kq, chunks = kq / 8;
  // lane (l32, hi) feeds MFMA step q of a chunk with k = chunk*8 + 4*hi + q
  const float* a_ptr = A_KMAJOR ? A + (size_t)(m0 + l32) * p.lda + k_begin + 4 * hi
                                : A + (size_t)(k_begin + 4 * hi) * p.lda + m0 + l32;
  const float* b_ptr = B_KMAJOR ? B + (size_t)(n0 + l32) * p.ldb + k_begin + 4 * hi
                                : B + (size_t)(k_begin + 4 * hi) * p.ldb + n0 + l32;
  const size_t a_step = A_KMAJOR ? 8 : (size_t)8 * p.lda, b_step = B_KMAJOR ? 8 : (size_t)8 * p.ldb;
  auto fetch = [](float (&f)[4], const float* ptr, int ld, bool kmajor) {
    if (kmajor) {
      const f32x4 t = *reinterpret_cast<const f32x4*>(ptr);
      f[0] = t[0]; f[1] = t[1]; f[2] = t[2]; f[3] = t[3];
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q) f[q] = ptr[(size_t)q * ld];
    }
  };
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
  const bool do_colsum = COLSUM && p.colsum != nullptr && tile_n == 0;
  float cs = 0.0f;
  float fa[DEPTH][4], fb[DEPTH][4];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (d < chunks) {
      fetch(fa[d], a_ptr + d * a_step, p.lda, A_KMAJOR);
      fetch(fb[d], b_ptr + d * b_step, p.ldb, B_KMAJOR);
    }
  for (int c = 0; c < chunks; c += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (c + d >= chunks) break;
      float ua[4], ub[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) { ua[q] = fa[d][q]; ub[q] = fb[d][q]; }
      if (c + d + DEPTH < chunks) {
        fetch(fa[d], a_ptr + (size_t)(c + d + DEPTH) * a_step, p.lda, A_KMAJOR);
        fetch(fb[d], b_ptr + (size_t)(c + d + DEPTH) * b_step, p.ldb, B_KMAJOR);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ua[q], ub[q], acc, 0, 0, 0);
        if (COLSUM && do_colsum) cs += ua[q];
      }
    }
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) part[wave][r][lane] = acc[r];
  if (COLSUM && do_colsum) {
    cs += __shfl_xor(cs, 32, 64);  // the two lane halves hold different k of the same column
    if (hi == 0) cs_part[wave][l32] = cs;
  }
  __syncthreads();
  if (COLSUM && do_colsum && tid < 32) {
    float total = cs_part[0][tid];
#pragma unroll
    for (int w = 1; w < NW; ++w) total += cs_part[w][tid];
    p.colsum[(size_t)z * p.batchColsum + m0 + tid] = total;
  }
  const int col = n0 + l32;
  const float bias_v = (EPI == EPI_BIAS_RELU && p.bias) ? p.bias[col] : 0.0f;
#pragma unroll
  for (int e = 0; e < 16 / NW; ++e) {
    const int r = (16 / NW) * wave + e;
    float v = part[0][r][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) v += part[w][r][lane];
    const int row = m0 + 8 * (r / 4) + 4 * hi + (r % 4);  // register r holds row 8*(r/4) + 4*hi + r%4
    if (EPI == EPI_BIAS_RELU) {
      v += bias_v;
      if (p.relu) v = v > 0.0f ? v : 0.0f;
    } else if (EPI == EPI_MASK) {
      if (!(p.mask[(size_t)row * p.ldmask + col] > 0.0f)) v = 0.0f;
    }
    C[(size_t)row * p.ldc + col] = v;
  }
}

// Eight wavefronts for the forward GEMM (both operands K-contiguous) when every wavefront still
// gets whole sub-blocks of the direct-load kernel below: the two kernels add the same partial sums
// in the same order and give the same bits.
static inline bool splitk_eight_waves(bool a_kmajor, bool b_kmajor, int K) {
  return a_kmajor && b_kmajor && K >= 512 && K % 256 == 0;
}

template <bool A_KMAJOR, bool B_KMAJOR, int EPI, bool COLSUM, int NW>
__global__ __launch_bounds__(NW * 64) void gemm_f32_splitk(GemmArgs p) {
  __shared__ float lds[SPLITK_LDS_FLOATS(NW)];
  splitk_block<A_KMAJOR, B_KMAJOR, EPI, COLSUM, NW>(p, blockIdx.x, blockIdx.z, lds);
}

// The split-K kernel for two K-contiguous operands (the forward GEMM) with direct-to-LDS loads.
// Loaded straight into registers, a K-contiguous fragment is 32-byte pieces of 32 different rows
// per instruction; brought in through the LDS, a load instruction of a wavefront covers 4 rows x
// 256 contiguous bytes.  Each wavefront owns its quarter of K and a private LDS region for it, so
// there is no barrier in the loop: sub-blocks of 64 k (8 KB per operand) travel through two
// buffers, the wavefront waits for its own loads (vmcnt) and multiplies from the LDS (rows of 256
// bytes, 16-byte chunks XOR-swizzled with the row so that fragment reads touch every bank once).
// NW = 8, SW = 32: eight wavefronts with an eighth of K each and sub-blocks of 32 k (rows of 128
// bytes, 8 rows per load instruction), the same 128 KB of LDS: half the chain of dependent MFMAs
// per wavefront (K = 512: 32 instead of 64), which is what a launch of one workgroup per CU waits for.
template <int EPI, int NW, int SW>
__global__ __launch_bounds__(NW * 64) void gemm_f32_splitk_dma(GemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr int SB = 32 * SW;         // floats of one operand's sub-block (SW = k per sub-block)
  constexpr int CH = SW / 4;          // 16-byte chunks per row
  constexpr int RPI = 64 / CH;        // rows one load instruction covers
  constexpr int NI = 32 / RPI;        // load instructions per operand and sub-block
  static_assert(NW * 4 * SB * sizeof(float) <= 128 * 1024 && (CH == 8 || CH == 16), "sub-block shape");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;
  const int tile_m = blockIdx.x / p.tiles_n, tile_n = blockIdx.x - tile_m * p.tiles_n;
  const int m0 = tile_m * 32, n0 = tile_n * 32;
  const int kq = p.K / NW, nsb = kq / SW;
  float* region = smem + wave * (4 * SB);  // [buffer][A | B]
  const unsigned lds_base = (unsigned)(size_t)((__attribute__((address_space(3))) const void*)region);
  // load instruction j covers rows RPI j .. RPI j + RPI - 1; lane i fills chunk position i % CH of row RPI j + i / CH
  unsigned offa[NI], offb[NI];
#pragma unroll
  for (int j = 0; j < NI; ++j) {
    const int row = RPI * j + lane / CH, pos = lane % CH;
    offa[j] = 4u * ((unsigned)row * (unsigned)p.lda + (unsigned)((pos ^ (row & (CH - 1))) * 4));
    offb[j] = 4u * ((unsigned)row * (unsigned)p.ldb + (unsigned)((pos ^ (row & (CH - 1))) * 4));
  }
  const float* a_base = p.A + (size_t)m0 * p.lda + (size_t)wave * kq;
  const float* b_base = p.B + (size_t)n0 * p.ldb + (size_t)wave * kq;
  auto issue = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NI; ++j) load_to_lds_f32(a_base, offa[j], lds_base + 4u * (unsigned)(buf * 2 * SB + j * 256));
#pragma unroll
    for (int j = 0; j < NI; ++j) load_to_lds_f32(b_base, offb[j], lds_base + 4u * (unsigned)(buf * 2 * SB + SB + j * 256));
    a_base += SW;
    b_base += SW;
  };
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
  issue(0);
  if (nsb > 1) issue(1);
  for (int sb = 0; sb < nsb; ++sb) {
    const int cur = sb & 1;
    if (sb + 1 < nsb) __builtin_amdgcn_s_waitcnt(vmcnt_only(2 * NI));  // the younger sub-block may stay in flight
    else __builtin_amdgcn_s_waitcnt(vmcnt_only(0));
    asm volatile("" ::: "memory");
    const float* a_tile = region + cur * 2 * SB + l32 * SW;
    const float* b_tile = a_tile + SB;
#pragma unroll
    for (int kk = 0; kk < SW / 8; ++kk) {
      const int chunk = ((2 * kk + hi) ^ (l32 & (CH - 1))) * 4;
      const f32x4 fa = *reinterpret_cast<const f32x4*>(a_tile + chunk);
      const f32x4 fb = *reinterpret_cast<const f32x4*>(b_tile + chunk);
#pragma unroll
      for (int q = 0; q < 4; ++q) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[q], fb[q], acc, 0, 0, 0);
    }
    if (sb + 2 < nsb) {
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this buffer's fragments are in registers
      asm volatile("" ::: "memory");
      issue(cur);
    }
  }
  // add the partial blocks in wavefront order, as the register-loading kernel does
  __syncthreads();
  float(*part)[16][64] = reinterpret_cast<float(*)[16][64]>(smem);
#pragma unroll
  for (int r = 0; r < 16; ++r) part[wave][r][lane] = acc[r];
  __syncthreads();
  const int col = n0 + l32;
  const float bias_v = (EPI == EPI_BIAS_RELU && p.bias) ? p.bias[col] : 0.0f;
#pragma unroll
  for (int e = 0; e < 16 / NW; ++e) {
    const int r = (16 / NW) * wave + e;
    float v = part[0][r][lane];
#pragma unroll
    for (int w = 1; w < NW; ++w) v += part[w][r][lane];
    const int row = m0 + 8 * (r / 4) + 4 * hi + (r % 4);  // register r holds row 8*(r/4) + 4*hi + r%4
    if (EPI == EPI_BIAS_RELU) {
      v += bias_v;
      if (p.relu) v = v > 0.0f ? v : 0.0f;
    }
    p.C[(size_t)row * p.ldc + col] = v;
  }
}

// The two backward GEMMs of one layer in one launch: the weight gradient (all replicas, bias
// gradient fused) and the input gradient read the same dZ and depend on nothing of each other.  For
// problems this small a step is a chain of launches of a few microseconds each, and one launch less
// per layer is worth more than anything inside the kernels.  Workgroups [0, dgrad_blocks) run the
// input gradient, the rest the weight gradient (tile fastest, then replica): a block of the input
// gradient walks R times the K of a weight-gradient block, so the long blocks start first and the
// short ones fill in behind them.
// Chunks of 8 k a wavefront of the paired launch requests ahead.  With three workgroups per CU
// the other eleven wavefronts of the CU cover a wavefront's wait, and every request more in flight
// (3 072 wavefronts ask at once) makes the launch slower: config 1 step 59.4 us with four chunks
// ahead, 58.5 with three, 57.3 with two, 53.7 with one, 62.9-66.5 with eight.  The separate
// launches (one or two workgroups per CU) keep four: with two their input gradient takes 24.5
// instead of 21 us.
constexpr int PAIR_DEPTH = 1;
template <int EPI_D>
__global__ __launch_bounds__(256) void gemm_f32_splitk_pair(GemmArgs pw, GemmArgs pd, int dgrad_blocks) {
  __shared__ float lds[SPLITK_LDS_FLOATS(4)];  // one region for either kind of block
  const int b = blockIdx.x;
  if (b < dgrad_blocks) {
    splitk_block<true, false, EPI_D, false, 4, PAIR_DEPTH>(pd, b, 0, lds);
  } else {
    const int per = pw.tiles_m * pw.tiles_n, w = b - dgrad_blocks, z = w / per;
    splitk_block<false, false, EPI_NONE, true, 4, PAIR_DEPTH>(pw, w - z * per, z, lds);
  }
}

// ---- any-shape fallback ----------------------------------------------------------------------
// Plain LDS-tiled SIMT kernel with fully guarded loads and stores; used when a dimension is not
// a multiple of the MFMA tile or a pointer / leading dimension is not 16-byte aligned.
// 16 x 16 threads, each computing a 4 x 4 patch of a 64 x 64 tile.
template <bool A_KMAJOR, bool B_KMAJOR, int EPI>
__global__ __launch_bounds__(256) void gemm_f32_generic(GemmArgs p) {
  constexpr int T = 64, KS = 16;
  __shared__ float As[KS][T + 1];
  __shared__ float Bs[KS][T + 1];
  const float* __restrict__ A = p.A + (size_t)blockIdx.z * p.batchA;
  const float* __restrict__ B = p.B + (size_t)blockIdx.z * p.batchB;
  float* __restrict__ C = p.C + (size_t)blockIdx.z * p.batchC;
  const int m0 = blockIdx.y * T, n0 = blockIdx.x * T;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < p.K; k0 += KS) {
    for (int e = threadIdx.x; e < T * KS; e += 256) {
      int r, k;
      if (A_KMAJOR) { r = e / KS; k = e % KS; } else { k = e / T; r = e % T; }
      const int gm = m0 + r, gka = k0 + k;
      float v = 0.0f;
      if (gm < p.M && gka < p.K) v = A_KMAJOR ? A[(size_t)gm * p.lda + gka] : A[(size_t)gka * p.lda + gm];
      As[k][r] = v;
      if (B_KMAJOR) { r = e / KS; k = e % KS; } else { k = e / T; r = e % T; }
      const int gn = n0 + r, gkb = k0 + k;
      v = 0.0f;
      if (gn < p.N && gkb < p.K) v = B_KMAJOR ? B[(size_t)gn * p.ldb + gkb] : B[(size_t)gkb * p.ldb + gn];
      Bs[k][r] = v;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < KS; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + ty * 4 + i;
    if (row >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (col >= p.N) continue;
      float v = acc[i][j];
      if (EPI == EPI_BIAS_RELU) {
        if (p.bias) v += p.bias[col];
        if (p.relu) v = v > 0.0f ? v : 0.0f;
      } else if (EPI == EPI_MASK) {
        if (!(p.mask[(size_t)row * p.ldmask + col] > 0.0f)) v = 0.0f;
      }
      C[(size_t)row * p.ldc + col] = v;
    }
  }
}

// ---- launch ------------------------------------------------------------------------------------

template <int BM, int BN, int BK, int WM, int WN, bool AK, bool BKM, int EPI, bool COLSUM, int STAGES = 2, int PF = 1,
          bool GUARD = false>
static hipError_t launch_mfma(GemmArgs& p, int batch, hipStream_t s) {
  using TA = TileShape<BM, BK, AK>;
  using TB = TileShape<BN, BK, BKM>;
  constexpr size_t lds_bytes = STAGES * (TA::kFloats + TB::kFloats) * sizeof(float);
  auto kern = gemm_f32_mfma<BM, BN, BK, WM, WN, AK, BKM, EPI, COLSUM, STAGES, PF, GUARD>;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) return e;
  p.tiles_m = GUARD ? (p.M + BM - 1) / BM : p.M / BM;
  p.tiles_n = GUARD ? (p.N + BN - 1) / BN : p.N / BN;
  set_raster(p, batch);
  launch_kernel(kern, dim3(p.tiles_m * p.tiles_n * batch), dim3(WM * WN * 64), lds_bytes, s, p);
  return hipGetLastError();
}

// `exclusive`: ask for more than half of the CU's LDS, so that no second workgroup (of this or of
// another kernel) shares the CU.  A workgroup of these kernels keeps the MFMA pipes of its CU busy
// on its own; co-resident ones only interfere, and with several rounds of workgroups they make the
// hardware's hand-out of workgroups to CUs uneven (measured on 1024 tiles: launches of 910 us and
// of 1120 us at random with three 48 KB workgroups per CU, 910 us always with one).
template <int BM, int BN, int BK, int WM, int WN, bool AK, bool BKM, int EPI, bool COLSUM, int STAGES, bool CHAIN = false>
static hipError_t launch_dma(GemmArgs& p, int batch, hipStream_t s, bool exclusive = false) {
  // CHAIN: one float per thread behind the ring for the column-sum partials of a replica
  constexpr size_t lds_bytes = STAGES * (size_t)(BM + BN) * BK * sizeof(float) + (CHAIN ? WM * WN * 64 * sizeof(float) : 0);
  static_assert(lds_bytes <= 160 * 1024, "tile does not fit the 160 KB of LDS");
  constexpr size_t kExclusiveBytes = 84 * 1024;
  const size_t request = exclusive && lds_bytes < kExclusiveBytes ? kExclusiveBytes : lds_bytes;
  auto kern = gemm_f32_dma<BM, BN, BK, WM, WN, AK, BKM, EPI, COLSUM, STAGES, CHAIN>;
  if (CHAIN) {  // a workgroup walks p.chain consecutive batch entries itself: the grid covers batch / p.chain groups
    if (p.chain <= 0 || batch % p.chain != 0) p.chain = batch;
    batch /= p.chain;
  }
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), request); e != hipSuccess) return e;
  p.tiles_m = p.M / BM;
  p.tiles_n = p.N / BN;
  set_raster(p, batch);
  launch_kernel(kern, dim3(p.tiles_m * p.tiles_n * batch), dim3(WM * WN * 64), request, s, p);
  return hipGetLastError();
}

template <bool AK, bool BKM, int EPI, bool COLSUM>
static hipError_t launch_splitk(GemmArgs& p, int batch, hipStream_t s) {
  p.tiles_m = p.M / 32;
  p.tiles_n = p.N / 32;
  if (splitk_eight_waves(AK, BKM, p.K))
    launch_kernel((gemm_f32_splitk<AK, BKM, EPI, COLSUM, 8>), dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(512), 0, s, p);
  else
    launch_kernel((gemm_f32_splitk<AK, BKM, EPI, COLSUM, 4>), dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(256), 0, s, p);
  return hipGetLastError();
}

template <int EPI>
static hipError_t launch_splitk_dma(GemmArgs& p, hipStream_t s) {
  constexpr size_t lds_bytes = 4 * 4 * 32 * 64 * sizeof(float);  // wavefronts x 2 buffers x 2 operands x sub-block: 128 KB either way
  p.tiles_m = p.M / 32;
  p.tiles_n = p.N / 32;
  if (splitk_eight_waves(true, true, p.K)) {
    auto kern = gemm_f32_splitk_dma<EPI, 8, 32>;
    static LdsOptIn opt_in;
    if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) return e;
    launch_kernel(kern, dim3(p.tiles_m * p.tiles_n), dim3(512), lds_bytes, s, p);
  } else {
    auto kern = gemm_f32_splitk_dma<EPI, 4, 64>;
    static LdsOptIn opt_in;
    if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) return e;
    launch_kernel(kern, dim3(p.tiles_m * p.tiles_n), dim3(256), lds_bytes, s, p);
  }
  return hipGetLastError();
}

template <bool AK, bool BKM, int EPI>
static hipError_t launch_generic(GemmArgs& p, int batch, hipStream_t s) {
  dim3 grid((p.N + 63) / 64, (p.M + 63) / 64, batch);
  launch_kernel((gemm_f32_generic<AK, BKM, EPI>), grid, dim3(256), 0, s, p);
  return hipGetLastError();
}

static inline bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

// The automatic choice as far as the shape decides it (aligned operands assumed): which tiling a
// GEMM of M x N x K with `batch` entries gets.  dispatch() and the paired backward launch of small
// models both ask this one function, so that the paired launch and the separate launches always
// run the same kernel on the same shape (and so add up in the same order).
enum AutoTile { AUTO_128, AUTO_128x64, AUTO_SPLITK, AUTO_64, AUTO_GUARDED };
static AutoTile auto_tile(int M, int N, int K, long long batch) {
  auto whole = [&](int bm, int bn, int bk) { return K > 0 && M % bm == 0 && N % bn == 0 && K % bk == 0; };
  const long long tiles128 = (long long)(M / 128) * (N / 128) * batch;
  // More than 128 big tiles: 128 x 128, one workgroup per CU.  Half tiles would then number more than
  // the 256 CUs, and the CUs that get two of them decide the launch (1536 x 1536 x 1536, 144 big
  // tiles: 95.7 us on 128 x 128, 120.8 us on 128 x 64; 3072 x 1024 x 1024: 70.7 / 85.3 us).  Up to 128
  // big tiles the half tiles still have a CU each (2048 x 1024 x 1024: 64.8 / 47.0 us).
  if (whole(128, 128, 16) && tiles128 > 128) return AUTO_128;
  if (whole(128, 64, 32) && tiles128 * 2 >= 192) return AUTO_128x64;
  if (whole(32, 32, 32) && (long long)(M / 64) * (N / 64) * batch < 192) return AUTO_SPLITK;  // fewer 64 x 64 tiles than CUs
  if (whole(64, 64, 16)) return AUTO_64;
  return AUTO_GUARDED;
}

// Picks a tile configuration.  `variant` (0 = automatic) lets the tuning harness force one.
// `fused_colsum` reports whether the chosen kernel also produced p.colsum.
template <bool AK, bool BKM, int EPI, bool COLSUM = false>
static hipError_t dispatch(GemmArgs& p, int batch, hipStream_t s, int variant, bool* fused_colsum = nullptr) {
  if (fused_colsum) *fused_colsum = false;
  if (p.M <= 0 || p.N <= 0 || batch <= 0) return hipSuccess;
  const bool vec_ok = aligned16(p.A) && aligned16(p.B) && aligned16(p.C) && p.lda % 4 == 0 &&
                      p.ldb % 4 == 0 && p.ldc % 4 == 0 && p.batchA % 4 == 0 && p.batchB % 4 == 0 &&
                      p.batchC % 4 == 0 && p.K > 0;
  // vector reads of the mask need the same alignment as the stores to C
  const bool mask_ok = EPI != EPI_MASK || (aligned16(p.mask) && p.ldmask % 4 == 0);
  auto fits = [&](int bm, int bn, int bk) {
    return vec_ok && mask_ok && p.M % bm == 0 && p.N % bn == 0 && p.K % bk == 0;
  };
  const bool forced = variant != 0;
  if (variant == 0) {
    // Automatic choice.  From about one 128 x 128 tile per CU on, the direct-to-LDS kernels with a
    // ring of three buffers.  Measured on the benchmark configurations, whole step:
    //   * BK = 16 with the CU to itself (variant 34) everywhere, except
    //   * a weight gradient with a short K (small per-replica batch: few K steps, so prologue and
    //     epilogue weigh most) takes BK = 16 at its natural 48 KB and shares CUs; its replicas are
    //     chained in groups (variant 35 with p.chain set) such that about two workgroups per CU
    //     remain: config 4 (8 replicas of 256 rows, 256 tiles each) 7.89 -> 7.78 ms with groups of
    //     4, but 8.0 ms with groups of 2 and 8.6 ms with all 8 in one workgroup, which leaves one
    //     long-lived workgroup per CU and nothing to fill the gaps of the input-gradient chain on
    //     the other stream.  (An earlier state gave the input-gradient GEMM next to such a weight
    //     gradient BK = 32 and 96 KB; with the current kernels BK = 16 is better there too:
    //     7.90 -> 7.76 ms.)
    // Smaller problems fall back to 128 x 64 and 64 x 64 tiles to get enough workgroups, the
    // smallest (config 1) to the split-K kernel.
    constexpr bool kWeightGradient = !AK && !BKM;
    const AutoTile tile = vec_ok && mask_ok ? auto_tile(p.M, p.N, p.K, batch) : AUTO_GUARDED;
    if (tile == AUTO_128) {
      variant = 34;
      if (kWeightGradient && p.K < 512) {
        variant = 33;
        const long long tiles_entry = (long long)(p.M / 128) * (p.N / 128);
        if (EPI == EPI_NONE && p.batchA == (long long)p.K * p.lda && p.batchB == (long long)p.K * p.ldb) {
          int chain = 1;  // largest divisor of the replica count that leaves two workgroups per CU
          for (int c = 2; c <= batch; ++c)
            if (batch % c == 0 && tiles_entry * (batch / c) >= 512) chain = c;
          if (chain > 1) {
            variant = 35;
            p.chain = chain;
          }
        }
      }
    } else if (tile == AUTO_128x64) {
      variant = 11;
    } else if (tile == AUTO_SPLITK) {
      variant = 50;  // fewer 64 x 64 tiles than CUs: 32 x 32 tiles with K split over the wavefronts
      if (AK && BKM && EPI != EPI_MASK && batch == 1 && p.K % 256 == 0) variant = 51;  // both operands K-contiguous: through the LDS
    } else if (tile == AUTO_64) {
      variant = 16;
    } else if (p.K > 0) {
      // ragged shape or unaligned storage: the guarded MFMA kernels, big tile if it fills the chip
      const long long t128 = (long long)((p.M + 127) / 128) * ((p.N + 127) / 128) * batch;
      variant = t128 >= 192 ? 21 : 22;
    } else {
      variant = -1;
    }
  }
  // what the guarded kernels may access with 16-byte vectors
  p.vec_flags = ((aligned16(p.A) && p.lda % 4 == 0 && p.batchA % 4 == 0) ? 1 : 0) |
                ((aligned16(p.B) && p.ldb % 4 == 0 && p.batchB % 4 == 0) ? 2 : 0) |
                ((aligned16(p.C) && p.ldc % 4 == 0 && p.batchC % 4 == 0 && mask_ok) ? 4 : 0);
  switch (variant) {
    case 8: if (fits(128, 128, 32)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<128, 128, 32, 2, 4, AK, BKM, EPI, COLSUM, 3>(p, batch, s); } break;
    case 9: if (fits(128, 128, 32)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<128, 128, 32, 2, 2, AK, BKM, EPI, COLSUM, 3>(p, batch, s); } break;
    case 10: if (fits(128, 128, 16)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<128, 128, 16, 2, 4, AK, BKM, EPI, COLSUM, 3>(p, batch, s); } break;
    case 11: if (fits(128, 64, 32)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<128, 64, 32, 2, 2, AK, BKM, EPI, COLSUM, 3>(p, batch, s); } break;
    case 12: if (fits(128, 64, 16)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<128, 64, 16, 2, 2, AK, BKM, EPI, COLSUM, 3>(p, batch, s); } break;
    case 15: if (fits(128, 64, 32)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<128, 64, 32, 2, 2, AK, BKM, EPI, COLSUM, 2>(p, batch, s); } break;
    case 16: if (fits(64, 64, 16)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<64, 64, 16, 2, 2, AK, BKM, EPI, COLSUM, 3>(p, batch, s); } break;
    case 17: if (fits(128, 128, 32)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<128, 128, 32, 2, 4, AK, BKM, EPI, COLSUM, 3, 2>(p, batch, s); } break;
    case 21: if (p.K > 0) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<128, 128, 32, 2, 4, AK, BKM, EPI, COLSUM, 3, 1, true>(p, batch, s); } break;
    case 22: if (p.K > 0) { if (fused_colsum) *fused_colsum = COLSUM; return launch_mfma<64, 64, 16, 2, 2, AK, BKM, EPI, COLSUM, 3, 1, true>(p, batch, s); } break;
    case 30: if (fits(128, 128, 32)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_dma<128, 128, 32, 2, 4, AK, BKM, EPI, COLSUM, 4>(p, batch, s); } break;
    case 31: if (fits(128, 128, 32)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_dma<128, 128, 32, 2, 4, AK, BKM, EPI, COLSUM, 3>(p, batch, s); } break;
    case 33: if (fits(128, 128, 16)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_dma<128, 128, 16, 2, 4, AK, BKM, EPI, COLSUM, 3>(p, batch, s); } break;
    case 34: if (fits(128, 128, 16)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_dma<128, 128, 16, 2, 4, AK, BKM, EPI, COLSUM, 3>(p, batch, s, true); } break;
    case 35: case 36: case 37:  // forced: 35 = all replicas in one workgroup, 36 / 37 = groups of 2 / 4; automatic: p.chain is set
      if (forced) p.chain = variant == 35 ? 0 : variant == 36 ? 2 : 4;
      if constexpr (!AK && !BKM && EPI == EPI_NONE) {
        if (fits(128, 128, 16) && batch >= 1 && p.batchA == (long long)p.K * p.lda && p.batchB == (long long)p.K * p.ldb) {
          if (fused_colsum) *fused_colsum = COLSUM;
          return launch_dma<128, 128, 16, 2, 4, AK, BKM, EPI, COLSUM, 3, true>(p, batch, s);
        }
      }
      break;
    case 51:
      if constexpr (AK && BKM && EPI != EPI_MASK && !COLSUM) {
        if (fits(32, 32, 256) && batch == 1) return launch_splitk_dma<EPI>(p, s);
      }
      break;
    case 50: if (fits(32, 32, 32)) { if (fused_colsum) *fused_colsum = COLSUM; return launch_splitk<AK, BKM, EPI, COLSUM>(p, batch, s); } break;
    default: break;
  }
  return launch_generic<AK, BKM, EPI>(p, batch, s);
}

hipError_t sgemm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                    int ldc, const float* bias, int relu, hipStream_t s, int variant) {
  // automatic choice: a layer of at most SKINNY_MAX outputs is matrix-vector work
  if (variant == 0 && N <= SKINNY_MAX && K > 0)
    return sgemv_nt(M, N, K, A, lda, B, ldb, C, ldc, bias, relu, s);
  GemmArgs p{};
  p.M = M; p.N = N; p.K = K; p.A = A; p.B = B; p.C = C; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.bias = bias; p.relu = relu;
  return dispatch<true, true, EPI_BIAS_RELU>(p, 1, s, variant);
}

hipError_t sgemm_nn(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                    int ldc, const float* mask, int ldmask, hipStream_t s, int variant) {
  if (variant == 0 && K <= SKINNY_MAX && K > 0)
    return sgemv_nn(M, N, K, A, lda, B, ldb, C, ldc, mask, ldmask, s);
  GemmArgs p{};
  p.M = M; p.N = N; p.K = K; p.A = A; p.B = B; p.C = C; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.mask = mask; p.ldmask = ldmask;
  if (mask) return dispatch<true, false, EPI_MASK>(p, 1, s, variant);
  return dispatch<true, false, EPI_NONE>(p, 1, s, variant);
}

hipError_t sgemm_tn(int R, int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                    float* C, int ldc, long long strideC, float* colsum, long long stride_colsum,
                    hipStream_t s, int variant) {
  if (variant == 0 && M <= SKINNY_MAX && K > 0)
    return sgemv_tn(R, M, N, K, A, lda, B, ldb, C, ldc, strideC, colsum, stride_colsum, s);
  GemmArgs p{};
  p.M = M; p.N = N; p.K = K; p.A = A; p.B = B; p.C = C; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.batchA = (long long)K * lda;  // replica r reads rows [r*K, (r+1)*K) of both operands
  p.batchB = (long long)K * ldb;
  p.batchC = strideC;
  if (!colsum) return dispatch<false, false, EPI_NONE>(p, R, s, variant);
  p.colsum = colsum;
  p.batchColsum = stride_colsum;
  bool fused = false;
  hipError_t e = dispatch<false, false, EPI_NONE, true>(p, R, s, variant, &fused);
  if (e != hipSuccess || fused) return e;
  return colsum_f32(R, M, K, A, lda, colsum, stride_colsum, s);  // any-shape path: separate kernel
}

// Whether the automatic choice takes the split-K kernel for a GEMM of this shape.
static bool splitk_shape(int M, int N, int K, int batch) {
  return M > 0 && N > 0 && K > 0 && auto_tile(M, N, K, batch) == AUTO_SPLITK;
}

bool sgemm_backward_pair_fits(int R, int rows, int nout, int nin) {
  // weight gradient: M = nout, N = nin, K = rows / R per replica; input gradient: M = rows, N = nin, K = nout
  return R > 0 && rows % R == 0 && splitk_shape(nout, nin, rows / R, R) && splitk_shape(rows, nin, nout, 1) &&
         nout % 4 == 0 && nin % 4 == 0;
}

hipError_t sgemm_backward_pair(int R, int rows, int nout, int nin, const float* dZ, const float* A, const float* W,
                               float* dW, long long strideW, float* db, long long stride_db, float* dA,
                               const float* mask, hipStream_t s) {
  if (!sgemm_backward_pair_fits(R, rows, nout, nin) || !aligned16(dZ) || !aligned16(A) || !aligned16(W) ||
      !aligned16(dW) || !aligned16(dA) || strideW % 4 != 0 || (mask && !aligned16(mask)))
    return hipErrorInvalidValue;
  const int Kw = rows / R;
  GemmArgs pw{};
  pw.M = nout; pw.N = nin; pw.K = Kw; pw.A = dZ; pw.B = A; pw.C = dW; pw.lda = nout; pw.ldb = nin; pw.ldc = nin;
  pw.batchA = (long long)Kw * nout; pw.batchB = (long long)Kw * nin; pw.batchC = strideW;
  pw.colsum = db; pw.batchColsum = stride_db;
  pw.tiles_m = nout / 32; pw.tiles_n = nin / 32;
  GemmArgs pd{};
  pd.M = rows; pd.N = nin; pd.K = nout; pd.A = dZ; pd.B = W; pd.C = dA; pd.lda = nout; pd.ldb = nin; pd.ldc = nin;
  pd.mask = mask; pd.ldmask = nin;
  pd.tiles_m = rows / 32; pd.tiles_n = nin / 32;
  const int wgrad_blocks = pw.tiles_m * pw.tiles_n * R, dgrad_blocks = pd.tiles_m * pd.tiles_n;
  if (mask) launch_kernel(gemm_f32_splitk_pair<EPI_MASK>, dim3(wgrad_blocks + dgrad_blocks), dim3(256), 0, s, pw, pd, dgrad_blocks);
  else launch_kernel(gemm_f32_splitk_pair<EPI_NONE>, dim3(wgrad_blocks + dgrad_blocks), dim3(256), 0, s, pw, pd, dgrad_blocks);
  return hipGetLastError();
}

}  // namespace mi
