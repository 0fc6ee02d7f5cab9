// bf16 GEMM for gfx950 on v_mfma_f32_32x32x16_bf16 (fp32 accumulation), plus the helpers the
// bf16 model needs around it (tiled transpose, row sums).
//
// One kernel shape serves all three GEMMs of the MLP step: C[M,N] = A[M,K] * B[N,K]^T with both
// operands K-contiguous.  A bf16 MFMA wants 8 consecutive k per lane for its row, so an operand
// whose rows are contiguous instead (B of the input-gradient GEMM, both operands of the weight
// gradient) would have to be transposed on its way into the registers; here the handle keeps
// K-contiguous bf16 copies instead (W^T next to W, A_l^T and dZ_l^T next to A_l and dZ_l, written
// by transpose_bf16) -- at the sizes the bf16 path is for, a transpose moves a few hundred MB
// while the GEMM it feeds does TFLOPs:
//   forward          Y   = X    * W^T            A = X,       B = W
//   input gradient   dA  = dZ   * W = dZ * (W^T)^T   A = dZ,  B = W^T
//   weight gradient  dW_r = dZ_r^T * A_r         A = dZ_r^T,  B = A_r^T      (reference call sites
//                                                mlp_omp.cc:474-488, 657-671, 565-580)
//
// Two kernels here.  gemm_bf16_mfma stages the tile through registers: three LDS buffers, tile t+1
// written to LDS at the top of step t, loads of tile t+2 issued right after, one LDS-only barrier
// in the middle of the step, operand fragments of the next 16-wide K chunk fetched while the
// current chunk is multiplied.  gemm_bf16_dma (further down) loads global -> LDS directly.  The
// large GEMMs (256 x 256 tiles covering the CUs, K a multiple of 64) run on a third kernel built
// on v_mfma_f32_16x16x32_bf16, gemm_bf16_x32.hip, which the dispatch below selects; gemm_bf16_dma
// stays for the BK = 32 ring, for outputs that allow no 16-byte stores, and for comparison.
// Tiles are stored [row][BK] with the 16-byte chunks of a row XOR-swizzled (no padding, no bank
// conflicts); a lane fetches its 8 k values of one 32 x 32 block with one 16-byte LDS read.
#include <hip/hip_runtime.h>

#include <type_traits>
#include <utility>

#include "gemm_bf16_common.h"
#include "kernels.h"

namespace mi {
// Writes a wavefront's TM x TN accumulator blocks (32 x 32 each) with the epilogue EPI.  Lane l,
// register r of a block hold row 8*(r/4) + 4*(l/32) + r%4, column l%32.
//
// Transposed second output (p.Ct).  Registers 4g .. 4g+3 of a block are four consecutive rows of
// one column, i.e. 8 contiguous bytes of the transposed copy.  Stored straight from the registers
// these are 8-byte pieces scattered over 32 columns per instruction, which the write path handles
// badly (measured: +160 us on a 1.8 ms GEMM).  With `lds` != nullptr (the caller guarantees the
// workgroup's LDS is free and gives each wavefront its own region of 32 * (TM*64 + 8) bytes) the
// pieces go through the LDS instead, one 32-column block at a time, columns padded by 8 bytes so
// that the 32 lanes of a half-wave hit distinct banks, and are read back as 16-byte chunks: one
// store instruction then writes whole runs of TM*64 contiguous bytes.
// `mask_lds` != nullptr (EPH_MASK): the workgroup's mask tile lies in the LDS, row-major with
// `mask_ld` elements per row; (row_l, col_l) is this wavefront's first row / column inside it.
// MASK_LDS is a template argument, not a test of mask_lds inside the loops: a pointer that may be
// either LDS or global memory turns every mask read into a flat load behind a branch.
// GUARD: the tile may stick out of C; rows >= p.M and columns >= p.N are skipped (and neither bias
// nor mask is read there).  Guarded instances have no transposed second output.
template <int TM, int TN, int EPI, bool MASK_LDS = false, bool GUARD = false>
__device__ __forceinline__ void store_tile_h(const HGemmArgs& p, f32x16 (&acc)[TM][TN], int row0, int colw, int l32,
                                             int hi, u16* lds = nullptr, const u16* mask_lds = nullptr, int mask_ld = 0,
                                             int row_l = 0, int col_l = 0) {
  typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
  const int col0 = colw + l32;
  float bias_v[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
    bias_v[j] = (EPI == EPH_BIAS_RELU && p.bias && (!GUARD || col0 + j * 32 < p.N)) ? p.bias[col0 + j * 32] : 0.0f;
  float* __restrict__ cf = reinterpret_cast<float*>(p.C) + (size_t)blockIdx.z * p.batchC;
  u16* __restrict__ ch = reinterpret_cast<u16*>(p.C) + (size_t)blockIdx.z * p.batchC;
  unsigned pk[TM][TN][8];  // bf16 results, two rows per register: (4g, 4g+1) and (4g+2, 4g+3)

  const unsigned mask_lds_addr = MASK_LDS ? (unsigned)(size_t)((__attribute__((address_space(3))) const void*)mask_lds) : 0u;
  (void)mask_lds_addr;
  if constexpr (EPI == EPH_F32) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = row0 + i * 32 + 8 * (r >> 2) + 4 * hi + (r & 3);
        if (GUARD && row >= p.M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j)
          if (!GUARD || col0 + j * 32 < p.N) cf[(size_t)row * p.ldc + col0 + j * 32] = acc[i][j][r];
      }
    return;
  } else {
    // Two consecutive rows at a time: one v_cvt_pk_bf16_f32 rounds both (round to nearest even, the
    // same result as the integer sequence of f2bf for finite values) and leaves them packed the way
    // the transposed output wants them; the halves go out with 16-bit stores.
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int rp = 0; rp < 8; ++rp) {
        const int row = row0 + i * 32 + 8 * (rp >> 1) + 4 * hi + 2 * (rp & 1);  // and row + 1
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int col = col0 + j * 32;
          if (GUARD && (col >= p.N || row >= p.M)) continue;
          const bool second_row = !GUARD || row + 1 < p.M;
          f32x2_t v = {acc[i][j][2 * rp], acc[i][j][2 * rp + 1]};
          if (EPI == EPH_BIAS_RELU) {
            v[0] += bias_v[j];
            v[1] += bias_v[j];
            if (p.relu) {
              v[0] = v[0] > 0.0f ? v[0] : 0.0f;
              v[1] = v[1] > 0.0f ? v[1] : 0.0f;
            }
          } else if (EPI == EPH_MASK) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              u16 mk;
              if constexpr (MASK_LDS) {
                typedef __attribute__((address_space(3))) const u16 lds_u16;
                mk = reinterpret_cast<lds_u16*>(
                    (__attribute__((address_space(3))) const char*)(size_t)mask_lds_addr)[(row + e - row0 + row_l) * mask_ld + col_l + l32 + j * 32];
              } else {
                mk = (e == 0 || second_row) ? p.mask[(size_t)(row + e) * p.ldmask + col] : (u16)0;
              }
              if (!(bf2f(mk) > 0.0f)) v[e] = 0.0f;
            }
          }
          const unsigned two = __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2_t));
          pk[i][j][rp] = two;
          ch[(size_t)row * p.ldc + col] = (u16)two;
          if (second_row) ch[(size_t)(row + 1) * p.ldc + col] = (u16)(two >> 16);
        }
      }
    }
  }
  if (EPI != EPH_F32 && !GUARD && p.colsum_part) {
    // the two lane halves hold different rows of the same column; one row block = this wavefront's TM * 32 rows
    // (summed from the packed results after the stores, so that nothing extra is live in the loop
    // above: the values added are the rounded ones, i.e. exactly what was written)
    float* part = p.colsum_part + (size_t)(row0 / (TM * 32)) * p.N;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      float c = 0.0f;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int rp = 0; rp < 8; ++rp)
          c += __uint_as_float(pk[i][j][rp] << 16) + __uint_as_float(pk[i][j][rp] & 0xffff0000u);
      const float total = c + __shfl_xor(c, 32, 64);
      if (hi == 0) part[col0 + j * 32] = total;
    }
  }
  if (EPI == EPH_F32 || GUARD || !p.Ct) return;
  if (MASK_LDS && lds) __syncthreads();  // the staging regions overlap the mask tile other wavefronts still read
  // the tile lies inside one row group: ct_rows is a multiple of the tile height
  const int group = row0 / p.ct_rows, m_local0 = row0 - group * p.ct_rows;
  u16* __restrict__ ct = p.Ct + (size_t)group * p.N * p.ct_rows + m_local0;
  if (lds == nullptr) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        u16* dst = ct + (size_t)(col0 + j * 32) * p.ct_rows + i * 32 + 4 * hi;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const u32x2 two = {pk[i][j][2 * g], pk[i][j][2 * g + 1]};
          *reinterpret_cast<u32x2*>(dst + 8 * g) = two;
        }
      }
    return;
  }
  constexpr int COL_BYTES = TM * 64 + 8;  // TM*32 rows of bf16 plus the pad
  constexpr int CHUNKS = TM * 4;          // 16-byte chunks per column
  const int lane = hi * 32 + l32;
  unsigned char* region = reinterpret_cast<unsigned char*>(lds);
#pragma unroll
  for (int j = 0; j < TN; ++j) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const u32x2 two = {pk[i][j][2 * g], pk[i][j][2 * g + 1]};
        *reinterpret_cast<u32x2*>(region + l32 * COL_BYTES + (i * 32 + 8 * g + 4 * hi) * 2) = two;
      }
#pragma unroll
    for (int q = lane; q < 32 * CHUNKS; q += 64) {
      const int c = q / CHUNKS, part = q % CHUNKS;
      // columns start at multiples of 8 bytes only: two 8-byte LDS reads per 16-byte global store
      const u32x2 lo = *reinterpret_cast<const u32x2*>(region + c * COL_BYTES + part * 16);
      const u32x2 up = *reinterpret_cast<const u32x2*>(region + c * COL_BYTES + part * 16 + 8);
      const u32x4 v = {lo[0], lo[1], up[0], up[1]};
      *reinterpret_cast<u32x4*>(ct + (size_t)(colw + j * 32 + c) * p.ct_rows + part * 8) = v;
    }
  }
}

// PF = distance, in K steps, between issuing a tile's global loads and writing it to LDS.  A bf16
// step is short (BK = 32 is two MFMA chunks, about 1000 cycles), so one step does not cover an
// L2 hit; PF register sets rotate, one per in-flight tile.
// STAGES = 2: two LDS buffers and the plain schedule (loads of tile t+1 at the top of step t,
// written to LDS at its end, barrier at the step boundary) -- what fits when BK = 64 makes a
// 256 x 256 tile 72 KB per buffer.  BK = 64 matters for bandwidth: a tile row is then one whole
// 128-byte cache line, where BK = 32 touches half a line per row and step.
// GUARD = true: M, N, K need not be multiples of the tile and nothing need be aligned: a tile's
// loads outside the operands read zero (whole 16-byte pieces where p.vec_a / p.vec_b say that the
// operand's alignment allows vector loads and the piece lies inside K, element by element
// otherwise), and the epilogue skips what lies outside C.
template <int BM, int BN, int BK, int WM, int WN, int EPI, int PF = 1, int STAGES = 3, bool GUARD = false>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_mfma(HGemmArgs p) {
  static_assert(PF >= 1 && PF <= 3, "prefetch distance");
  static_assert(!GUARD || (STAGES == 3 && PF == 1), "the guarded loads are written for the three-buffer loop");
  static_assert(STAGES == 3 || (STAGES == 2 && PF == 1), "two buffers only with the plain schedule");
  constexpr int NT = WM * WN * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int STRIDE = BK;                     // bf16 elements per LDS row: no padding, chunks swizzled
  constexpr int A_ELEMS = BM * STRIDE, B_ELEMS = BN * STRIDE;
  constexpr int VPR = BK / 8;                    // 16-byte vectors per tile row
  constexpr int NVA = BM * VPR / NT, NVB = BN * VPR / NT;
  constexpr int CH = BK / 16;                    // 16-wide K chunks per step
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 16 == 0, "tile shape");
  static_assert((BM * VPR) % NT == 0 && (BN * VPR) % NT == 0, "tile must divide over the threads");
  static_assert(CH % 2 == 0, "two fragment sets alternate per chunk");

  extern __shared__ __attribute__((aligned(16))) u16 smem_h[];
  auto As = [&](int buf) { return smem_h + buf * A_ELEMS; };
  auto Bs = [&](int buf) { return smem_h + STAGES * A_ELEMS + buf * B_ELEMS; };

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hi = lane >> 5;
  const int wm0 = (wave / WN) * WTM, wn0 = (wave % WN) * WTN;

  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const u16* __restrict__ a_ptr = p.A + (size_t)blockIdx.z * p.batchA + (size_t)m0 * p.lda;
  const u16* __restrict__ b_ptr = p.B + (size_t)blockIdx.z * p.batchB + (size_t)n0 * p.ldb;

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  u32x4 ra[PF][NVA], rb[PF][NVB];
  int k_next = 0;  // GUARD: first k of the next tile to fetch
  // one 16-byte piece (8 consecutive k of one row) that may lie partly or wholly outside the operand
  auto piece = [&](const u16* row_ptr, bool row_ok, int k, bool vec) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (!row_ok || k >= p.K) return v;
    if (vec && k + 8 <= p.K) return *reinterpret_cast<const u32x4*>(row_ptr + k);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const unsigned x = (k + e < p.K) ? (unsigned)row_ptr[k + e] : 0u;
      v[e >> 1] |= x << ((e & 1) * 16);
    }
    return v;
  };
  auto fetch = [&](u32x4 (&sa)[NVA], u32x4 (&sb)[NVB]) {
    if constexpr (GUARD) {
#pragma unroll
      for (int i = 0; i < NVA; ++i) {
        const int idx = tid + i * NT, row = idx / VPR, c = idx % VPR;
        sa[i] = piece(a_ptr + (size_t)row * p.lda, m0 + row < p.M, k_next + c * 8, p.vec_a);
      }
#pragma unroll
      for (int i = 0; i < NVB; ++i) {
        const int idx = tid + i * NT, row = idx / VPR, c = idx % VPR;
        sb[i] = piece(b_ptr + (size_t)row * p.ldb, n0 + row < p.N, k_next + c * 8, p.vec_b);
      }
      k_next += BK;
      return;
    }
#pragma unroll
    for (int i = 0; i < NVA; ++i) {
      const int idx = tid + i * NT, row = idx / VPR, c = idx % VPR;
      sa[i] = *reinterpret_cast<const u32x4*>(a_ptr + (size_t)row * p.lda + c * 8);
    }
#pragma unroll
    for (int i = 0; i < NVB; ++i) {
      const int idx = tid + i * NT, row = idx / VPR, c = idx % VPR;
      sb[i] = *reinterpret_cast<const u32x4*>(b_ptr + (size_t)row * p.ldb + c * 8);
    }
    a_ptr += BK;
    b_ptr += BK;
  };
  // LDS layout.  Rows are stored back to back; the 16-byte chunk c of row r sits at chunk
  // position c ^ swz(r), swz(r) = (r / rows per 256 bytes) mod chunks per row.  The LDS has 64
  // banks of 4 bytes and serves a 16-byte access 16 lanes at a time: 16 lanes reading the same
  // chunk of 16 consecutive rows (the fragment read) and 16 lanes writing consecutive chunks (the
  // tile store) both touch every bank exactly once.
  constexpr int ROWS_PER_LINE = 256 / (BK * 2) > 0 ? 256 / (BK * 2) : 1;
  auto swz = [](int row) { return (row / ROWS_PER_LINE) % VPR; };
  auto stash = [&](int buf, const u32x4 (&sa)[NVA], const u32x4 (&sb)[NVB]) {
#pragma unroll
    for (int i = 0; i < NVA; ++i) {
      const int idx = tid + i * NT, row = idx / VPR, c = idx % VPR;
      *reinterpret_cast<u32x4*>(As(buf) + row * STRIDE + (c ^ swz(row)) * 8) = sa[i];
    }
#pragma unroll
    for (int i = 0; i < NVB; ++i) {
      const int idx = tid + i * NT, row = idx / VPR, c = idx % VPR;
      *reinterpret_cast<u32x4*>(Bs(buf) + row * STRIDE + (c ^ swz(row)) * 8) = sb[i];
    }
  };
  auto load_frags = [&](bf16x8 (&fa)[TM], bf16x8 (&fb)[TN], int buf, int kk) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = wm0 + i * 32 + l32;
      fa[i] = *reinterpret_cast<const bf16x8*>(As(buf) + row * STRIDE + ((kk * 2 + hi) ^ swz(row)) * 8);
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int row = wn0 + j * 32 + l32;
      fb[j] = *reinterpret_cast<const bf16x8*>(Bs(buf) + row * STRIDE + ((kk * 2 + hi) ^ swz(row)) * 8);
    }
  };

  const int nk = GUARD ? (p.K + BK - 1) / BK : p.K / BK;
  fetch(ra[0], rb[0]);
  stash(0, ra[0], rb[0]);
  if constexpr (STAGES == 2) {
    __syncthreads();
    for (int t = 0; t < nk; ++t) {
      const int cur = t & 1;
      if (t + 1 < nk) fetch(ra[0], rb[0]);
#pragma unroll
      for (int kk = 0; kk < CH; ++kk) {
        bf16x8 fa[TM], fb[TN];
        load_frags(fa, fb, cur, kk);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
      if (t + 1 < nk) stash(cur ^ 1, ra[0], rb[0]);
      __syncthreads();
    }
  } else {
  // tile j (j >= 1) travels through register set j % PF
#pragma unroll
  for (int j = 1; j <= PF; ++j)
    if (j < nk) fetch(ra[j % PF], rb[j % PF]);
  lds_barrier_h();
  bf16x8 fa[2][TM], fb[2][TN];
  load_frags(fa[0], fb[0], 0, 0);
  int cur = 0;
  // one K step; `set` holds tile t+1 on entry and receives tile t+1+PF
  auto step = [&](int t, u32x4 (&sa)[NVA], u32x4 (&sb)[NVB]) {
    const int nxt = cur == 2 ? 0 : cur + 1;
#pragma unroll
    for (int kk = 0; kk < CH; ++kk) {
      const int fc = kk & 1, fn = fc ^ 1;
      if (kk + 1 < CH) load_frags(fa[fn], fb[fn], cur, kk + 1);
      else if (t + 1 < nk) load_frags(fa[fn], fb[fn], nxt, 0);
      if (kk == 0) {
        if (t + 1 < nk) stash(nxt, sa, sb);
        if (t + 1 + PF < nk) fetch(sa, sb);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[fc][i], fb[fc][j], acc[i][j], 0, 0, 0);
      if (kk == CH - 2) lds_barrier_h();
    }
    cur = nxt;
  };
  for (int t = 0; t < nk; t += PF) {
#pragma unroll
    for (int u = 0; u < PF; ++u)
      if (t + u < nk) step(t + u, ra[(u + 1) % PF], rb[(u + 1) % PF]);  // t is a multiple of PF
  }
  }

  store_tile_h<TM, TN, EPI, false, GUARD>(p, acc, m0 + wm0, n0 + wn0, l32, hi);
}

// ---- the same GEMM with direct global -> LDS loads ------------------------------------------------
// global_load_lds_dwordx4 moves 16 bytes per lane from global memory straight into the LDS: the
// 64 lanes of one instruction fill 1 KB of consecutive LDS bytes starting at a wave-uniform base
// (lane i lands at base + 16 i), while each lane names its own global address.  The tile never
// passes through VGPRs, so the ds_write traffic of the register-staged kernel (which costs about
// as much LDS time as the fragment reads and kept the MFMA pipe waiting) disappears.  The XOR
// swizzle of the LDS layout is produced on the global side: the lane that fills chunk position
// pc of row r fetches the row's logical chunk pc ^ swz(r).
//
// Ring of STAGES LDS buffers.  In the middle of step t every wave waits (vmcnt) until its own
// loads of tile t+1 have landed, all waves meet at one barrier, and the loads of tile t+STAGES-1
// are issued into the buffer that step t-1 read.  Loads therefore have STAGES-2 whole steps to
// complete; the counter wait leaves the younger tiles in flight.
// The order of fragment reads and MFMAs inside a chunk is left to the compiler (pinning "reads of
// the next chunk first, then this chunk's MFMAs" everywhere with sched_barrier was measured 3.5 %
// slower); only the chunk in front of the barrier is fenced, see the steps below.
//
// The load is written as inline assembly on purpose.  The compiler models the corresponding builtin
// as a FLAT access that may touch both memories and then turns every later LDS-counter wait into
// lgkmcnt(0) while such a load is pending, which serialises the fragment reads with the MFMAs.
// Written this way the compiler does not track the load at all; the kernel waits on vmcnt itself
// (its own waits can only become longer through the extra loads in flight, never shorter, because
// vmcnt retires in order).  m0 carries the wave-uniform LDS byte address.
// The lambdas are always_inline: left to its cost model the compiler keeps the K-step lambdas of
// large instantiations as real functions, and the accumulators they capture then live in memory.
template <int BM, int BN, int BK, int WM, int WN, int EPI, int STAGES, int PRIO = 0>
__global__ __launch_bounds__(WM* WN * 64) void gemm_bf16_dma(HGemmArgs p) {
  constexpr int NW = WM * WN;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int STRIDE = BK;
  constexpr int A_ELEMS = BM * STRIDE, B_ELEMS = BN * STRIDE;
  constexpr int VPR = BK / 8;        // 16-byte chunks per tile row
  constexpr int RPI = 64 / VPR;      // tile rows one load instruction of a wave fills
  constexpr int NIA = BM / (RPI * NW), NIB = BN / (RPI * NW);
  constexpr int INSTR = NIA + NIB;   // load instructions per wave and tile
  constexpr int CH = BK / 16;
  static_assert(STAGES >= 2 && STAGES <= 5, "ring depth");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && CH % 2 == 0, "tile shape");
  static_assert(BM % (RPI * NW) == 0 && BN % (RPI * NW) == 0, "tile must divide over the waves");
  static_assert(STAGES == 2 || (STAGES - 2) * INSTR <= 63, "vmcnt is a 6-bit counter");

  extern __shared__ __attribute__((aligned(16))) u16 smem_h[];
  const unsigned lds_base = (unsigned)(size_t)((__attribute__((address_space(3))) const void*)smem_h);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, hi = lane >> 5;
  const int wm0 = (wave / WN) * WTM, wn0 = (wave % WN) * WTN;

  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  constexpr int ROWS_PER_LINE = 256 / (BK * 2) > 0 ? 256 / (BK * 2) : 1;
  auto swz = [](int row) { return (row / ROWS_PER_LINE) % VPR; };

  // Global source of the load instructions: a wave-uniform base pointer per operand (the tile's
  // first element for the current K step, advanced with scalar adds) plus a constant 32-bit byte
  // offset per lane and instruction.  Together with the compile-time ring positions below this
  // keeps vector arithmetic out of the K loop: VALU instructions share the issue port with the
  // MFMAs, and a handful per step cost the fp32 kernel 4-6 %.
  const int lrow = lane / VPR, pc = lane % VPR;
  unsigned offa[NIA], offb[NIB];
#pragma unroll
  for (int j = 0; j < NIA; ++j) {
    const int row = (j * NW + wave) * RPI + lrow;
    offa[j] = 2u * ((unsigned)row * (unsigned)p.lda + (unsigned)(pc ^ swz(row)) * 8u);
  }
#pragma unroll
  for (int j = 0; j < NIB; ++j) {
    const int row = (j * NW + wave) * RPI + lrow;
    offb[j] = 2u * ((unsigned)row * (unsigned)p.ldb + (unsigned)(pc ^ swz(row)) * 8u);
  }
  const u16* a_base = p.A + (size_t)blockIdx.z * p.batchA + (size_t)m0 * p.lda;
  const u16* b_base = p.B + (size_t)blockIdx.z * p.batchB + (size_t)n0 * p.ldb;
  // The loads of a tile are issued in two halves, A right after the barrier that frees the buffer
  // and B one chunk later: the LDS takes tile loads and fragment reads at the same time, and 64 KB
  // arriving in one burst get in the way of the reads more than two bursts of 32 KB (measured 1 %).
  auto issue_a = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NIA; ++j)
      load_to_lds(a_base, offa[j], lds_base + 2u * (unsigned)(buf * A_ELEMS + (j * NW + wave) * RPI * STRIDE));
    a_base += BK;
  };
  auto issue_b = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NIB; ++j)
      load_to_lds(b_base, offb[j], lds_base + 2u * (unsigned)(STAGES * A_ELEMS + buf * B_ELEMS + (j * NW + wave) * RPI * STRIDE));
    b_base += BK;
  };
  auto issue = [&](int buf) __attribute__((always_inline)) {
    issue_a(buf);
    issue_b(buf);
  };
  // LDS byte addresses of this lane's fragments for each 16-wide K chunk of a step (block 0 of
  // the wavefront, ring buffer 0).  swz(row) is the same for all 32 x 32 blocks of a wavefront
  // (they are 32 rows apart), so the other blocks and buffers are immediate offsets from these.
  // The empty asm keeps the compiler from re-deriving them with vector adds inside the K loop.
  static_assert(32 % (ROWS_PER_LINE * VPR) == 0, "the swizzle must repeat every 32 rows");
  unsigned a_addr[CH], b_addr[CH];
#pragma unroll
  for (int kk = 0; kk < CH; ++kk) {
    const int ra = wm0 + l32, rb = wn0 + l32;
    a_addr[kk] = lds_base + 2u * (unsigned)(ra * STRIDE + ((kk * 2 + hi) ^ swz(ra)) * 8);
    b_addr[kk] = lds_base + 2u * (unsigned)(STAGES * A_ELEMS + rb * STRIDE + ((kk * 2 + hi) ^ swz(rb)) * 8);
    asm volatile("" : "+v"(a_addr[kk]), "+v"(b_addr[kk]));
  }
  typedef __attribute__((address_space(3))) const bf16x8 lds_frag;
  auto load_frags = [&](bf16x8 (&fa)[TM], bf16x8 (&fb)[TN], int buf, int kk) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[i] = *reinterpret_cast<lds_frag*>((__attribute__((address_space(3))) const char*)(size_t)(
          a_addr[kk] + 2u * (unsigned)(buf * A_ELEMS + i * 32 * STRIDE)));
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[j] = *reinterpret_cast<lds_frag*>((__attribute__((address_space(3))) const char*)(size_t)(
          b_addr[kk] + 2u * (unsigned)(buf * B_ELEMS + j * 32 * STRIDE)));
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int nk = p.K / BK;
  bf16x8 fa[2][TM], fb[2][TN];
  // PRIO = 1: a wavefront raises its issue priority for the MFMAs of a chunk and drops it for the
  // fragment reads and tile loads in between.  The two wavefronts of a SIMD then fall into
  // alternation (one multiplies while the other fetches) instead of competing for the MFMA pipe
  // with half-issued chunks: 3-3.5 % on the two-buffer BK = 64 kernel, nothing on the BK = 32 ring
  // and a small loss on the fp32 kernel, which therefore keep equal priorities.
  auto multiply = [&](int fc) __attribute__((always_inline)) {
    if (PRIO == 1) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[fc][i], fb[fc][j], acc[i][j], 0, 0, 0);
    if (PRIO == 1) __builtin_amdgcn_s_setprio(0);
  };
  if constexpr (STAGES == 2) {
    // Two buffers (what fits when BK = 64 makes a 256 x 256 tile 64 KB).  BK = 64 rows are whole
    // 128-byte lines, which the load path moves markedly faster than the half lines of BK = 32.
    // Step t multiplies buffer t % 2.  Before its last chunk every wavefront has issued all its
    // reads of that buffer; it waits for them and for tile t+1 (the other buffer), then the
    // barrier, then tile t+2 is requested into the buffer just read out and has a whole step to
    // land.  The first fragments of tile t+1 are fetched during the last chunk's MFMAs, so no
    // step starts with an empty MFMA pipe.
    if (nk > 0) issue(0);
    if (nk > 1) {
      issue(1);
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(INSTR));
    } else {
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    }
    ring_barrier();
    load_frags(fa[0], fb[0], 0, 0);
    // ring positions are compile-time constants (loop unrolled over the two buffers): every LDS
    // address is a register plus an immediate
    auto step2 = [&](int t, auto cur_c, auto steady_c) __attribute__((always_inline)) {
      constexpr int cur = decltype(cur_c)::value;
      constexpr bool steady = decltype(steady_c)::value;  // tile t+2 exists
#pragma unroll
      for (int kk = 0; kk < CH; ++kk) {
        const int fc = kk & 1, fn = fc ^ 1;
        if (kk + 1 < CH) load_frags(fa[fn], fb[fn], cur, kk + 1);
        else load_frags(fa[fn], fb[fn], cur ^ 1, 0);  // after the last tile: a harmless read of ring memory
        // The last reads of this buffer must have returned at the barrier below: issue them before
        // this chunk's MFMAs, not (as the scheduler would) right in front of the wait.
        if (kk == CH - 2) __builtin_amdgcn_sched_barrier(0);
        multiply(fc);
        if (kk == CH - 2) {
          // keeps this chunk's MFMAs above the barrier (it does not order register-only
          // instructions, and an MFMA pipe that is empty at the barrier is lost time)
          __builtin_amdgcn_sched_barrier(0);
          __builtin_amdgcn_s_waitcnt(vmcnt_imm(0) & 0xc07f);  // vmcnt(0) and lgkmcnt(0)
          ring_barrier();
          if (steady || t + 2 < nk) issue_a(cur);
        }
        if (kk == CH - 1) {
          if (steady || t + 2 < nk) issue_b(cur);
        }
      }
    };
    int t = 0;
    for (; t + 4 <= nk; t += 2) {
      step2(t, std::integral_constant<int, 0>{}, std::true_type{});
      step2(t + 1, std::integral_constant<int, 1>{}, std::true_type{});
    }
    static_for_h<3>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      if (t + s < nk) step2(t + s, std::integral_constant<int, s % 2>{}, std::false_type{});
    });
  } else {
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
      if (s < nk) issue(s);
    if (nk >= STAGES - 1) __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * INSTR));
    else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    ring_barrier();

    load_frags(fa[0], fb[0], 0, 0);
    auto step = [&](int t, auto cur_c, auto steady_c) __attribute__((always_inline)) {
      constexpr int cur = decltype(cur_c)::value;
      constexpr bool steady = decltype(steady_c)::value;  // tiles t+1 .. t+STAGES-1 all exist
      constexpr int nxt = cur + 1 == STAGES ? 0 : cur + 1;
      constexpr int fill = cur == 0 ? STAGES - 1 : cur - 1;
#pragma unroll
      for (int kk = 0; kk < CH; ++kk) {
        const int fc = kk & 1, fn = fc ^ 1;
        if (kk + 1 < CH) load_frags(fa[fn], fb[fn], cur, kk + 1);
        else load_frags(fa[fn], fb[fn], nxt, 0);  // after the last tile: a harmless read of ring memory, keeps one code path
        multiply(fc);
        if (kk == CH - 2) {
          __builtin_amdgcn_sched_barrier(0);  // this chunk's MFMAs stay above the barrier
          // tiles t+1 .. t+STAGES-2 are in flight; tile t+1 must have landed
          if (steady || t + STAGES - 2 < nk) __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 3) * INSTR));
          else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
          ring_barrier();
          if (steady || t + STAGES - 1 < nk) issue_a(fill);
        }
        if (kk == CH - 1) {
          if (steady || t + STAGES - 1 < nk) issue_b(fill);
        }
      }
    };
    int t = 0;
    for (; t + 2 * STAGES - 1 <= nk; t += STAGES)
      static_for_h<STAGES>([&](auto sc) { step(t + decltype(sc)::value, sc, std::true_type{}); });
    static_for_h<2 * STAGES - 2>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      if (t + s < nk) step(t + s, std::integral_constant<int, s % STAGES>{}, std::false_type{});
    });
  }
  u16* stage = nullptr;
  const u16* mask_lds = nullptr;
  bool synced = false;
  if constexpr (EPI == EPH_MASK) {
    // The ReLU mask is read at the output position: 2 bytes per lane and element straight from
    // global memory are 64-byte pieces (measured +300 us on a 1.9 ms GEMM).  Bring the tile's
    // mask into the idle LDS with direct loads (two 512-byte rows per instruction) instead.
    constexpr int MASK_UNITS = BM * BN / 512;  // 1 KB pieces
    static_assert((size_t)BM * BN <= STAGES * (size_t)(BM + BN) * BK, "the mask tile must fit the ring");
    static_assert(BN * 2 % 16 == 0 && 1024 % (BN * 2) == 0 && MASK_UNITS % NW == 0, "mask tile shape");
    if (p.ldmask % 8 == 0 && (reinterpret_cast<uintptr_t>(p.mask) & 15) == 0) {  // uniform
      __syncthreads();  // every wavefront is done with the operand tiles
      synced = true;
      constexpr int CPR = BN / 8, RPU = 64 / CPR;  // 16-byte chunks per mask row, rows per piece
#pragma unroll
      for (int u = 0; u < MASK_UNITS / NW; ++u) {
        const int unit = u * NW + wave;
        const int row = unit * RPU + lane / CPR, c = lane % CPR;
        load_to_lds(p.mask + (size_t)m0 * p.ldmask + n0, 2u * ((unsigned)row * (unsigned)p.ldmask + (unsigned)c * 8u),
                    lds_base + 1024u * (unsigned)unit);
      }
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
      __syncthreads();
      mask_lds = smem_h;
    }
  }
  if (EPI != EPH_F32 && p.Ct) {
    // every wavefront is done with the operand tiles (and all direct loads have landed): the LDS
    // is free for the staging of the transposed output, one private region per wavefront
    constexpr int REGION = 32 * (TM * 64 + 8);
    static_assert((size_t)NW * REGION <= STAGES * (size_t)(BM + BN) * BK * sizeof(u16), "staging must fit the ring");
    if (!synced) __syncthreads();
    stage = smem_h + (size_t)wave * (REGION / 2);
  }
  if (mask_lds) store_tile_h<TM, TN, EPI, true>(p, acc, m0 + wm0, n0 + wn0, l32, hi, stage, mask_lds, BN, wm0, wn0);
  else store_tile_h<TM, TN, EPI, false>(p, acc, m0 + wm0, n0 + wn0, l32, hi, stage, nullptr, BN, wm0, wn0);
}

// Fallback for an empty contraction (K = 0) and for forced variants that do not fit: one thread per
// output element, fp32 accumulation in k order.
template <int EPI>
__global__ __launch_bounds__(256) void gemm_bf16_generic(HGemmArgs p) {
  const int col = blockIdx.x * 16 + (threadIdx.x & 15), row = blockIdx.y * 16 + (threadIdx.x >> 4);
  if (row >= p.M || col >= p.N) return;
  const u16* a = p.A + (size_t)blockIdx.z * p.batchA + (size_t)row * p.lda;
  const u16* b = p.B + (size_t)blockIdx.z * p.batchB + (size_t)col * p.ldb;
  float v = 0.0f;
  for (int k = 0; k < p.K; ++k) v = fmaf(bf2f(a[k]), bf2f(b[k]), v);
  if (EPI == EPH_F32) {
    (reinterpret_cast<float*>(p.C) + (size_t)blockIdx.z * p.batchC)[(size_t)row * p.ldc + col] = v;
    return;
  }
  if (EPI == EPH_BIAS_RELU) {
    if (p.bias) v += p.bias[col];
    if (p.relu) v = v > 0.0f ? v : 0.0f;
  } else if (EPI == EPH_MASK) {
    if (!(bf2f(p.mask[(size_t)row * p.ldmask + col]) > 0.0f)) v = 0.0f;
  }
  (reinterpret_cast<u16*>(p.C) + (size_t)blockIdx.z * p.batchC)[(size_t)row * p.ldc + col] = f2bf(v);
}

template <int BM, int BN, int BK, int WM, int WN, int EPI, int PF = 1, int STAGES = 3, bool GUARD = false>
static hipError_t launch_h(HGemmArgs& p, int batch, hipStream_t s) {
  constexpr size_t lds_bytes = STAGES * (size_t)(BM + BN) * BK * sizeof(u16);
  static_assert(lds_bytes <= 160 * 1024, "tile does not fit the 160 KB of LDS");
  auto kern = gemm_bf16_mfma<BM, BN, BK, WM, WN, EPI, PF, STAGES, GUARD>;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) return e;
  p.tiles_m = GUARD ? (p.M + BM - 1) / BM : p.M / BM;
  p.tiles_n = GUARD ? (p.N + BN - 1) / BN : p.N / BN;
  launch_kernel(kern, dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(WM * WN * 64), lds_bytes, s, p);
  return hipGetLastError();
}

template <int BM, int BN, int BK, int WM, int WN, int EPI, int STAGES, int PRIO = 0>
static hipError_t launch_dma(HGemmArgs& p, int batch, hipStream_t s) {
  constexpr size_t lds_bytes = STAGES * (size_t)(BM + BN) * BK * sizeof(u16);
  static_assert(lds_bytes <= 160 * 1024, "tile does not fit the 160 KB of LDS");
  auto kern = gemm_bf16_dma<BM, BN, BK, WM, WN, EPI, STAGES, PRIO>;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), lds_bytes); e != hipSuccess) return e;
  p.tiles_m = p.M / BM;
  p.tiles_n = p.N / BN;
  launch_kernel(kern, dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(WM * WN * 64), lds_bytes, s, p);
  return hipGetLastError();
}

template <int EPI>
static hipError_t dispatch_h(HGemmArgs& p, int batch, hipStream_t s, int variant, bool* wrote_ct, bool* wrote_colsum) {
  if (wrote_ct) *wrote_ct = p.Ct != nullptr && EPI != EPH_F32;
  if (p.M <= 0 || p.N <= 0 || batch <= 0) return hipSuccess;
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec_ok = al16(p.A) && al16(p.B) && p.lda % 8 == 0 && p.ldb % 8 == 0 && p.batchA % 8 == 0 &&
                      p.batchB % 8 == 0 && p.K > 0;
  // the transposed second output needs whole tiles inside one row group and 16-byte aligned stores
  const bool want_ct = p.Ct != nullptr;
  auto ct_ok = [&](int bm) {
    return !want_ct || (p.ct_rows % bm == 0 && p.ct_rows % 8 == 0 && al16(p.Ct) && batch == 1);
  };
  auto fits = [&](int bm, int bn, int bk) { return vec_ok && p.M % bm == 0 && p.N % bn == 0 && p.K % bk == 0; };
  if (variant == 0 && hgemm_is_skinny(p.M, p.N, p.K)) {
    // a layer of at most SKINNY_MAX outputs is matrix-vector work (forward: N, weight gradient: M,
    // input gradient: K); the caller makes the transposed copy and the bias gradient by itself
    if (wrote_ct) *wrote_ct = false;
    if (wrote_colsum) *wrote_colsum = false;
    p.Ct = nullptr;
    p.colsum_part = nullptr;
    return launch_skinny(p, batch, EPI, s);
  }
  if (variant == 0) {
    // 256 x 256 tiles with 8 wavefronts and direct-to-LDS loads (whole 128-byte lines per row when
    // K allows BK = 64) from somewhat more than half a round of the 256 CUs on, else 128 x 128 tiles
    // with direct loads, two workgroups per CU: with more than one tile per CU eight wavefronts on
    // two buffers of BK = 64 (variant 18), else four wavefronts on a ring of four of BK = 32
    // (variant 17).  One box, forward entry point, us per launch with 256 x 256 x 64 / variant 18 /
    // variant 17 / 128 x 128 x 32 through registers (variant 3), number of 256 x 256 tiles in brackets:
    //   8192 x 1536 x 1536 (192) 45.7 / 48.0 / 60.1 / 68.4    6144 x 2048 x 1024 (192) 31.8 / 32.4 / 37.2 / -
    //   4096 x 2048 x 2048 (128) 50.1 / 38.6 / 50.5 / 47.9    4096 x 2048 x  512 (128) 19.5 / 13.2 / 14.9 / -
    //   3072 x 2048 x 2048  (96) 45.6 / 32.2 / 40.7 / -       4096 x 1536 x 1536  (96) 37.2 / 25.0 / 32.9 / -
    //   2048 x 2048 x 2048  (64) 43.5 / 25.0 / 23.0 / 33.4    4096 x 1024 x 4096  (64) 77.1 / 48.6 / 46.4 / 64.4
    //   4096 x 1024 x 1024  (64) 25.4 / 12.1 / 12.3 / 16.5    2048 x 1024 x 1024  (32) 24.2 / 10.0 / 10.2 / 15.1
    const long long t256 = (long long)(p.M / 256) * (p.N / 256) * batch;
    const long long t128 = (long long)(p.M / 128) * (p.N / 128) * batch;
    // The 256 x 256 kernel: four wavefronts of 128 x 128 with the hand-ordered K step (variant 32),
    // 3-4 % faster than eight wavefronts of 128 x 64 (variant 27).  Both leave registers free for a
    // wavefront of the update kernel that the step launches beside a GEMM (76 registers, 16 KB of LDS:
    // the eight-wavefront kernel takes 2 x 206-211 of a SIMD's 512, this one 372-396 since its
    // epilogue reads the accumulators out of the AGPRs row block by row block), so the two share CUs
    // instead of taking them in turns.
    if (fits(256, 256, 64) && t256 >= 144) variant = 32;  // falls back to 19 below if C or the mask is not 16-byte aligned
    else if (fits(256, 256, 32) && t256 >= 256) variant = 13;
    else if (fits(128, 128, 64) && t128 > 256) variant = 18;
    else if (fits(128, 128, 32) && t128 >= 128) variant = 17;
    else if (fits(64, 64, 32)) variant = 5;
    else if (p.K > 0)  // ragged shape or unaligned storage: the guarded MFMA instances
      variant = (long long)((p.M + 127) / 128) * ((p.N + 127) / 128) * batch >= 192 ? 21 : 22;
    else variant = -1;
  }
  // the 16x16x32 kernel writes C and reads the mask in 16-byte pieces
  auto x32_ok = [&]() {
    const int per16 = EPI == EPH_F32 ? 4 : 8;
    return fits(256, 256, 64) && al16(p.C) && p.ldc % per16 == 0 && p.batchC % per16 == 0 &&
           (EPI != EPH_MASK || (al16(p.mask) && p.ldmask % 8 == 0)) &&
           (EPI != EPH_F32 || (long long)p.M * p.ldc * 4 < (1ll << 32));  // fp32 stores: 32-bit byte offsets within an entry
  };
  // Variants of the 16x16x32 kernel: 27 = raised wave priority around the MFMAs (the automatic
  // choice), 28 = without it; 29 / 30 = 27 with all / pairs of the batch entries of an fp32-result
  // GEMM (the replicas of a weight gradient) chained in one workgroup.  Chaining is not chosen
  // automatically: on four replicas of 8192 x 8192 x 4096 one workgroup per replica and tile takes
  // 1.63 ms, pairs 1.65 ms, all four in one workgroup 1.73 ms -- the tile stores of an entry have
  // one K step to drain before the next wait has to see them gone (the counter retires loads and
  // stores in order), the wavefronts stall there for longer than a workgroup turnover costs.
  const bool x32 = (variant >= 27 && variant <= 30) || variant == 32;
  if (x32 && !x32_ok()) variant = 19;
  p.chain = 1;
  if (EPI == EPH_F32 && batch > 1) {
    if (variant == 29) p.chain = batch;
    else if (variant == 30 && batch % 2 == 0) p.chain = 2;
  }
  p.vec_a = al16(p.A) && p.lda % 8 == 0 && p.batchA % 8 == 0;
  p.vec_b = al16(p.B) && p.ldb % 8 == 0 && p.batchB % 8 == 0;
  // column-sum partials come from the 256 x 256 direct-load kernels (wavefront tiles of 128 rows) only
  if (p.colsum_part && !((variant == 13 || variant == 19 || variant == 25 || (variant >= 27 && variant <= 30) || variant == 32) && EPI != EPH_F32 && batch == 1 && p.M % 128 == 0)) p.colsum_part = nullptr;
  if (wrote_colsum) *wrote_colsum = p.colsum_part != nullptr;
  {  // the tile height decides whether the transposed output is possible; if not, drop it
    const int bm = (variant == 3 || variant == 17 || variant == 18) ? 128 : variant == 5 ? 64 : 256;  // (variants 13, 19, 25, 27 .. 30: 256)
    if (want_ct && (EPI == EPH_F32 || variant == 21 || variant == 22 || !ct_ok(bm))) {
      p.Ct = nullptr;
      if (wrote_ct) *wrote_ct = false;
    }
  }
  switch (variant) {
    case 3: if (fits(128, 128, 32)) return launch_h<128, 128, 32, 2, 2, EPI>(p, batch, s); break;
    case 4: if (fits(256, 256, 32)) return launch_h<256, 256, 32, 2, 4, EPI>(p, batch, s); break;
    case 5: if (fits(64, 64, 32)) return launch_h<64, 64, 32, 2, 2, EPI>(p, batch, s); break;
    case 13: if (fits(256, 256, 32)) return launch_dma<256, 256, 32, 2, 4, EPI, 4>(p, batch, s); break;
    case 17: if (fits(128, 128, 32)) return launch_dma<128, 128, 32, 2, 2, EPI, 4>(p, batch, s); break;
    case 18: if (fits(128, 128, 64)) return launch_dma<128, 128, 64, 2, 4, EPI, 2, 1>(p, batch, s); break;
    case 19: if (fits(256, 256, 64)) return launch_dma<256, 256, 64, 2, 4, EPI, 2, 1>(p, batch, s); break;
    case 25: if (fits(256, 256, 64)) return launch_dma<256, 256, 64, 2, 4, EPI, 2, 0>(p, batch, s); break;
    case 27: case 29: case 30: return launch_x32(p, batch, EPI, true, s);
    case 28: return launch_x32(p, batch, EPI, false, s);
    case 32: return launch_x32w4(p, batch, EPI, s);
    case 21: if (p.K > 0) return launch_h<128, 128, 32, 2, 2, EPI, 1, 3, true>(p, batch, s); break;
    case 22: if (p.K > 0) return launch_h<64, 64, 32, 2, 2, EPI, 1, 3, true>(p, batch, s); break;
    default: break;
  }
  if (wrote_ct) *wrote_ct = false;  // the any-shape kernel has no transposed output
  if (wrote_colsum) *wrote_colsum = false;
  p.Ct = nullptr;
  p.colsum_part = nullptr;
  launch_kernel((gemm_bf16_generic<EPI>), dim3((p.N + 15) / 16, (p.M + 15) / 16, batch), dim3(256), 0, s, p);
  return hipGetLastError();
}

// C = A[M,K] * B[N,K]^T, both bf16 and K-contiguous.  out_kind: 0 fp32 plain, 1 bf16 bias+ReLU,
// 2 bf16 masked, 3 bf16 plain.
hipError_t hgemm_nt(int batch, int M, int N, int K, const uint16_t* A, int lda, long long batchA, const uint16_t* B,
                    int ldb, long long batchB, void* C, int ldc, long long batchC, int out_kind, const float* bias,
                    int relu, const uint16_t* mask, int ldmask, hipStream_t s, int variant, uint16_t* Ct, int ct_rows,
                    bool* wrote_ct, float* colsum_part, bool* wrote_colsum) {
  HGemmArgs p{};
  p.Ct = Ct; p.ct_rows = ct_rows;
  p.colsum_part = colsum_part;
  p.M = M; p.N = N; p.K = K; p.A = A; p.B = B; p.C = C; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
  p.batchA = batchA; p.batchB = batchB; p.batchC = batchC;
  p.bias = bias; p.relu = relu; p.mask = mask; p.ldmask = ldmask;
  switch (out_kind) {
    case 0: return dispatch_h<EPH_F32>(p, batch, s, variant, wrote_ct, wrote_colsum);
    case 1: return dispatch_h<EPH_BIAS_RELU>(p, batch, s, variant, wrote_ct, wrote_colsum);
    case 2: return dispatch_h<EPH_MASK>(p, batch, s, variant, wrote_ct, wrote_colsum);
    default: return dispatch_h<EPH_BF16>(p, batch, s, variant, wrote_ct, wrote_colsum);
  }
}

// ---- bias gradient from the column-sum partials of the GEMM that produced dZ ------------------------
// out[r * stride_out + c] = sum over the `blocks` row blocks of replica r of part[(r * blocks + q) * N + c],
// in block order (deterministic).
__global__ __launch_bounds__(256) void colsum_fold_kernel(float* __restrict__ out, long long stride_out,
                                                          const float* __restrict__ part, int N, int blocks) {
  const int c = blockIdx.x * 256 + threadIdx.x, r = blockIdx.y;
  if (c >= N) return;
  const float* q = part + (size_t)r * blocks * N + c;
  float v = 0.0f;
  for (int b = 0; b < blocks; ++b) v += q[(size_t)b * N];
  out[(size_t)r * stride_out + c] = v;
}

hipError_t colsum_fold(int R, int N, int blocks_per_replica, const float* part, float* out, long long stride_out,
                       hipStream_t s) {
  if (R <= 0 || N <= 0) return hipSuccess;
  launch_kernel(colsum_fold_kernel, dim3((N + 255) / 256, R), dim3(256), 0, s, out, stride_out, part, N, blocks_per_replica);
  return hipGetLastError();
}

// ---- batched transpose: dst[z][c][r] = src[z][r][c], 16-bit elements, 64 x 64 tiles through LDS ----
// VEC = true (tile-aligned shapes, 16-byte aligned rows on both sides): a thread moves 8 elements
// with one 16-byte access on either side of the LDS tile; else element by element with bounds
// checks.
template <bool VEC>
__global__ __launch_bounds__(256) void transpose16_kernel(u16* __restrict__ dst, const u16* __restrict__ src, int rows,
                                                          int cols, int ld_src, int ld_dst, long long batch_src,
                                                          long long batch_dst) {
  __shared__ __attribute__((aligned(16))) u16 tile[64][72];  // 144-byte rows: 16-byte aligned, odd multiple of 16
  const u16* s = src + (size_t)blockIdx.z * batch_src;
  u16* d = dst + (size_t)blockIdx.z * batch_dst;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  if (VEC) {
    const int part = threadIdx.x & 7, line = threadIdx.x >> 3;  // 8 threads per 64-element row, 32 rows per pass
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = line + 32 * i;
      *reinterpret_cast<u32x4*>(&tile[r][part * 8]) =
          *reinterpret_cast<const u32x4*>(s + (size_t)(r0 + r) * ld_src + c0 + part * 8);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int c = line + 32 * i;  // output row = input column
      u16 e[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) e[k] = tile[part * 8 + k][c];
      const u32x4 v = {(unsigned)e[0] | ((unsigned)e[1] << 16), (unsigned)e[2] | ((unsigned)e[3] << 16),
                       (unsigned)e[4] | ((unsigned)e[5] << 16), (unsigned)e[6] | ((unsigned)e[7] << 16)};
      *reinterpret_cast<u32x4*>(d + (size_t)(c0 + c) * ld_dst + r0 + part * 8) = v;
    }
    return;
  }
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    tile[i][tx] = (r < rows && c < cols) ? s[(size_t)r * ld_src + c] : (u16)0;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int c = c0 + i, r = r0 + tx;
    if (c < cols && r < rows) d[(size_t)c * ld_dst + r] = tile[tx][i];
  }
}

hipError_t transpose_bf16(int batch, int rows, int cols, const uint16_t* src, int ld_src, long long batch_src,
                          uint16_t* dst, int ld_dst, long long batch_dst, hipStream_t s) {
  if (batch <= 0 || rows <= 0 || cols <= 0) return hipSuccess;
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
  const bool vec = rows % 64 == 0 && cols % 64 == 0 && ld_src % 8 == 0 && ld_dst % 8 == 0 && batch_src % 8 == 0 &&
                   batch_dst % 8 == 0 && al16(src) && al16(dst);
  const dim3 grid((cols + 63) / 64, (rows + 63) / 64, batch);
  if (vec) launch_kernel(transpose16_kernel<true>, grid, dim3(256), 0, s, dst, src, rows, cols, ld_src, ld_dst, batch_src, batch_dst);
  else launch_kernel(transpose16_kernel<false>, grid, dim3(256), 0, s, dst, src, rows, cols, ld_src, ld_dst, batch_src, batch_dst);
  return hipGetLastError();
}

// ---- row sums of a bf16 matrix in fp32: out[z*stride_out + r] = sum_c src[z][r][c] -------------------
// One wavefront per row.  VEC = true (cols a multiple of 8, 16-byte aligned rows): a lane adds up
// 8 consecutive elements per 16-byte load in element order, lanes stride over the row; else one
// element per load.  Fixed-order tree over the lanes at the end.
template <bool VEC>
__global__ __launch_bounds__(256) void rowsum16_kernel(float* __restrict__ out, const u16* __restrict__ src, int rows,
                                                       int cols, int ld, long long batch_src, long long stride_out) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const u16* s = src + (size_t)blockIdx.y * batch_src + (size_t)row * ld;
  float v = 0.0f;
  if (VEC) {
    // four loads in flight per lane; the additions keep the element order of the plain loop
    for (int c = lane * 8; c < cols; c += 4 * 512) {
      u32x4 t[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (c + u * 512 < cols) t[u] = *reinterpret_cast<const u32x4*>(s + c + u * 512);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (c + u * 512 >= cols) break;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          v += __uint_as_float(t[u][k] << 16);
          v += __uint_as_float(t[u][k] & 0xffff0000u);
        }
      }
    }
  } else {
    for (int c = lane; c < cols; c += 64) v += bf2f(s[c]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  if (lane == 0) out[(size_t)blockIdx.y * stride_out + row] = v;
}

hipError_t rowsum_bf16(int batch, int rows, int cols, const uint16_t* src, int ld, long long batch_src, float* out,
                       long long stride_out, hipStream_t s) {
  if (batch <= 0 || rows <= 0) return hipSuccess;
  const bool vec = cols % 8 == 0 && ld % 8 == 0 && batch_src % 8 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0;
  if (vec) launch_kernel(rowsum16_kernel<true>, dim3((rows + 3) / 4, batch), dim3(256), 0, s, out, src, rows, cols, ld, batch_src, stride_out);
  else launch_kernel(rowsum16_kernel<false>, dim3((rows + 3) / 4, batch), dim3(256), 0, s, out, src, rows, cols, ld, batch_src, stride_out);
  return hipGetLastError();
}

}  // namespace mi
