// Shared pieces of the bf16 GEMM kernels: argument block, epilogue kinds, the workgroup -> tile
// mapping, the direct global -> LDS load and the small helpers of the LDS ring.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>
#include <utility>

#include "kernels.h"

namespace mi {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short u16;

enum EpilogueH { EPH_F32 = 0, EPH_BIAS_RELU = 1, EPH_MASK = 2, EPH_BF16 = 3 };

struct HGemmArgs {
  int M, N, K;
  const u16* A;
  const u16* B;
  void* C;  // bf16 or fp32, see the epilogue
  int lda, ldb, ldc;
  long long batchA, batchB, batchC;  // element offsets per blockIdx.z
  const float* bias;
  int relu;
  const u16* mask;  // bf16 [M x N]: result zeroed where mask <= 0
  int ldmask;
  int tiles_m, tiles_n;
  // optional second output (bf16 epilogues): the same values transposed per group of ct_rows
  // rows, Ct[(row / ct_rows)][col][row % ct_rows] with row stride ct_rows and N * ct_rows elements
  // per group -- the K-contiguous per-replica copy the weight-gradient GEMM reads
  u16* Ct;
  int ct_rows;
  // guarded instances: whether A / B may be read with 16-byte vector loads
  int vec_a, vec_b;
  // optional third output (bf16 epilogues of the 256 x 256 kernels): column sums of the values
  // written, per wavefront tile of 128 rows -- colsum_part[row / 128][col], N floats per row block.
  // Folded over a replica's row blocks they are the bias gradient of the layer whose dZ this GEMM
  // produces, which saves a separate pass over that dZ.
  float* colsum_part;
  // fp32 results of the 16x16x32 kernel: consecutive batch entries one workgroup walks as one K loop
  // (0 or 1: one workgroup per entry and tile)
  int chain;
};

__device__ __forceinline__ u16 f2bf(float f) {
  unsigned int u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u16)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (u16)(u >> 16);
}
__device__ __forceinline__ float bf2f(u16 h) { return __uint_as_float((unsigned int)h << 16); }

__device__ __forceinline__ void lds_barrier_h() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Maps the flat workgroup index to a C tile.  Workgroups are handed to the 8 XCDs round-robin
// (id % 8), each XCD has a private 4 MB L2, and about 32 workgroups (one per CU) of an XCD run at
// the same time.
//   * Large grids (tile counts divisible as needed): the grid is cut into super-tiles of 4 x 8
//     tiles; XCD x owns super-tiles x, x+8, ... and walks each row by row, so the 32 tiles it
//     runs together share 4 A panels and 8 B panels -- 12 panel slices per K step from the
//     fabric instead of the 33 a single tile row needs.
//   * Otherwise, if the tile count is a multiple of 8: XCD x gets the contiguous range
//     [x*T/8, (x+1)*T/8) of the row-major order (tiles of one row share their A panel).
//   * Otherwise the identity.
__device__ __forceinline__ void tile_of_workgroup(int id, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  if ((tiles_m & 3) == 0 && (tiles_n & 7) == 0 && (total & 255) == 0) {
    const int xcd = id & 7, j = id >> 3;
    const int super = (j >> 5) * 8 + xcd, within = j & 31;
    const int super_cols = tiles_n >> 3;
    tm = (super / super_cols) * 4 + (within >> 3);
    tn = (super % super_cols) * 8 + (within & 7);
    return;
  }
  if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
  tm = id / tiles_n;
  tn = id - tm * tiles_n;
}

// Direct global -> LDS load of 16 bytes per lane (global_load_lds_dwordx4): the 64 lanes fill 1 KB
// of consecutive LDS bytes from the wave-uniform address in m0, each lane names its own global
// address (uniform base + 32-bit byte offset).  Inline assembly on purpose: the compiler models
// the builtin as a FLAT access and then waits lgkmcnt(0) before every later LDS read; written this
// way it does not track the load and the kernels wait on vmcnt themselves.
__device__ __forceinline__ void load_to_lds(const u16* uniform_base, unsigned lane_byte_offset, unsigned lds_byte_addr) {
  const unsigned lds_addr = __builtin_amdgcn_readfirstlane(lds_byte_addr);
  const unsigned long long b = reinterpret_cast<unsigned long long>(uniform_base);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b), hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  const unsigned long long sbase = ((unsigned long long)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(lane_byte_offset), "s"(sbase)
               : "memory", "m0");
}

// The same for callers whose LDS address is wave-uniform by construction (derived from values
// that went through readfirstlane once): taking it as a scalar operand directly keeps the compiler
// from parking one copy per load instruction in vector registers for a readfirstlane of its own.
__device__ __forceinline__ void load_to_lds_uniform(const u16* uniform_base, unsigned lane_byte_offset,
                                                    unsigned uniform_lds_byte_addr) {
  const unsigned long long b = reinterpret_cast<unsigned long long>(uniform_base);
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b), hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
  const unsigned long long sbase = ((unsigned long long)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(uniform_lds_byte_addr), "v"(lane_byte_offset), "s"(sbase)
               : "memory", "m0");
}

template <int... S, class F>
__device__ __forceinline__ void static_for_h_impl(std::integer_sequence<int, S...>, F&& f) {
  (f(std::integral_constant<int, S>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for_h(F&& f) {
  static_for_h_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14,
// expcnt 6:4, lgkmcnt 11:8; the other counters at their maximum = no wait).
constexpr int vmcnt_imm(int n) { return (n & 15) | ((n >> 4) << 14) | 0x70 | 0xf00; }

// Barrier of the ring: no LDS-counter wait is attached (nothing was written with ds_write, and a
// buffer is refilled only after the MFMAs that consumed its last fragments, i.e. after those reads
// returned); the empty asm statements keep the compiler from moving LDS reads across it.
__device__ __forceinline__ void ring_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Launches the 256 x 256 x 64 kernel built on v_mfma_f32_16x16x32_bf16 (gemm_bf16_x32.hip); the
// caller has checked the shape and alignment rules listed there.  epi: an EpilogueH value.
hipError_t launch_x32(HGemmArgs& p, int batch, int epi, bool prio, hipStream_t s);
// The same tile with four wavefronts of 128 x 128 and a hand-ordered K step (same rules; no chained entries).
hipError_t launch_x32w4(HGemmArgs& p, int batch, int epi, hipStream_t s);

// gemv_bf16.hip: the same product when M, N or K is at most SKINNY_MAX, as matrix-vector passes
// (any alignment, any epilogue; no transposed second output, no column-sum partials).
bool hgemm_is_skinny(int M, int N, int K);
hipError_t launch_skinny(HGemmArgs& p, int batch, int epi, hipStream_t s);

}  // namespace mi
