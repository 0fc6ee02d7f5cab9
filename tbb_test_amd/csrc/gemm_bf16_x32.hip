// bf16 GEMM for gfx950 on v_mfma_f32_16x16x32_bf16: C[M,N] = A[M,K] * B[N,K]^T, both operands
// K-contiguous, fp32 accumulation -- the kernel of the large GEMMs of the MLP step (reference call
// sites mlp_omp.cc:474-488, 565-580, 657-671).
//
// Why this instruction.  The bf16 matrix cores of this device are power-limited: a register-resident
// loop of 32x32x16 MFMAs sustains about 1 800 TFLOP/s on random operands, the same loop of 16x16x32
// MFMAs about 2 050 (a 16 x 16 block accumulates 32 k per instruction: half the accumulator traffic
// per flop).  The clock the GEMM runs at follows.
//
// Tile 256 x 256 x 64, eight wavefronts of 128 (m) x 64 (n), two LDS buffers filled by direct
// global -> LDS loads, one barrier per K step: the ring of gemm_bf16_dma (gemm_bf16.hip) with other
// fragments.  A step is four sub-chunks of 16 MFMAs: K chunk kc = 0, 1 (32 k each) times the lower
// and upper four 16-row blocks of the wavefront's m range; the n-side fragments of a K chunk stay
// in registers for both halves.
//
// Orientation.  The MFMA's register-side index (row 4 * (lane / 16) + r of the 16 x 16 result) is
// given to n and its lane-side index (lane % 16) to m, and the rows of the B tile are dealt to the
// four n blocks so that a lane ends up with two runs of eight consecutive columns of one row of C
// (columns 8q .. 8q+7 and 32 + 8q .. 32 + 8q+7 of the wavefront's 64, q = lane / 16):
//   block ip, register-side index 4q + r  ->  column 32 * (ip / 2) + 8q + 4 * (ip % 2) + r.
// The epilogue therefore writes C, and reads the ReLU mask, in 16-byte pieces per lane with no
// shuffling.  (The fp32 instance keeps the natural row order instead: there a block's four
// registers are 16 contiguous bytes already.)  The B tile's LDS swizzle is chosen for
// that row order: the 16 lanes of a quarter-wave read rows 8q' + r' (+ multiples of 4 and 32),
// swizzle = 2 * ((row / 8) % 4) + (row / 2) % 2 gives them 16 distinct 16-byte slots.
//
// The transposed per-replica copy (Ct) wants runs along m instead: it goes through the then idle
// LDS, one private region per wavefront, as in gemm_bf16_dma.
//
// Two kernels share this tile, layout and epilogue: gemm_bf16_x32 (eight wavefronts of 128 x 64, the
// K step ordered by the compiler; also the chained-replica instance) and gemm_bf16_x32w4 (four
// wavefronts of 128 x 128, the K step written out instruction by instruction), further down.
#include <hip/hip_runtime.h>

#include "gemm_bf16_common.h"

namespace mi {

namespace {

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) const bf16x8 lds_frag;

constexpr int BM = 256, BN = 256, BK = 64, WM = 2, WN = 4, NW = WM * WN;
constexpr int WTM = BM / WM, WTN = BN / WN;   // 128 x 64 per wavefront
constexpr int QB = WTM / 16, PB = WTN / 16;   // 8 lane-side (m) blocks, 4 register-side (n) blocks
constexpr int A_ELEMS = BM * BK, B_ELEMS = BN * BK;
constexpr int VPR = BK / 8;                   // 16-byte chunks per tile row (a whole 128-byte line)
constexpr int RPI = 64 / VPR;                 // tile rows one load instruction of a wave fills
constexpr int NIA = BM / (RPI * NW), NIB = BN / (RPI * NW);
constexpr int INSTR = NIA + NIB;
constexpr size_t LDS_BYTES = 2 * (size_t)(A_ELEMS + B_ELEMS) * sizeof(u16);  // 128 KB
constexpr int STAGE_COL_BYTES = WTM * 2 + 8;  // one staged column of the transposed output + pad
constexpr int STAGE_REGION = 32 * STAGE_COL_BYTES;
static_assert((size_t)NW * STAGE_REGION <= LDS_BYTES, "staging must fit the ring");

__device__ __forceinline__ int swz_a(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int swz_b(int row) { return ((row >> 3) & 3) * 2 + ((row >> 1) & 1); }

// Epilogue of one wavefront: acc[jq][ip] is the 16 x 16 block of rows row0 + 16 jq + lane % 16 and
// the four columns described at the top of the file.
template <int EPI, bool ACC_IN_AGPRS = false>
__device__ __forceinline__ void store_x32(const HGemmArgs& p, f32x4 (&acc)[QB][PB], int row0, int colw, int lane,
                                          unsigned char* region, int bz) {
  const int l16 = lane & 15, q = lane >> 4;
  if constexpr (EPI == EPH_F32) {
    // natural B order, see the kernel.  A wave-uniform base (the batch entry's matrix) plus one 32-bit
    // byte offset per lane that walks down the rows: one register of address state, so that the
    // store burst between two K steps of the chained instance costs no registers the loop needs
    // (the launcher checks that a matrix spans less than 4 GB).
    const char* cbase = reinterpret_cast<const char*>(reinterpret_cast<float*>(p.C) + (size_t)bz * p.batchC);
    unsigned off = 4u * ((unsigned)(row0 + l16) * (unsigned)p.ldc + (unsigned)(colw + 4 * q));
    asm volatile("" : "+v"(off));  // derived here, not kept in registers across the K loop
    const unsigned row_step = 64u * (unsigned)p.ldc;  // 16 rows
#pragma unroll
    for (int jq = 0; jq < QB; ++jq) {
#pragma unroll
      for (int ip = 0; ip < PB; ++ip)
        *reinterpret_cast<f32x4*>(const_cast<char*>(cbase) + off + 64 * ip) = acc[jq][ip];
      off += row_step;
    }
    return;
  } else {
    u16* __restrict__ ch = reinterpret_cast<u16*>(p.C) + (size_t)bz * p.batchC;
    u32x4 pk[QB][2];  // the rounded results: eight consecutive columns per register quadruple
    // The whole mask of the wavefront's tile is requested before the first result is stored: the
    // counter that a load is waited for with retires loads and stores in order, so a mask load
    // issued after a store would wait for that store to reach the L2 first, sixteen times in a row.
    u32x4 mk_all[QB][2];
    if (EPI == EPH_MASK) {
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int jq = 0; jq < QB; ++jq)
          mk_all[jq][h] = *reinterpret_cast<const u32x4*>(p.mask + (size_t)(row0 + 16 * jq + l16) * p.ldmask + colw + 32 * h + 8 * q);
    }
    float bias_all[2][8];  // likewise the bias of the lane's sixteen columns
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e)
        bias_all[h][e] = (EPI == EPH_BIAS_RELU && p.bias) ? p.bias[colw + 32 * h + 8 * q + e] : 0.0f;
    asm volatile("" ::: "memory");  // the stores below stay below
#pragma unroll
    for (int jq = 0; jq < QB; ++jq) {
      const int row = row0 + 16 * jq + l16;
#pragma unroll
      for (int h = 0; h < 2; ++h) {  // both halves of a row's 128-byte line back to back
        const int col = colw + 32 * h + 8 * q;
        const float(&bias_v)[8] = bias_all[h];
        float v[8];
        if constexpr (ACC_IN_AGPRS) {
          // read out here and nowhere earlier: left to the compiler, all 256 accumulators are copied to
          // VGPRs in front of the epilogue, which then needs the whole register file
#pragma unroll
          for (int e = 0; e < 8; ++e) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v[e]) : "a"(acc[jq][2 * h + (e >> 2)][e & 3]));
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = acc[jq][2 * h + (e >> 2)][e & 3];
        }
        if (EPI == EPH_BIAS_RELU) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            v[e] += bias_v[e];
            if (p.relu) v[e] = v[e] > 0.0f ? v[e] : 0.0f;
          }
        } else if (EPI == EPH_MASK) {
          const u32x4 mk = mk_all[jq][h];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const u16 m = (u16)(mk[e >> 1] >> (16 * (e & 1)));
            if (!(bf2f(m) > 0.0f)) v[e] = 0.0f;
          }
        }
        u32x4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const f32x2_t two = {v[2 * e], v[2 * e + 1]};
          out[e] = __builtin_bit_cast(unsigned, __builtin_convertvector(two, bf16x2_t));  // round to nearest even
        }
        pk[jq][h] = out;
        *reinterpret_cast<u32x4*>(ch + (size_t)row * p.ldc + col) = out;
        if constexpr (ACC_IN_AGPRS) asm volatile("" : : "v"(out));  // (volatile statements keep their order: this row's work stays in front of the next row's reads)
      }
    }
    if (p.colsum_part) {
      // Column sums of the rounded values over the wavefront's 128 rows: a lane adds its eight rows
      // in block order, the 16 lanes of a quarter-wave are folded with a fixed butterfly.
      float* part = p.colsum_part + (size_t)(row0 / WTM) * p.N;
      float tot[2][8];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float c = 0.0f;
#pragma unroll
          for (int jq = 0; jq < QB; ++jq) {
            const unsigned two = pk[jq][h][e >> 1];
            c += (e & 1) ? __uint_as_float(two & 0xffff0000u) : __uint_as_float(two << 16);
          }
#pragma unroll
          for (int off = 1; off < 16; off <<= 1) c += __shfl_xor(c, off, 64);
          tot[h][e] = c;
        }
      // one lane of each quarter-wave writes its two runs of eight sums as 16-byte pieces (single
      // floats, a store instruction apart, reached the memory as one 64-byte write each)
      if (l16 == 0) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          float* dst = part + colw + 32 * h + 8 * q;
          *reinterpret_cast<f32x4*>(dst) = f32x4{tot[h][0], tot[h][1], tot[h][2], tot[h][3]};
          *reinterpret_cast<f32x4*>(dst + 4) = f32x4{tot[h][4], tot[h][5], tot[h][6], tot[h][7]};
        }
      }
    }
    if (!p.Ct) return;
    // Transposed copy: the tile lies inside one row group (ct_rows is a multiple of the tile height).
    // 32 columns at a time are staged [column][row] in the wavefront's LDS region (columns padded by
    // 8 bytes) and read back as 16-byte chunks: a store instruction writes runs of 256 contiguous bytes.
    const int group = row0 / p.ct_rows, m_local0 = row0 - group * p.ct_rows;
    u16* __restrict__ ct = p.Ct + (size_t)group * p.N * p.ct_rows + m_local0;
    // Neighbouring lanes hold neighbouring rows.  One exchange with lane ^ 1 turns a register (columns
    // 2k, 2k+1 of one row) into (rows 2p, 2p+1 of one column): even lanes keep the even columns, odd
    // lanes the odd ones, and the staging writes are 4 bytes instead of 2.
    const bool odd = lane & 1;
    const unsigned sel = odd ? 0x07060302u : 0x01000504u;  // bytes of {own (4-7), partner (0-3)}
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int jq = 0; jq < QB; ++jq)
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const unsigned own = pk[jq][h][k];
          const unsigned partner = (unsigned)__builtin_amdgcn_update_dpp(0, (int)own, 0xB1, 0xf, 0xf, false);  // lane ^ 1
          // even lane: (own.lo, partner.lo) = rows (m, m+1) of column 2k; odd lane: (partner.hi, own.hi) = rows (m-1, m) of column 2k+1
          const unsigned two = __builtin_amdgcn_perm(own, partner, sel);
          *reinterpret_cast<unsigned*>(region + (8 * q + 2 * k + (lane & 1)) * STAGE_COL_BYTES + (16 * jq + (l16 & 14)) * 2) = two;
        }
      constexpr int CHUNKS = WTM / 8;  // 16-byte chunks per column
#pragma unroll
      for (int i = lane; i < 32 * CHUNKS; i += 64) {
        const int c = i / CHUNKS, piece = i % CHUNKS;
        // columns start at multiples of 8 bytes only: two 8-byte LDS reads per 16-byte global store
        const u32x2 lo = *reinterpret_cast<const u32x2*>(region + c * STAGE_COL_BYTES + piece * 16);
        const u32x2 up = *reinterpret_cast<const u32x2*>(region + c * STAGE_COL_BYTES + piece * 16 + 8);
        const u32x4 v = {lo[0], lo[1], up[0], up[1]};
        // non-temporal: the copy is read by a weight-gradient GEMM much later, and as a second stream of
        // ordinary stores next to C's it costs more than its bytes (8192-wide layers, batch 16384:
        // forward 1.535 -> 1.524 ms, input gradient 1.570 -> 1.542 ms per GEMM)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(ct + (size_t)(colw + 32 * h + c) * p.ct_rows + piece * 8));
      }
    }
  }
}

// CHAIN = true (fp32 results, i.e. the weight gradient): the batch entries of one launch are the
// replicas of a layer, all with the same (m, n) tiles.  A workgroup keeps its tile and walks
// p.chain consecutive entries as one long K loop whose two LDS buffers never drain: at the end of an
// entry's K range the operand bases jump to the next entry, the accumulators are stored as that
// entry's tile and cleared, and the loop goes on.  The tile loads of the first step of the next
// entry were requested before those stores, so the wait in front of that step's barrier leaves
// exactly the stores outstanding (the counter retires loads and stores in order); they have one K
// step to drain before the next wait has to see them gone.  Prologue, epilogue and workgroup
// turnover are paid once per p.chain entries.  Needs K / 64 even and at least 4.
// (The chained instance keeps one loop-invariant value in scratch memory; it is reloaded only in the
// epilogue after the last step, so no scratch access sits between the tile loads the loop counts.)
constexpr int TILE_STORES_F32 = QB * PB;  // 16-byte store instructions per wavefront and tile

template <int EPI, int PRIO, bool CHAIN = false>
__global__ __launch_bounds__(NW * 64) void gemm_bf16_x32(HGemmArgs p) {
  static_assert(!CHAIN || EPI == EPH_F32, "chained batch entries: fp32 results only");
  extern __shared__ __attribute__((aligned(16))) u16 smem_x[];
  // (made wave-uniform explicitly: everything derived from it for the tile loads then stays in
  // scalar registers instead of one vector register per load instruction and buffer)
  const unsigned lds_base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)((__attribute__((address_space(3))) const void*)smem_x));
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kg = lane >> 4;
  // fp32 results: a lane's four registers of a block are 16 contiguous bytes, so the rows of the B
  // tile keep their natural order (block ip = columns 16 ip .. 16 ip + 15, lane quarter q columns
  // 4q .. 4q+3 of them) and a store instruction writes 64 contiguous bytes per row; the dealt order
  // described at the top would leave 16-byte holes that the next instruction fills.
  constexpr bool NAT = EPI == EPH_F32;
  const int wm0 = (wave / WN) * WTM, wn0 = (wave % WN) * WTN;

  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  // tile loads: a wave-uniform base per operand, advanced with scalar adds, plus one constant byte
  // offset per lane and instruction (no vector arithmetic in the K loop)
  const int lrow = lane / VPR, pc = lane % VPR;
  unsigned offa[NIA], offb[NIB];
#pragma unroll
  for (int j = 0; j < NIA; ++j) {
    const int row = (j * NW + wave) * RPI + lrow;
    offa[j] = 2u * ((unsigned)row * (unsigned)p.lda + (unsigned)(pc ^ swz_a(row)) * 8u);
  }
#pragma unroll
  for (int j = 0; j < NIB; ++j) {
    const int row = (j * NW + wave) * RPI + lrow;
    offb[j] = 2u * ((unsigned)row * (unsigned)p.ldb + (unsigned)(pc ^ (NAT ? swz_a(row) : swz_b(row))) * 8u);
  }
  int bz = CHAIN ? (int)blockIdx.z * p.chain : (int)blockIdx.z;  // first (or only) batch entry of this workgroup
  const u16* a_base = p.A + (size_t)bz * p.batchA + (size_t)m0 * p.lda;
  const u16* b_base = p.B + (size_t)bz * p.batchB + (size_t)n0 * p.ldb;
  const int steps_per_entry = p.K / BK;
  int a_left = steps_per_entry, b_left = steps_per_entry;  // CHAIN: tiles still to request from the current entry
  auto issue_a = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NIA; ++j)
      load_to_lds_uniform(a_base, offa[j], lds_base + 2u * (unsigned)(buf * A_ELEMS + (j * NW + wave) * RPI * BK));
    a_base += BK;
    if (CHAIN && --a_left == 0) {  // on to the next entry's first K step
      a_left = steps_per_entry;
      a_base += p.batchA - p.K;
    }
  };
  auto issue_b = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NIB; ++j)
      load_to_lds_uniform(b_base, offb[j], lds_base + 2u * (unsigned)(2 * A_ELEMS + buf * B_ELEMS + (j * NW + wave) * RPI * BK));
    b_base += BK;
    if (CHAIN && --b_left == 0) {
      b_left = steps_per_entry;
      b_base += p.batchB - p.K;
    }
  };

  // LDS byte addresses of this lane's fragments for K chunk 0 / 1 (block 0, buffer 0); blocks and
  // buffers are immediate offsets.  The empty asm keeps the compiler from re-deriving them in the loop.
  unsigned q_addr[2], p_addr[2];
#pragma unroll
  for (int kc = 0; kc < 2; ++kc) {
    const int ra = wm0 + l16, rb = NAT ? wn0 + l16 : wn0 + 8 * (l16 >> 2) + (l16 & 3);
    q_addr[kc] = lds_base + 2u * (unsigned)(ra * BK + ((kc * 4 + kg) ^ swz_a(ra)) * 8);
    p_addr[kc] = lds_base + 2u * (unsigned)(2 * A_ELEMS + rb * BK + ((kc * 4 + kg) ^ (NAT ? swz_a(rb) : swz_b(rb))) * 8);
    asm volatile("" : "+v"(q_addr[kc]), "+v"(p_addr[kc]));
  }
  auto load_q = [&](bf16x8 (&f)[4], int buf, int kc, int half) __attribute__((always_inline)) {
#pragma unroll
    for (int jj = 0; jj < 4; ++jj)
      f[jj] = *reinterpret_cast<lds_frag*>((__attribute__((address_space(3))) const char*)(size_t)(
          q_addr[kc] + 2u * (unsigned)(buf * A_ELEMS + (half * 4 + jj) * 16 * BK)));
  };
  auto load_p = [&](bf16x8 (&f)[PB], int buf, int kc) __attribute__((always_inline)) {
#pragma unroll
    for (int ip = 0; ip < PB; ++ip)
      f[ip] = *reinterpret_cast<lds_frag*>((__attribute__((address_space(3))) const char*)(size_t)(
          p_addr[kc] + 2u * (unsigned)(buf * B_ELEMS + (NAT ? 16 * ip : 32 * (ip >> 1) + 4 * (ip & 1)) * BK)));
  };

  f32x4 acc[QB][PB];
  auto clear_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int jq = 0; jq < QB; ++jq)
#pragma unroll
      for (int ip = 0; ip < PB; ++ip)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[jq][ip][r] = 0.0f;
  };
  clear_acc();

  const int nk = CHAIN ? steps_per_entry * p.chain : steps_per_entry;
  bool stores_in_flight = false;  // CHAIN: the step before ended with the store burst of an entry
  bf16x8 fq[2][4], fp[2][PB];
  // sub-chunk s of a step: K chunk s / 2, m blocks 4 (s % 2) .. 4 (s % 2) + 3
  auto multiply = [&](int s) __attribute__((always_inline)) {
    if (PRIO == 1) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int jj = 0; jj < 4; ++jj)
#pragma unroll
      for (int ip = 0; ip < PB; ++ip)
        acc[(s & 1) * 4 + jj][ip] =
            __builtin_amdgcn_mfma_f32_16x16x32_bf16(fp[(s >> 1) & 1][ip], fq[s & 1][jj], acc[(s & 1) * 4 + jj][ip], 0, 0, 0);
    if (PRIO == 1) __builtin_amdgcn_s_setprio(0);
  };

  if (nk > 0) {
    issue_a(0);
    issue_b(0);
  }
  if (nk > 1) {
    issue_a(1);
    issue_b(1);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(INSTR));
  } else {
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  }
  ring_barrier();
  load_q(fq[0], 0, 0, 0);
  load_p(fp[0], 0, 0);
  // Step t multiplies buffer t % 2.  Before its last sub-chunk every wavefront has issued all its
  // reads of that buffer; it waits for them and for tile t+1 (the other buffer), then the barrier,
  // then tile t+2 is requested into the buffer just read out.  The first fragments of tile t+1 are
  // fetched under the last sub-chunk's MFMAs.
  auto step = [&](int t, auto cur_c, auto steady_c) __attribute__((always_inline)) {
    constexpr int cur = decltype(cur_c)::value;
    constexpr bool steady = decltype(steady_c)::value;  // tile t+2 exists
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int ns = s + 1;
      if (ns < 4) {
        load_q(fq[ns & 1], cur, ns >> 1, ns & 1);
        if ((ns & 1) == 0) load_p(fp[(ns >> 1) & 1], cur, ns >> 1);
      } else {  // after the last tile: a harmless read of ring memory, keeps one code path
        load_q(fq[0], cur ^ 1, 0, 0);
        load_p(fp[0], cur ^ 1, 0);
      }
      if (s == 2) __builtin_amdgcn_sched_barrier(0);  // the last reads of this buffer go out before these MFMAs
      multiply(s);
      if (s == 2) {
        __builtin_amdgcn_sched_barrier(0);  // and the MFMAs stay above the barrier
        // lgkmcnt(0), and the tile of step t+1 must have landed; the stores of an entry that ended
        // with the step before are younger than its loads and may stay outstanding
        if (CHAIN && stores_in_flight) __builtin_amdgcn_s_waitcnt(vmcnt_imm(TILE_STORES_F32) & 0xc07f);
        else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0) & 0xc07f);
        ring_barrier();
        if (steady || t + 2 < nk) issue_a(cur);
      }
      if (s == 3) {
        if (steady || t + 2 < nk) issue_b(cur);
      }
    }
  };
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  int t = 0;
  if constexpr (CHAIN) {
    // Per entry: a first pair of steps (the first of them right behind the stores of the entry
    // before), the pairs in between, and -- all entries but the last -- the store of the finished
    // tile; the last entry ends with the two steps that request nothing more and leaves through the
    // epilogue below.  An entry has an even number of steps, at
    // least four, so every step here but those last two has a tile t+2 to request.
    for (int e = 0; e < p.chain; ++e) {
      const bool last_entry = e + 1 == p.chain;
      step(t, C0{}, std::true_type{});
      stores_in_flight = false;
      step(t + 1, C1{}, std::true_type{});
      t += 2;
      const int pairs_end = (e + 1) * steps_per_entry - (last_entry ? 2 : 0);
      for (; t < pairs_end; t += 2) {
        step(t, C0{}, std::true_type{});
        step(t + 1, C1{}, std::true_type{});
      }
      if (!last_entry) {
        // fenced on both sides: stores drifting down among the next step's MFMAs would keep the old
        // sums alive next to the new ones, which the register file has no room for
        __builtin_amdgcn_sched_barrier(0);
        store_x32<EPI>(p, acc, m0 + wm0, n0 + wn0, lane, nullptr, bz);
        __builtin_amdgcn_sched_barrier(0);
        clear_acc();
        __builtin_amdgcn_sched_barrier(0);
        ++bz;
        stores_in_flight = true;
      }
    }
    step(t, C0{}, std::false_type{});
    step(t + 1, C1{}, std::false_type{});
  } else {
    for (; t + 4 <= nk; t += 2) {
      step(t, C0{}, std::true_type{});
      step(t + 1, C1{}, std::true_type{});
    }
    static_for_h<3>([&](auto sc) {
      constexpr int s = decltype(sc)::value;
      if (t + s < nk) step(t + s, std::integral_constant<int, s % 2>{}, std::false_type{});
    });
  }

  unsigned char* region = nullptr;
  if (EPI != EPH_F32 && p.Ct) {
    __syncthreads();  // every wavefront is done with the operand tiles: the LDS is free for the staging
    region = reinterpret_cast<unsigned char*>(smem_x) + (size_t)wave * STAGE_REGION;
  }
  store_x32<EPI>(p, acc, m0 + wm0, n0 + wn0, lane, region, bz);
}

// ---- the same tile with four wavefronts of 128 x 128, one per SIMD -------------------------------
// A wavefront that owns 128 x 128 of the tile reads a third fewer fragment bytes from the LDS per MFMA
// than one that owns 128 x 64, and the matrix cores of this device are power-limited: what the LDS
// does not draw, the clock gets.  With one wavefront per SIMD, though, nothing covers a wait, so the
// whole K step is written out as volatile asm statements, which the compiler keeps in source order:
//   * 64 accumulator blocks (256 registers) live in AGPRs and every MFMA accumulates in place (left
//     to itself the compiler moves them between the two register files around the MFMAs: 416 moves
//     per K step);
//   * a step is four sub-chunks of 32 MFMAs (K chunk 0 / 1 times the lower / upper four 16-row
//     blocks); the fragments of the next sub-chunk are read one ds_read_b128 after every second MFMA
//     and waited for once, at the end of the sub-chunk, so no MFMA ever waits for a read issued
//     right in front of it;
//   * the 16 tile loads of a wavefront and step go out one after every fifth MFMA, starting behind the
//     barrier that frees their buffer: each direct-to-LDS load holds up the wavefront that issues it,
//     and spread like this the MFMA already in the pipe covers most of it (all 16 in two bursts:
//     +9 %; one per 2 / 3 / 4 / 6 MFMAs: +12 / +5 / +0.5 / +1 %);
//   * the counters are waited for by hand (the compiler does not see these loads and reads).
// Measured on 16384 x 8192 x 8192 against the eight-wavefront kernel above on the same box and data:
// 1450-1512 us against 1477-1584 us (2-5 % less; boxes differ).  The same loop with its tile loads
// taken out runs 1196-1290 us, with loads that always hit the caches 1342-1490 us.
// Prologue / epilogue as above; the epilogue runs store_x32 once per 64-column half.
constexpr int W4_NW = 4, W4_WN = 2;
constexpr int W4_WTN = BN / W4_WN;                 // 128 columns per wavefront
constexpr int W4_PB = W4_WTN / 16;                 // 8 register-side (n) blocks
constexpr int W4_NI = BM / (RPI * W4_NW);          // 8 load instructions per wavefront, operand and tile
constexpr int W4_SP = 5;                           // a tile load after every fifth MFMA ...
constexpr int W4_FIRST = (4 * W4_PB - W4_SP / 2 + W4_SP - 1) / W4_SP;  // ... so many of a tile's 16 in the first sub-chunk of their window
typedef int i32x4_t __attribute__((ext_vector_type(4)));

template <int EPI>
__global__ __launch_bounds__(W4_NW * 64) void gemm_bf16_x32w4(HGemmArgs p) {
  extern __shared__ __attribute__((aligned(16))) u16 smem_x[];
  const unsigned lds_base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)((__attribute__((address_space(3))) const void*)smem_x));
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15, kg = lane >> 4;
  constexpr bool NAT = EPI == EPH_F32;  // fp32 results: natural row order of the B tile, as in the kernel above
  const int wm0 = (wave / W4_WN) * WTM, wn0 = (wave % W4_WN) * W4_WTN;

  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int bz = blockIdx.z;

  const int lrow = lane / VPR, pc = lane % VPR;
  unsigned offa[W4_NI], offb[W4_NI];
#pragma unroll
  for (int j = 0; j < W4_NI; ++j) {
    const int row = (j * W4_NW + wave) * RPI + lrow;
    offa[j] = 2u * ((unsigned)row * (unsigned)p.lda + (unsigned)(pc ^ swz_a(row)) * 8u);
    offb[j] = 2u * ((unsigned)row * (unsigned)p.ldb + (unsigned)(pc ^ (NAT ? swz_a(row) : swz_b(row))) * 8u);
  }
  // the operand bases as scalar values (the builtin returns int: widen as unsigned)
  auto uniform64 = [](const void* q) {
    const unsigned long long b = reinterpret_cast<unsigned long long>(q);
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)b), hi = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32));
    return ((unsigned long long)hi << 32) | lo;
  };
  unsigned long long sa = uniform64(p.A + (size_t)bz * p.batchA + (size_t)m0 * p.lda);
  unsigned long long sb = uniform64(p.B + (size_t)bz * p.batchB + (size_t)n0 * p.ldb);
  auto load_s = [](unsigned long long sbase, unsigned lane_off, unsigned lds_addr) __attribute__((always_inline)) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_addr), "v"(lane_off), "s"(sbase) : "memory", "m0");
  };
  // load i of a tile's 16 (A's eight, then B's eight) into ring buffer buf; the base moves on to the
  // next K step behind an operand's last load
  auto tile_load = [&](auto i_c, int buf) __attribute__((always_inline)) {
    constexpr int i = decltype(i_c)::value;
    if constexpr (i < W4_NI) {
      load_s(sa, offa[i], lds_base + 2u * (unsigned)(buf * A_ELEMS + (i * W4_NW + wave) * RPI * BK));
      if (i == W4_NI - 1) sa += 2 * BK;
    } else {
      constexpr int j = i - W4_NI;
      load_s(sb, offb[j], lds_base + 2u * (unsigned)(2 * A_ELEMS + buf * B_ELEMS + (j * W4_NW + wave) * RPI * BK));
      if (j == W4_NI - 1) sb += 2 * BK;
    }
  };

  unsigned q_addr[2], p_addr[2];
#pragma unroll
  for (int kc = 0; kc < 2; ++kc) {
    const int ra = wm0 + l16, rb = NAT ? wn0 + l16 : wn0 + 8 * (l16 >> 2) + (l16 & 3);
    q_addr[kc] = lds_base + 2u * (unsigned)(ra * BK + ((kc * 4 + kg) ^ swz_a(ra)) * 8);
    p_addr[kc] = lds_base + 2u * (unsigned)(2 * A_ELEMS + rb * BK + ((kc * 4 + kg) ^ (NAT ? swz_a(rb) : swz_b(rb))) * 8);
    asm volatile("" : "+v"(q_addr[kc]), "+v"(p_addr[kc]));
  }
  // fragment r of the 4 (m side) + 8 (n side) that sub-chunk (kc, half) multiplies, from ring buffer buf
  i32x4_t fq[2][4], fp[2][W4_PB];
  auto frag_read = [&](auto r_c, auto buf_c, auto kc_c, auto half_c, auto qslot_c, auto pslot_c) __attribute__((always_inline)) {
    constexpr int r = decltype(r_c)::value, buf = decltype(buf_c)::value, kc = decltype(kc_c)::value;
    constexpr int half = decltype(half_c)::value, qslot = decltype(qslot_c)::value, pslot = decltype(pslot_c)::value;
    auto& fq_ = fq; auto& fp_ = fp; auto& qa_ = q_addr; auto& pa_ = p_addr;  // (named so that the lambda captures them: operands of asm statements alone do not)
    if constexpr (r < 4) {
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(fq_[qslot][r]) : "v"(qa_[kc]), "i"(2 * (buf * A_ELEMS + (half * 4 + r) * 16 * BK)));
    } else {
      constexpr int ip = r - 4;
      asm volatile("ds_read_b128 %0, %1 offset:%2"
                   : "=&v"(fp_[pslot][ip])
                   : "v"(pa_[kc]), "i"(2 * (buf * B_ELEMS + (NAT ? 16 * ip : 32 * (ip >> 1) + 4 * (ip & 1)) * BK)));
    }
  };

  // acc[h][jq][ip]: rows 16 jq .. 16 jq + 15 of the wavefront's 128, n block 4 h + ip (64-column half h)
  f32x4 acc[2][QB][4];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int jq = 0; jq < QB; ++jq)
#pragma unroll
      for (int ip = 0; ip < 4; ++ip)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[h][jq][ip][r] = 0.0f;

  const int nk = p.K / BK;
  // Prologue: tile 0 whole, and of tile 1 what a step requests in the first sub-chunk of a tile's
  // window; step 0 requests the rest like every other step.
  static_for_h<2 * W4_NI>([&](auto ic) { tile_load(ic, 0); });
  if (nk > 1) {
    static_for_h<W4_FIRST>([&](auto ic) { tile_load(ic, 1); });
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(W4_FIRST));
  } else {
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  }
  ring_barrier();
  using I0 = std::integral_constant<int, 0>;
  static_for_h<4 + W4_PB>([&](auto rc) { frag_read(rc, I0{}, I0{}, I0{}, I0{}, I0{}); });
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

  // Step t multiplies buffer t % 2.  Sub-chunk s uses the m-side fragments in slot s % 2 and the n-side
  // fragments in slot s / 2 and reads those of sub-chunk s + 1 (s = 3: of step t + 1, from the other
  // buffer) into the other slots.  Behind sub-chunk 2: every read of this buffer and tile t+1 are
  // waited for, then the barrier; the window of tile t+2 (into this buffer) opens with sub-chunk 3 and
  // runs on through sub-chunks 0 and 1 of step t+1.
  auto step = [&](int t, auto cur_c, auto steady_c) __attribute__((always_inline)) {
    constexpr int cur = decltype(cur_c)::value;
    constexpr bool steady = decltype(steady_c)::value;  // tiles t+1 and t+2 exist
    static_for_h<4>([&](auto s_c) {
      constexpr int s = decltype(s_c)::value, ns = (s + 1) & 3;
      using RBuf = std::integral_constant<int, (s == 3 ? (cur ^ 1) : cur)>;
      using NKc = std::integral_constant<int, (ns >> 1)>;
      using NHalf = std::integral_constant<int, (ns & 1)>;
      using QSlot = std::integral_constant<int, (ns & 1)>;
      using PSlot = std::integral_constant<int, ((ns >> 1) & 1)>;
      constexpr int nreads = 4 + ((ns & 1) == 0 ? W4_PB : 0);  // the n-side fragments change with the K chunk only
      static_for_h<4 * W4_PB>([&](auto ic) {
        constexpr int idx = decltype(ic)::value, jj = idx / W4_PB, ip = idx % W4_PB;
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                     : "+a"(acc[ip >> 2][(s & 1) * 4 + jj][ip & 3])
                     : "v"(fp[(s >> 1) & 1][ip]), "v"(fq[s & 1][jj]));
        if constexpr ((idx & 1) == 1 && idx / 2 < nreads)
          frag_read(std::integral_constant<int, idx / 2>{}, RBuf{}, NKc{}, NHalf{}, QSlot{}, PSlot{});
        constexpr int w = ((s + 1) & 3) * 4 * W4_PB + idx;  // position in the window that sub-chunk 3 opens
        if constexpr (s != 2 && w % W4_SP == W4_SP / 2 && w / W4_SP < 2 * W4_NI) {
          // s == 3: tile t+2 into this buffer; s == 0, 1: the rest of tile t+1 into the other one
          if (s == 3 ? (steady || t + 2 < nk) : (steady || t + 1 < nk))
            tile_load(std::integral_constant<int, w / W4_SP>{}, s == 3 ? cur : cur ^ 1);
        }
      });
      if constexpr (s == 2) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
      else asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    });
  };
  using C0 = std::integral_constant<int, 0>;
  using C1 = std::integral_constant<int, 1>;
  int t = 0;
  for (; t + 4 <= nk; t += 2) {
    step(t, C0{}, std::true_type{});
    step(t + 1, C1{}, std::true_type{});
  }
  static_for_h<3>([&](auto sc) {
    constexpr int s = decltype(sc)::value;
    if (t + s < nk) step(t + s, std::integral_constant<int, s % 2>{}, std::false_type{});
  });
  // the compiler does not know that MFMAs have just written the accumulators it is about to read
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

  unsigned char* region = nullptr;
  if (EPI != EPH_F32 && p.Ct) {
    __syncthreads();  // every wavefront is done with the operand tiles: the LDS is free for the staging
    region = reinterpret_cast<unsigned char*>(smem_x) + (size_t)wave * STAGE_REGION;
  }
  // what the epilogue derives its addresses from is made opaque here, so that none of it is computed
  // ahead of the K loop and kept in registers through it
  int lane_e = lane, row_e = m0 + wm0, col_e = n0 + wn0;
  asm volatile("" : "+v"(lane_e), "+s"(row_e), "+s"(col_e));
  store_x32<EPI, EPI != EPH_F32>(p, acc[0], row_e, col_e, lane_e, region, bz);
  store_x32<EPI, EPI != EPH_F32>(p, acc[1], row_e, col_e + 64, lane_e, region, bz);
}

template <int EPI>
hipError_t launch_w4(HGemmArgs& p, int batch, hipStream_t s) {
  p.tiles_m = p.M / BM;
  p.tiles_n = p.N / BN;
  p.chain = 1;
  auto kern = gemm_bf16_x32w4<EPI>;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), LDS_BYTES); e != hipSuccess) return e;
  launch_kernel(kern, dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(W4_NW * 64), LDS_BYTES, s, p);
  return hipGetLastError();
}

template <int EPI, int PRIO>
hipError_t launch_one(HGemmArgs& p, int batch, hipStream_t s) {
  p.tiles_m = p.M / BM;
  p.tiles_n = p.N / BN;
  if constexpr (EPI == EPH_F32) {
    // chained batch entries (p.chain > 1, set by the caller's choice): groups of p.chain entries per workgroup
    const int steps = p.K / BK;
    if (p.chain > 1 && batch % p.chain == 0 && steps >= 4 && steps % 2 == 0) {
      auto kern = gemm_bf16_x32<EPI, PRIO, true>;
      static LdsOptIn opt_in;
      if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), LDS_BYTES); e != hipSuccess) return e;
      launch_kernel(kern, dim3(p.tiles_m * p.tiles_n, 1, batch / p.chain), dim3(NW * 64), LDS_BYTES, s, p);
      return hipGetLastError();
    }
  }
  p.chain = 1;
  auto kern = gemm_bf16_x32<EPI, PRIO, false>;
  static LdsOptIn opt_in;
  if (hipError_t e = opt_in.ensure(reinterpret_cast<const void*>(kern), LDS_BYTES); e != hipSuccess) return e;
  launch_kernel(kern, dim3(p.tiles_m * p.tiles_n, 1, batch), dim3(NW * 64), LDS_BYTES, s, p);
  return hipGetLastError();
}

template <int PRIO>
hipError_t launch_prio(HGemmArgs& p, int batch, int epi, hipStream_t s) {
  switch (epi) {
    case EPH_F32: return launch_one<EPH_F32, PRIO>(p, batch, s);
    case EPH_BIAS_RELU: return launch_one<EPH_BIAS_RELU, PRIO>(p, batch, s);
    case EPH_MASK: return launch_one<EPH_MASK, PRIO>(p, batch, s);
    default: return launch_one<EPH_BF16, PRIO>(p, batch, s);
  }
}

}  // namespace

hipError_t launch_x32(HGemmArgs& p, int batch, int epi, bool prio, hipStream_t s) {
  return prio ? launch_prio<1>(p, batch, epi, s) : launch_prio<0>(p, batch, epi, s);
}

hipError_t launch_x32w4(HGemmArgs& p, int batch, int epi, hipStream_t s) {
  switch (epi) {
    case EPH_F32: return launch_w4<EPH_F32>(p, batch, s);
    case EPH_BIAS_RELU: return launch_w4<EPH_BIAS_RELU>(p, batch, s);
    case EPH_MASK: return launch_w4<EPH_MASK>(p, batch, s);
    default: return launch_w4<EPH_BF16>(p, batch, s);
  }
}

}  // namespace mi
