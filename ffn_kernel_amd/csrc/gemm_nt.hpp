// Routed "NT" GEMM core for gfx950: C[rows, N] = A[rows, K] * B_g[N, K]^T with both operands
// K-contiguous, bf16 in, fp32 MFMA accumulation.  Rows are processed in routed order (visual
// group first); a workgroup tile never mixes groups, so each tile multiplies by exactly one
// modality's weight.  This replaces the per-tile three-way branch of the reference kernels
// (ffn_kernel/linear.py:127-153, ffn_kernel/ffn.py:68-105), which pay two dots and a select
// on every mixed tile.
//
// Data path per workgroup: 64-column K slabs of the A and B panels go global -> LDS, two stages
// deep (directly, bypassing registers, when K is a multiple of 64; staged through registers
// otherwise); wavefronts read 16-byte MFMA fragments from an XOR-swizzled LDS layout and issue
// v_mfma_f32_16x16x32_bf16 on the 256-row direct tiles (gemm_mainloop_fixed16) and v_mfma_f32_32x32x16_bf16
// on the others (gemm_mainloop_slab_dma, gemm_mainloop_ring, gemm_mainloop_staged).
//
// The backward GEMMs find one operand with the contraction running over its rows ([K, N], N
// contiguous: a forward weight seen from the output side, or activations whose rows are summed).
// RoutedGemmCfg::B_KMAJOR reads such a panel in place: same slabs and stages, the fragments built by
// the transposing LDS read (see KMajorB).
#pragma once
#include <type_traits>
#include "common.hpp"
#include "gemm_args.hpp"
#include "gemm_sched.hpp"

namespace ffnk {

constexpr int kBK = 64;          // K elements per LDS stage
constexpr int kRowBytes = 128;   // kBK * sizeof(bf16)
constexpr int kXcds = 8;         // MI355X: 8 XCDs, workgroups are dealt to them round-robin

// ---------------------------------------------------------------------------------------------
// LDS layout: a slab holds 128-byte rows (64 K elements).  The swizzle keeps every ds_read_b128 of
// an MFMA fragment (16 consecutive tile rows, same logical 16-byte chunk, per 16-lane phase) on 16
// distinct 16-byte bank groups, and lets a wavefront fill LDS in lane order (lane -> 16 bytes at
// lane * 16), which is what a global->LDS load requires.
// ---------------------------------------------------------------------------------------------
__host__ __device__ constexpr uint32_t lds_swizzle(uint32_t r, uint32_t c) {  // c in 0..7
  return ((r >> 1) << 8) | (((((r & 1u) ^ ((r >> 3) & 1u)) << 3) | (c ^ (r & 7u))) << 4);
}

#define FFNK_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// ---------------------------------------------------------------------------------------------
// K-major weight panels (RoutedGemmCfg::B_KMAJOR).  The backward GEMMs contract over the axis that
// is the forward's output axis, so they find a weight as [K, N] rows with N contiguous.  A slab of
// such a panel is 64 rows of BN elements, stored row by row in LDS (again in lane order of the
// global->LDS loads).  ds_read_b64_tr_b16 turns it into MFMA operands: within a group of 16 lanes,
// lane j addresses 4 consecutive elements and lane i receives elements i, 16 + i, 32 + i, 48 + i of
// the 64 the group addressed.  With lanes 4r ... 4r+3 on 16 consecutive columns of row k + r, lane i
// gets column i of rows k ... k+3; two reads make the 8-element K run of an MFMA operand (32x32x16: two groups of
// 16 lanes side by side cover a tile's 32 columns and the lane halves its two K runs; 16x16x32: one group covers the
// tile's 16 columns and the four groups of a wave its four K runs).
// Rows are BN * 2 bytes, a multiple of the 256 bytes the banks span, so the four rows of a read are
// spread by XOR-ing the 64-byte unit index of a row with kmajor_swizzle_key(row).
// ---------------------------------------------------------------------------------------------
template <int BN>
__host__ __device__ constexpr uint32_t kmajor_swizzle_key(uint32_t k) {
  return BN >= 128 ? (k & 3u) : ((k >> 1) & 1u);  // BN = 64: rows 128 bytes apart, two units each
}

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;

// The transposing read is written as an asm statement: through its builtin the compiler takes it for
// a possible LDS store and puts s_waitcnt vmcnt(0) before every one that follows a global->LDS load,
// which would drain the slab prefetch at each K step.  The compiler therefore does not know that the
// result arrives later: kmajor_wait_frags() must stand between the reads and the first use.
template <int OFFSET>
__device__ __forceinline__ bf16x4_t lds_read_tr16_b64(uint32_t addr) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "DS offset field is 16 bits");
  bf16x4_t r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFFSET));
  return r;
}
// Wait for every outstanding LDS read of the wave; the fragments pass through the statement so that
// no use of them can be moved above it.
template <int TN>
__device__ __forceinline__ void kmajor_wait_frags(bf16x4_t (&lo)[TN], bf16x4_t (&hi)[TN]) {
  static_assert(TN == 1 || TN == 2 || TN == 4, "weight fragments per K step");
  if constexpr (TN == 1) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[0]), "+v"(hi[0]));
  if constexpr (TN == 2) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[0]), "+v"(hi[0]), "+v"(lo[1]), "+v"(hi[1]));
  if constexpr (TN == 4)
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(lo[0]), "+v"(hi[0]), "+v"(lo[1]), "+v"(hi[1]), "+v"(lo[2]), "+v"(hi[2]), "+v"(lo[3]), "+v"(hi[3]));
}

struct KMajorB {
  const uint16_t* w[2] = {nullptr, nullptr};  // slabs [0, kt_switch) of the contraction come from w[0], the rest from w[1]
  int kt_first = 0;                           // first slab of this workgroup's K range
  int kt_switch = 0x7fffffff;
  uint32_t slab_bytes = 0;                    // 64 rows: 64 * ldb * 2
  // Rows of the range's last slab that belong to the contraction (1..64).  The rest of that slab is
  // cleared in LDS before it is read, so whatever lies behind the operand's last row never counts.
  int last_rows = 64;
};

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, bool DUAL_, bool GATHER_A_, bool SCATTER_C_,
          bool DIRECT_, int GROUP_M_, bool B_KMAJOR_ = false, int STAGES_ = 2>
struct RoutedGemmCfg {
  static constexpr int BM = BM_;            // token rows per tile
  static constexpr int BN = BN_;            // B rows held in LDS per tile (DUAL: half gate, half up)
  static constexpr int WAVES_M = WAVES_M_;
  static constexpr int WAVES_N = WAVES_N_;
  static constexpr bool DUAL = DUAL_;
  static constexpr bool GATHER_A = GATHER_A_;
  static constexpr bool SCATTER_C = SCATTER_C_;
  static constexpr bool DIRECT = DIRECT_;   // global->LDS loads bypass registers (needs K % 64 == 0)
  static constexpr int GROUP_M = GROUP_M_;
  // Weight panels are [K, N] rows with N contiguous (the backward's view of a forward weight) and
  // are transposed on the way from LDS to the MFMA operand, see KMajorB.
  static constexpr bool B_KMAJOR = B_KMAJOR_;
  static constexpr int NWAVES = WAVES_M * WAVES_N;
  static constexpr int NT = NWAVES * kWave;
  static constexpr int BN_OUT = DUAL ? BN / 2 : BN;        // output columns per tile
  static constexpr int WTM = BM / WAVES_M;                 // rows per wave
  static constexpr int WTN_OUT = BN_OUT / WAVES_N;         // output columns per wave
  // The 256-row direct tiles accumulate with v_mfma_f32_16x16x32_bf16 (four accumulator registers read
  // and written per 16 K-products of a lane instead of sixteen per 16: the kernel runs at the board's
  // power limit and the narrower accumulator traffic is worth 5 % there); the others with 32x32x16.  K-major
  // weight panels included: MaskedFFN forward + backward at d = 4096, h = 14336 runs 4.5 % (M = 4096) to 7 %
  // (M = 32768) faster than with the backward's 256-row GEMMs on the two-stage 32x32x16 loop.
  static constexpr bool MFMA16 = DIRECT_ && BM_ == 256;
  // Cache policy of the token panel's global->LDS loads.  The down projection's token rows (the routed intermediate,
  // read in place) pass each XCD once: a round of tiles reads a line and no later round does.  Loaded with the
  // non-temporal hint they do not push the weight panels out of L2 (cfg4 down projection 2.91 -> 2.85 ms, M = 16384
  // 1.47 -> 1.45 ms on the two-stage form; no difference left behind the three-stage token ring, and none on the
  // smaller tiles, which keep the default).  Gathered token rows
  // are read again by the next rounds (the hint costs 9 % there), and so are the weights (2-4 %).
  static constexpr int AUX_A = (MFMA16 && !GATHER_A_ && SCATTER_C_) ? 2 : 0;
  static constexpr int MT = MFMA16 ? 16 : 32;              // edge of an accumulator tile
  static constexpr int ACC_N = MT * MT / kWave;            // accumulator registers per tile
  using Acc = std::conditional_t<MFMA16, f32x4_t, f32x16_t>;
  static constexpr int TM = WTM / MT;                      // accumulator tiles per wave, M direction
  static constexpr int TN_OUT = WTN_OUT / MT;
  static constexpr int TN = DUAL ? 2 * TN_OUT : TN_OUT;    // accumulator tiles per wave, N direction
  static constexpr int A_BYTES = BM * kRowBytes;           // slab layout
  static constexpr int STAGE_BYTES = (BM + BN) * kRowBytes;
  // More than two stages: a ring of K slabs with the loads STAGES - 1 slabs ahead (gemm_mainloop_ring) -
  // for small tiles whose slab of MFMAs is shorter than the memory latency; one workgroup per CU.
  static constexpr int STAGES = STAGES_;
  // The 256-row direct tiles take STAGES == 3 to mean: token panel in a ring of three stages, weight panel in two
  // (gemm_mainloop_fixed16) - exactly the 160 KB of LDS a CU has.
  static constexpr bool A_RING3 = MFMA16 && STAGES_ == 3;
  static constexpr bool RING = STAGES_ > 2 && !MFMA16;
  static constexpr int LDS_BYTES = A_RING3 ? 3 * A_BYTES + 2 * BN * kRowBytes : STAGES * STAGE_BYTES;
  static_assert(STAGES_ >= 2 && STAGES_ <= 6 && LDS_BYTES <= 160 * 1024, "LDS stages");
  static_assert(STAGES_ == 2 || A_RING3 || (DIRECT_ && BM_ <= 128), "ring: direct path of the small tiles");
  static_assert(WTM % 32 == 0 && WTN_OUT % 32 == 0, "wave tile must be a multiple of 32x32");
  static_assert(NWAVES % 2 == 0, "lane mapping of the slab layout needs an even wave count");
  static_assert((BM / 16) % NWAVES == 0 && (BN / 16) % NWAVES == 0, "panel rows must split evenly over waves");
  static_assert(!DUAL || (BN / 2) % 16 == 0, "gate/up split must fall on a 16-row load group");
  static_assert(!B_KMAJOR || (DIRECT && !DUAL && BN >= 64 && BN <= 512), "K-major weights: direct path, one weight");
};

// Accumulator tile b of the wave reads B-panel rows starting here.
template <class Cfg>
__device__ __forceinline__ int b_frag_row(int wn, int tn) {
  if (Cfg::DUAL) return (tn < Cfg::TN_OUT ? 0 : Cfg::BN / 2) + wn * Cfg::WTN_OUT + (tn % Cfg::TN_OUT) * Cfg::MT;
  return wn * Cfg::WTN_OUT + tn * Cfg::MT;
}

template <class Cfg>
__device__ __forceinline__ void zero_acc(typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN]) {
#pragma unroll
  for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
    for (int j = 0; j < Cfg::TN; ++j)
#pragma unroll
      for (int v = 0; v < Cfg::ACC_N; ++v) acc[i][j][v] = 0.f;
}

// Where element v of an accumulator tile lies: the lane holds token row `lr` of the tile (the MFMA's
// second operand) and, of the tile's weight rows (= output columns), those at acc_col(v, lh):
//   32x32x16: lr = lane & 31, lh = lane >> 5, columns 8 * (v / 4) + 4 * lh + v % 4
//   16x16x32: lr = lane & 15, lh = lane >> 4, columns 4 * lh + v
template <class Cfg>
__device__ __forceinline__ constexpr int acc_col(int v, int lh) {
  return Cfg::MT == 32 ? 8 * (v / 4) + 4 * lh + (v % 4) : 4 * lh + v;
}

constexpr int waitcnt_imm(int vm, int lgkm) {  // gfx9 s_waitcnt encoding, expcnt untouched
  return (vm & 15) | (7 << 4) | ((lgkm & 15) << 8) | ((vm >> 4) << 14);
}

// Wait until at most N of this wave's global->LDS loads are outstanding and all of its LDS reads
// have returned, then barrier.  Written with builtins (not a fence) so that younger loads stay
// in flight across the barrier.
template <int N>
__device__ __forceinline__ void dma_wait_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(N, 0));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// Which 16-byte chunks a lane moves into LDS (both paths).  A panel is moved as 1 KB groups of
// eight 128-byte rows; group id = j * NWAVES + wave; the lane fills physical slot `lane` of its group.
template <class Cfg>
struct TileLanes {
  static constexpr int NJA = Cfg::BM / 8 / Cfg::NWAVES;  // 1 KB (8-row) groups of the A panel per wave
  static constexpr int NJB = Cfg::BN / 8 / Cfg::NWAVES;
  int lane, wave, wm, wn;
  int wave_s;      // the wave index again, held in a scalar register (LDS destinations of the global->LDS loads)
  uint32_t r_in;   // row inside the 8-row group this lane loads
  uint32_t c_log;  // logical 16-byte chunk (0..7) of that row
  uint32_t lr, lh; // MFMA fragment row (0 .. MT-1) and 8-element K piece of the lane (0..1 or 0..3)
  // K-major weight panel: a 64-row slab of BN-element rows is moved as 1 KB groups of 64 / (BN / 8)
  // whole rows; this lane fills physical slot `lane` of its group, which holds logical chunk kb_chunk
  // of row kb_row of the group.
  uint32_t kb_row, kb_chunk;
  static constexpr int KB_CPR = Cfg::BN / 8;    // 16-byte chunks per K-major row
  static constexpr int KB_RPG = 64 / (KB_CPR > 64 ? 64 : KB_CPR);  // rows per 1 KB group

  __device__ __forceinline__ void init() {
    const int tid = threadIdx.x;
    lane = tid & (kWave - 1);
    wave = tid / kWave;
    wave_s = __builtin_amdgcn_readfirstlane(wave);
    wm = wave / Cfg::WAVES_N;
    wn = wave % Cfg::WAVES_N;
    // Group id = j * NWAVES + wave, so the group's parity (which the swizzle needs) is the wave's
    // parity.  lds_swizzle(group * 8 + r_in, c_log) == group * 1024 + lane * 16.
    const uint32_t q = lane & 15;
    r_in = 2 * (lane >> 4) + ((q >> 3) ^ (wave & 1));
    c_log = (q & 7) ^ r_in;
    lr = lane & (Cfg::MT - 1);
    lh = lane / Cfg::MT;
    kb_row = kb_chunk = 0;
    if (Cfg::B_KMAJOR) {
      static_assert(!Cfg::B_KMAJOR || (KB_CPR <= 64 && (KB_RPG == 2 || KB_RPG == 4 || KB_RPG == 8)), "BN of 64, 128 or 256");
      kb_row = lane / KB_CPR;
      const uint32_t c_phys = lane % KB_CPR;
      // kmajor_swizzle_key() of slab row group * KB_RPG + kb_row; the group's parity is the wave's.
      const uint32_t key = KB_RPG == 2 ? 2 * (wave & 1) + kb_row : KB_RPG == 4 ? kb_row : (kb_row >> 1) & 1;
      kb_chunk = (((c_phys >> 2) ^ key) << 2) | (c_phys & 3);
    }
  }
  __device__ __forceinline__ int kb_group_row(int j) const { return (j * Cfg::NWAVES + wave) * KB_RPG + (int)kb_row; }
  __device__ __forceinline__ int group_row(int j) const { return (j * Cfg::NWAVES + wave) * 8; }
  __device__ __forceinline__ int load_row(int j) const { return group_row(j) + (int)r_in; }
};

// =============================================================================================
// Register-staged path: 64-element K slabs, global -> registers -> LDS, double-buffered.  Handles
// any K that is a multiple of 8 (chunks past the end are zero-filled).
// pa[j] / pb[j] point at this lane's chunk of slab 0 for each of its rows.
// =============================================================================================
template <class Cfg>
__device__ __forceinline__ void gemm_mainloop_staged(const TileLanes<Cfg>& tl,
                                                     const uint16_t* const (&pa)[TileLanes<Cfg>::NJA],
                                                     const uint16_t* const (&pb)[TileLanes<Cfg>::NJB], int k_len,
                                                     uint8_t* lds, typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN]) {
  static_assert(!Cfg::MFMA16, "the register-staged loop issues 32x32x16 MFMAs");
  constexpr int NWAVES = Cfg::NWAVES, TM = Cfg::TM, TN = Cfg::TN;
  constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
  const int lane = tl.lane, wave = tl.wave;
  uint8_t* lds0 = lds;
  uint8_t* lds1 = lds + Cfg::STAGE_BYTES;

  uint32_t koff[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) koff[s] = lds_swizzle(tl.lr, 2 * s + tl.lh);
  const uint32_t a_base = (uint32_t)(tl.wm * Cfg::WTM) * kRowBytes;
  uint32_t b_base[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) b_base[tn] = Cfg::A_BYTES + (uint32_t)b_frag_row<Cfg>(tl.wn, tn) * kRowBytes;

  zero_acc<Cfg>(acc);
  const int nk = cdiv(k_len, kBK);

  uint4 ra[NJA], rb[NJB];
  auto load_regs = [&](int kt) {
    // k_len % 8 == 0, so a 16-byte chunk is entirely inside or entirely outside the tail.
    const bool ok = kt * kBK + (int)tl.c_log * 8 + 8 <= k_len;
    const int64_t ko = (int64_t)kt * kBK;
#pragma unroll
    for (int j = 0; j < NJA; ++j)
      ra[j] = ok ? *reinterpret_cast<const uint4*>(pa[j] + ko) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < NJB; ++j)
      rb[j] = ok ? *reinterpret_cast<const uint4*>(pb[j] + ko) : make_uint4(0, 0, 0, 0);
  };
  auto store_regs = [&](uint8_t* stage) {
#pragma unroll
    for (int j = 0; j < NJA; ++j)
      *reinterpret_cast<uint4*>(stage + (j * NWAVES + wave) * 1024 + lane * 16) = ra[j];
#pragma unroll
    for (int j = 0; j < NJB; ++j)
      *reinterpret_cast<uint4*>(stage + Cfg::A_BYTES + (j * NWAVES + wave) * 1024 + lane * 16) = rb[j];
  };
  auto compute = [&](const uint8_t* stage) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      bf16x8_t af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[i] = *reinterpret_cast<const bf16x8_t*>(stage + a_base + i * 32 * kRowBytes + koff[s]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bfr[j] = *reinterpret_cast<const bf16x8_t*>(stage + b_base[j] + koff[s]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
    }
  };

  if (nk <= 0) return;
  load_regs(0);
  store_regs(lds0);
  for (int kt = 0; kt < nk; kt += 2) {
    __syncthreads();
    if (kt + 1 < nk) load_regs(kt + 1);
    compute(lds0);
    if (kt + 1 < nk) {
      store_regs(lds1);
      __syncthreads();
      if (kt + 2 < nk) load_regs(kt + 2);
      compute(lds1);
      if (kt + 2 < nk) store_regs(lds0);
    }
  }
}

// =============================================================================================
// Direct path: two stages of 64-element K slabs filled by buffer_load ... lds; k_len is a positive
// multiple of 64.  Load j of the A panel reads 16 bytes at baseA[j] + offA[j] (+ 128 bytes per
// slab); baseA[j] is uniform over the wave, offA[j] is this lane's 32-bit byte offset.  Likewise
// for B.  Every load instruction moves eight whole 128-byte rows, so each cache line is requested
// once (32-element half slabs cost a twentieth more time at d=4096, h=14336: the kernel runs at
// the board's power limit, and the second request per line is paid for in shader clock).
// One barrier per slab: it sits before the last K step, when every fragment of the current slab
// has been read (its stage can be refilled with the slab after next) and the next slab, issued
// one iteration earlier, has landed (its first fragments are read during the last K step).
// =============================================================================================
template <class Cfg>
__device__ __forceinline__ void gemm_mainloop_slab_dma(const TileLanes<Cfg>& tl,
                                                       const uint16_t* const (&baseA)[TileLanes<Cfg>::NJA],
                                                       const uint32_t (&offA)[TileLanes<Cfg>::NJA],
                                                       const uint16_t* const (&baseB)[TileLanes<Cfg>::NJB],
                                                       const uint32_t (&offB)[TileLanes<Cfg>::NJB], int k_len,
                                                       uint8_t* lds, typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN],
                                                       const KMajorB& kb = KMajorB()) {
  static_assert(!Cfg::MFMA16, "16x16x32 tiles run gemm_mainloop_fixed16");
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int NWAVES = Cfg::NWAVES, TM = Cfg::TM, TN = Cfg::TN;
  constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
  constexpr int L = NJA + NJB;
  constexpr int STAGE = Cfg::STAGE_BYTES, A_BYTES = Cfg::A_BYTES;
  constexpr int NM = TM * TN, ND = TM + TN;
  constexpr int RB = Cfg::BN * 2;  // K-major weight panel: bytes per row
  const int wave = tl.wave_s;  // scalar: the loads' LDS destinations (M0) then need no readfirstlane each

  auto wave_uniform = [](const uint16_t* p) {
    if (!Cfg::DUAL) return reinterpret_cast<void*>(const_cast<uint16_t*>(p));
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<void*>(((uint64_t)hi << 32) | lo);
  };
  __amdgpu_buffer_rsrc_t rsA[NJA], rsB[NJB];
#pragma unroll
  for (int j = 0; j < NJA; ++j) rsA[j] = __builtin_amdgcn_make_buffer_rsrc(wave_uniform(baseA[j]), 0, 0xffffffff, 0x00020000);
  if constexpr (!Cfg::B_KMAJOR) {
#pragma unroll
    for (int j = 0; j < NJB; ++j) rsB[j] = __builtin_amdgcn_make_buffer_rsrc(wave_uniform(baseB[j]), 0, 0xffffffff, 0x00020000);
  }
  // K-major: one base per weight, uniform over the wave; the slab offset goes into the base.
  uint64_t kw[2] = {0, 0};
  if constexpr (Cfg::B_KMAJOR) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      // readfirstlane returns int: take both halves through uint32_t, or the low half sign-extends
      const uint64_t v = reinterpret_cast<uint64_t>(kb.w[q]);
      const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
      const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
      kw[q] = ((uint64_t)hi << 32) | lo;
    }
  }

  uint32_t koff[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) koff[s] = lds_swizzle(tl.lr, 2 * s + tl.lh);
  const uint32_t a_base = (uint32_t)(tl.wm * Cfg::WTM) * kRowBytes;
  uint32_t b_base[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) b_base[tn] = A_BYTES + (uint32_t)b_frag_row<Cfg>(tl.wn, tn) * kRowBytes;
  if constexpr (Cfg::B_KMAJOR) {
    // This lane's 8 bytes of the first transposing read of K step 0: row 8 * lh + (i >> 2) of the slab,
    // columns 16 * (group & 1) + 4 * (i & 3) ... of the accumulator tile's 32 (i = lane & 15).
    const uint32_t i = tl.lane & 15, grp16 = tl.lane >> 4;
    const uint32_t row = 8 * tl.lh + (i >> 2);
    const uint32_t key = kmajor_swizzle_key<Cfg::BN>(row);  // K steps and halves add multiples of 4 rows: same key
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const uint32_t unit = (uint32_t)b_frag_row<Cfg>(tl.wn, tn) / 32;
      b_base[tn] = A_BYTES + row * RB + ((unit ^ key) << 6) + 32 * (grp16 & 1) + 8 * (i & 3);
    }
  }

  zero_acc<Cfg>(acc);
  const int nk = k_len / kBK;

  auto issue_a = [&](int stage, int kt) {
    uint8_t* st = lds + stage * STAGE;
    const int ko = kt * kRowBytes;
#pragma unroll
    for (int j = 0; j < NJA; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA[j], FFNK_LDS_PTR(st + (j * NWAVES + wave) * 1024), 16, offA[j], ko, 0, 0);
  };
  // K-major: the slab's resource (weight and slab offset folded into the base, all scalar).
  auto kmajor_rsrc = [&](int kt) {
    const int ka = kb.kt_first + kt;
    const bool second = ka >= kb.kt_switch;
    const uint64_t base = (second ? kw[1] : kw[0]) + (uint64_t)(uint32_t)(second ? ka - kb.kt_switch : ka) * kb.slab_bytes;
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(base), 0, 0xffffffff, 0x00020000);
  };
  auto issue_b = [&](int stage, int kt) {
    uint8_t* st = lds + stage * STAGE;
    if constexpr (Cfg::B_KMAJOR) {
      const __amdgpu_buffer_rsrc_t rs = kmajor_rsrc(kt);
#pragma unroll
      for (int j = 0; j < NJB; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs, FFNK_LDS_PTR(st + A_BYTES + (j * NWAVES + wave) * 1024), 16, offB[j], 0, 0, 0);
    } else {
      const int ko = kt * kRowBytes;
#pragma unroll
      for (int j = 0; j < NJB; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB[j], FFNK_LDS_PTR(st + A_BYTES + (j * NWAVES + wave) * 1024), 16, offB[j], ko, 0, 0);
    }
  };
  auto issue = [&](int stage, int kt) {
    issue_a(stage, kt);
    issue_b(stage, kt);
  };
  bf16x8_t fa[2][TM], fb[2][TN];
  auto load_frags = [&](int buf, int stage, int s) {
    const uint8_t* st = lds + stage * STAGE;
    // In the order the MFMAs first use them: all weight fragments, then the token fragments.
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[buf][j] = *reinterpret_cast<const bf16x8_t*>(st + b_base[j] + koff[s]);
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[buf][i] = *reinterpret_cast<const bf16x8_t*>(st + a_base + i * 32 * kRowBytes + koff[s]);
  };
  auto mfmas = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[buf][j], fa[buf][i], acc[i][j], 0, 0, 0);
  };

  // ---- K-major weights: the same pipeline written out in source order.  The transposing reads are
  // asm statements, which scheduling hints cannot place, so every K step is a fixed sequence held by
  // scheduling barriers: wait for the step's fragments, then its MFMAs with the next step's LDS
  // reads behind the first ones and (last step of a slab) the global->LDS loads behind the rest. ----
  constexpr int NR = 2 * TN + TM;                        // LDS reads per K step
  constexpr int RSLOTS = NM >= 2 ? NM / 2 : 1;
  constexpr int RPS = (NR + RSLOTS - 1) / RSLOTS;        // reads behind each of the first MFMAs
  constexpr int RUSED = (NR + RPS - 1) / RPS;
  constexpr int DPS = (L + (NM - RUSED) - 1) / (NM - RUSED);  // loads behind each of the other MFMAs
  static_assert(NM > RUSED, "no MFMA left to carry the global->LDS loads");
  bf16x4_t fb_lo[2][TN], fb_hi[2][TN];  // halves of a weight fragment as the two reads deliver them
  uint32_t kaddr[2][TN][2];             // LDS address of this lane's reads: [stage][tile][half] (K step: immediate)
  if constexpr (Cfg::B_KMAJOR) {
    const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>(FFNK_LDS_PTR(lds));
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        kaddr[st][j][0] = lds_addr + st * STAGE + b_base[j];
        kaddr[st][j][1] = kaddr[st][j][0] + 4 * RB;
      }
  }
  // Reads [r0, r1) of K step `step` of the slab in `stage` into fragment buffer `buf`.
  auto kmajor_reads = [&](int buf, int stage, auto step, int r0, int r1) {
    constexpr int ks = decltype(step)::value;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (r < r0 || r >= r1) continue;
      if (r < 2 * TN) {
        const bf16x4_t v = lds_read_tr16_b64<16 * ks * RB>(kaddr[stage][r / 2][r & 1]);
        if (r & 1) fb_hi[buf][r / 2] = v;
        else fb_lo[buf][r / 2] = v;
      } else {
        fa[buf][r - 2 * TN] =
            *reinterpret_cast<const bf16x8_t*>(lds + stage * STAGE + a_base + (r - 2 * TN) * 32 * kRowBytes + koff[ks]);
      }
    }
  };
  auto kmajor_step = [&](int cur, int stage_next, auto step_next, bool reads, bool dma, int stage_dma, int kt_dma) {
    __amdgpu_buffer_rsrc_t rsk = rsA[0];
    if (dma) rsk = kmajor_rsrc(kt_dma);
    kmajor_wait_frags<TN>(fb_lo[cur], fb_hi[cur]);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[cur][j] = __builtin_shufflevector(fb_lo[cur][j], fb_hi[cur][j], 0, 1, 2, 3, 4, 5, 6, 7);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < NM; ++q) {
      acc[q / TN][q % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][q % TN], fa[cur][q / TN], acc[q / TN][q % TN], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (q < RUSED) {
        if (reads) kmajor_reads(cur ^ 1, stage_next, step_next, q * RPS, (q + 1) * RPS);
      } else if (dma) {
        uint8_t* st = lds + stage_dma * STAGE;
#pragma unroll
        for (int l = (q - RUSED) * DPS; l < (q - RUSED + 1) * DPS && l < L; ++l) {
          if (l < NJA)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA[l], FFNK_LDS_PTR(st + (l * NWAVES + wave) * 1024), 16, offA[l],
                                                     kt_dma * kRowBytes, 0, 0);
          else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsk, FFNK_LDS_PTR(st + A_BYTES + ((l - NJA) * NWAVES + wave) * 1024), 16,
                                                     offB[l - NJA], 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Clear rows [last_rows, 64) of the weight panel in `stage` (the range's last slab, after it has landed
  // and before anyone reads it).  Rows are RB contiguous bytes each, whatever the swizzle inside them.
  auto kmajor_clear_tail = [&](int stage) {
    uint8_t* first = lds + stage * STAGE + A_BYTES + kb.last_rows * RB;
    const int bytes = (kBK - kb.last_rows) * RB;
    for (int o = (int)threadIdx.x * 16; o < bytes; o += Cfg::NT * 16) *reinterpret_cast<uint4*>(first + o) = make_uint4(0, 0, 0, 0);
    dma_wait_barrier<0>();
  };
  constexpr std::integral_constant<int, 0> s0{};
  constexpr std::integral_constant<int, 1> s1{};
  constexpr std::integral_constant<int, 2> s2{};
  constexpr std::integral_constant<int, 3> s3{};
  auto kmajor_body = [&](int u, int kt, bool full) {
    kmajor_step(0, u, s1, true, false, 0, 0);
    kmajor_step(1, u, s2, true, false, 0, 0);
    kmajor_step(0, u, s3, true, false, 0, 0);
    dma_wait_barrier<0>();  // every wave has read the last of stage u; the next slab has landed in the other stage
    if (!full && kt + 2 == nk && kb.last_rows < kBK) kmajor_clear_tail(u ^ 1);  // never in the steady loop
    kmajor_step(1, u ^ 1, s0, full || kt + 1 < nk, full || kt + 2 < nk, u, kt + 2);
  };

  // Head of the tile: the weight panels of the first two slabs go out first - their addresses do not
  // depend on the routing - so that they fly while the gathered token rows' indices are still loading.
  issue_b(0, 0);
  if (nk > 1) issue_b(1, 1);
  issue_a(0, 0);
  if (nk > 1) {
    issue_a(1, 1);
    dma_wait_barrier<NJA>();  // in issue order only the token panel of slab 1 may still be under way
  } else {
    dma_wait_barrier<0>();
  }
  if constexpr (Cfg::B_KMAJOR) {
    if (nk == 1 && kb.last_rows < kBK) kmajor_clear_tail(0);
    kmajor_reads(0, 0, s0, 0, NR);
  } else {
    load_frags(0, 0, 0);
  }

  auto body = [&](int u, int kt, bool full) {
    load_frags(1, u, 1);
    mfmas(0);
    load_frags(0, u, 2);
    mfmas(1);
    load_frags(1, u, 3);
    mfmas(0);
    dma_wait_barrier<0>();
    if (full || kt + 2 < nk) issue(u, kt + 2);
    if (full || kt + 1 < nk) load_frags(0, u ^ 1, 0);
    mfmas(1);
    if (full) {
      // One LDS read after each of the first TM+TN MFMAs of a K step; the global->LDS loads
      // of the slab after next follow the barrier, spread over the MFMAs of the last K step.
      constexpr int PER = (L + NM - 1) / NM;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int q = 0; q < NM; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (q < ND) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          if (ks == 3 && q * PER < L) __builtin_amdgcn_sched_group_barrier(0x020, PER, 0);
        }
    }
  };
  int k0 = 0;
  if constexpr (Cfg::B_KMAJOR) {
    for (; k0 + 3 < nk; k0 += 2) {
      kmajor_body(0, k0, true);
      kmajor_body(1, k0 + 1, true);
    }
    for (; k0 < nk; k0 += 2) {
      kmajor_body(0, k0, false);
      if (k0 + 1 < nk) kmajor_body(1, k0 + 1, false);
    }
  } else {
    for (; k0 + 3 < nk; k0 += 2) {  // every guard inside is true: no branches
      body(0, k0, true);
      body(1, k0 + 1, true);
    }
    for (; k0 < nk; k0 += 2) {
      body(0, k0, false);
      if (k0 + 1 < nk) body(1, k0 + 1, false);
    }
  }
#endif
}

// =============================================================================================
// Direct path of the 256-row tiles: 64-element slabs accumulated with v_mfma_f32_16x16x32_bf16 in a schedule
// written out in source order (every MFMA fenced by scheduling barriers), because with one or two wavefronts
// per SIMD nothing else hides a wait, and an instruction that cannot issue - a load while the address unit's
// queue is full - holds back the MFMAs behind it.
//  * A slab is two K steps of 32.  A step runs its TM x TN MFMAs row group by row group: the token
//    fragment of a group (16 rows x 32 K) is single-buffered and re-read in place for the next step as
//    soon as the group's last MFMA has issued (a whole step ahead of its next use); the TN weight
//    fragments are double-buffered and read during the previous step, one behind the middle MFMA of each row group.
//  * Two barriers per slab, both in its second step.  The release barrier, behind the step's first four
//    MFMAs: the stage's last fragment reads were issued at the end of the first step and have returned
//    (lgkmcnt only), so the stage is free for the slab after next.  The data barrier, behind the first two
//    row groups: the next slab has landed (vmcnt leaves the loads issued since in flight).  One barrier doing
//    both jobs started the loads twelve MFMAs later (1-3 % slower; the waves run in step, a barrier by itself
//    measures nothing).
//  * The global->LDS loads go out no faster than the address unit takes them, one 1 KB load per wave
//    behind every fourth or fifth MFMA (16 cycles per load and CU), not in a burst behind the barrier.
//  * Two LDS layouts.  Two stages of (token panel, weight panel): the first loads of the slab after next go
//    out through the rest of the second step, the others during the first step of the following slab - the
//    last of them 61 MFMAs ahead of the data barrier that waits for them.  Cfg::A_RING3 (all 160 KB of LDS):
//    three token stages and two weight stages; the token stage that slab kt + 2 will use was released a slab
//    ago, so its loads go out during slab kt's first step and only the weight panel's wait for the release
//    barrier - every load is at least 100 MFMAs ahead of its data barrier.  Cycle stamps around the barriers
//    (s_memtime, one lane per workgroup) put the data barrier of the two-stage form at 120 cycles per slab on
//    the SwiGLU GEMM (K = 4096) and at 270 of 2 700 on the down projection (K = 14336), whose panels miss L2
//    more often; the ring takes the down projection from 2.66 to 2.55 ms and leaves the SwiGLU GEMM where it was.
//  * K-major weight panels (Cfg::B_KMAJOR, see KMajorB): the same schedule; a weight fragment is two transposing
//    reads, issued as asm statements in the slot where the row-major form issues its one read, and every K step
//    starts with an s_waitcnt lgkmcnt(n) that leaves outstanding only the token reads issued behind the last of
//    them.  The range's last slab may be ragged: its surplus rows are cleared behind the data barrier that
//    announces it (tail of the loop only).
// =============================================================================================
template <class Cfg>
__device__ __forceinline__ void gemm_mainloop_fixed16(const TileLanes<Cfg>& tl,
                                                      const uint16_t* const (&baseA)[TileLanes<Cfg>::NJA],
                                                      const uint32_t (&offA)[TileLanes<Cfg>::NJA],
                                                      const uint16_t* const (&baseB)[TileLanes<Cfg>::NJB],
                                                      const uint32_t (&offB)[TileLanes<Cfg>::NJB], int k_len,
                                                      uint8_t* lds, typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN],
                                                      const KMajorB& kb = KMajorB()) {
  static_assert(Cfg::MFMA16 && Cfg::DIRECT, "16x16x32 schedule of the direct 256-row tiles");
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int NWAVES = Cfg::NWAVES, TM = Cfg::TM, TN = Cfg::TN;
  constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
  constexpr int L = NJA + NJB;
  constexpr int A_BYTES = Cfg::A_BYTES, B_BYTES = Cfg::BN * kRowBytes;
  constexpr int NM = TM * TN;
  constexpr int BAR = 2 * TN;            // MFMAs of a slab's second step ahead of the data barrier (two row groups)
  constexpr int RPOS = 4;                // ... ahead of the release barrier
  // Token panel in a ring of three stages: slab kt's token rows sit in stage kt % 3, its weight rows in stage kt % 2.
  constexpr bool R3 = Cfg::A_RING3;
  constexpr bool KM = Cfg::B_KMAJOR;     // weight panel stored K-major: fragments come from transposing reads (see KMajorB)
  constexpr int RB = Cfg::BN * 2;        // ... bytes of one of its 64 rows
  // One load per wave behind every LEV-th MFMA.  One per four MFMAs is the address unit's own rate (16 cycles per
  // load and CU).  The four-wave tiles measure faster a notch slower (SwiGLU tile 3 %, down projection 2.4 %, the
  // gathered single-weight GEMM the same either way), the eight-wave tile 1-4 % slower; six is no better than five.
  constexpr int LEV = NWAVES == 4 ? 5 : 4;
  // Two-stage form: loads of the slab after next that go out in the second step (the rest follow in the next slab's first).
  constexpr int L1 = R3 ? NJB : ((NM - RPOS) / LEV < L ? (NM - RPOS) / LEV : L);
  constexpr int NPRE = (BAR - RPOS) / LEV;  // ... of them ahead of the data barrier (a load follows the last MFMA of its group of LEV)
  static_assert(RPOS >= 0 && RPOS < BAR && NPRE <= L1, "release barrier ahead of the data barrier");
  static_assert(TM >= 3 && TM >= TN && L1 >= 1 && L1 <= L && (L - L1) * LEV <= NM, "schedule does not fit this wave tile");
  static_assert(!R3 || (NJA * LEV <= NM && RPOS + NJB * LEV <= NM), "ring schedule does not fit this wave tile");
  const int wave = tl.wave_s;

  auto wave_uniform = [](const uint16_t* p) {
    if (!Cfg::DUAL) return reinterpret_cast<void*>(const_cast<uint16_t*>(p));
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<void*>(((uint64_t)hi << 32) | lo);
  };
  __amdgpu_buffer_rsrc_t rsA[NJA], rsB[NJB];
#pragma unroll
  for (int j = 0; j < NJA; ++j) rsA[j] = __builtin_amdgcn_make_buffer_rsrc(wave_uniform(baseA[j]), 0, 0xffffffff, 0x00020000);
#pragma unroll
  for (int j = 0; j < NJB; ++j) rsB[j] = __builtin_amdgcn_make_buffer_rsrc(wave_uniform(baseB[j]), 0, 0xffffffff, 0x00020000);
  // K-major: one base per weight, uniform over the wave; a slab's offset goes into its resource (all scalar).
  uint64_t kw[2] = {0, 0};
  if constexpr (KM) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const uint64_t v = reinterpret_cast<uint64_t>(kb.w[i]);
      const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
      const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
      kw[i] = ((uint64_t)hi << 32) | lo;
    }
  }
  auto kmajor_rsrc = [&](int kt) {
    const int ka = kb.kt_first + kt;
    const bool second = ka >= kb.kt_switch;
    const uint64_t base = (second ? kw[1] : kw[0]) + (uint64_t)(uint32_t)(second ? ka - kb.kt_switch : ka) * kb.slab_bytes;
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(base), 0, 0xffffffff, 0x00020000);
  };

  // LDS layout.  Two stages: stage s holds a slab's token panel, then its weight panel.  Ring: three token panels,
  // then two weight panels.  Token stages are named by their byte offset (a run-time value in the ring form).
  auto a_stage = [](int s) { return R3 ? s * A_BYTES : s * Cfg::STAGE_BYTES; };
  auto b_stage = [](int t) { return R3 ? 3 * A_BYTES + t * B_BYTES : t * Cfg::STAGE_BYTES + A_BYTES; };
  // Fragment of K step s: tile row lr, logical 16-byte chunks 4 s + lh (lh = 0..3: 8 K elements each).
  uint32_t koff[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) koff[s] = lds_swizzle(tl.lr, 4 * s + tl.lh);
  const uint32_t a_base = (uint32_t)(tl.wm * Cfg::WTM) * kRowBytes;
  uint32_t b_base[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) b_base[tn] = (uint32_t)b_frag_row<Cfg>(tl.wn, tn) * kRowBytes;
  if constexpr (KM) {
    // This lane's 8 bytes of the first transposing read of K step 0: row 8 * lh + (i >> 2) of the slab (lh = 0..3: the
    // lane's 8-row K run), columns 4 * (i & 3) ... of the accumulator tile's 16 (i = lane & 15); the second read of a
    // fragment lies four rows on, the second K step 32 rows on (immediate offsets; the swizzle key repeats every 4 rows).
    const uint32_t i = tl.lane & 15;
    const uint32_t row = 8 * tl.lh + (i >> 2);
    const uint32_t key = kmajor_swizzle_key<Cfg::BN>(row);
    const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>(FFNK_LDS_PTR(lds));
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const uint32_t col = (uint32_t)b_frag_row<Cfg>(tl.wn, tn);  // first of the tile's 16 columns
      b_base[tn] = lds_addr + row * RB + (((col / 32) ^ key) << 6) + 32 * ((col / 16) & 1) + 8 * (i & 3);
    }
  }

  zero_acc<Cfg>(acc);
  const int nk = k_len / kBK;

  bf16x8_t fa[TM], fb[2][TN];
  bf16x4_t fb_lo[2][TN], fb_hi[2][TN];  // K-major: halves of a weight fragment as the two transposing reads deliver them
  auto read_a = [&](int i, int a_off, int ks) {
    fa[i] = *reinterpret_cast<const bf16x8_t*>(lds + a_off + a_base + i * 16 * kRowBytes + koff[ks]);
  };
  auto read_b = [&](int buf, int j, int b_off, int ks) {
    if constexpr (KM) {
      // asm statements (see lds_read_tr16_b64): the compiler does not know that they are LDS reads, wait_b() stands
      // between them and the first use
      if (ks == 0) {
        fb_lo[buf][j] = lds_read_tr16_b64<0>(b_base[j] + b_off);
        fb_hi[buf][j] = lds_read_tr16_b64<4 * RB>(b_base[j] + b_off);
      } else {
        fb_lo[buf][j] = lds_read_tr16_b64<32 * RB>(b_base[j] + b_off);
        fb_hi[buf][j] = lds_read_tr16_b64<36 * RB>(b_base[j] + b_off);
      }
    } else {
      fb[buf][j] = *reinterpret_cast<const bf16x8_t*>(lds + b_off + b_base[j] + koff[ks]);
    }
  };
  // K-major: wait until at most `younger` LDS operations of this wave are outstanding - LDS operations return in
  // order, so that covers every transposing read issued before the last `younger` ones - and assemble the weight
  // fragments of buffer `buf`.  The compiler's own waits for the token fragments count only the reads it knows, i.e.
  // they ask for no less than is needed.
  auto wait_b = [&](int buf, auto younger) {
    if constexpr (KM) {
      constexpr int imm = waitcnt_imm(63, decltype(younger)::value);
      static_assert(TN == 4 || TN == 8, "weight fragments per K step");
      if constexpr (TN == 4)
        asm volatile("s_waitcnt %8"
                     : "+v"(fb_lo[buf][0]), "+v"(fb_hi[buf][0]), "+v"(fb_lo[buf][1]), "+v"(fb_hi[buf][1]), "+v"(fb_lo[buf][2]),
                       "+v"(fb_hi[buf][2]), "+v"(fb_lo[buf][3]), "+v"(fb_hi[buf][3])
                     : "n"(imm));
      else
        asm volatile("s_waitcnt %16"
                     : "+v"(fb_lo[buf][0]), "+v"(fb_hi[buf][0]), "+v"(fb_lo[buf][1]), "+v"(fb_hi[buf][1]), "+v"(fb_lo[buf][2]),
                       "+v"(fb_hi[buf][2]), "+v"(fb_lo[buf][3]), "+v"(fb_hi[buf][3]), "+v"(fb_lo[buf][4]), "+v"(fb_hi[buf][4]),
                       "+v"(fb_lo[buf][5]), "+v"(fb_hi[buf][5]), "+v"(fb_lo[buf][6]), "+v"(fb_hi[buf][6]), "+v"(fb_lo[buf][7]),
                       "+v"(fb_hi[buf][7])
                     : "n"(imm));
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[buf][j] = __builtin_shufflevector(fb_lo[buf][j], fb_hi[buf][j], 0, 1, 2, 3, 4, 5, 6, 7);
    }
  };
  auto load_b = [&](int l, int b_off, int kt) {
    if constexpr (KM)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(kmajor_rsrc(kt), FFNK_LDS_PTR(lds + b_off + (l * NWAVES + wave) * 1024), 16,
                                               offB[l], 0, 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB[l], FFNK_LDS_PTR(lds + b_off + (l * NWAVES + wave) * 1024), 16, offB[l],
                                               kt * kRowBytes, 0, 0);
  };
  // K-major: clear rows [last_rows, 64) of the weight panel at b_off (the range's last slab, after it has landed and
  // before anyone reads it).  Rows are RB contiguous bytes each, whatever the swizzle inside them.
  auto clear_tail = [&](int b_off) {
    uint8_t* first = lds + b_off + kb.last_rows * RB;
    const int bytes = (kBK - kb.last_rows) * RB;
    for (int o = (int)threadIdx.x * 16; o < bytes; o += Cfg::NT * 16) *reinterpret_cast<uint4*>(first + o) = make_uint4(0, 0, 0, 0);
    dma_wait_barrier<0>();
  };
  auto load_a = [&](int l, int a_off, int kt) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA[l], FFNK_LDS_PTR(lds + a_off + (l * NWAVES + wave) * 1024), 16, offA[l],
                                             kt * kRowBytes, 0, Cfg::AUX_A);
  };
  // Two-stage form: load l of a slab - the weight panel's first, then the token panel's - into stage t.
  auto load = [&](int l, int t, int kt) {
    if (l < NJB) load_b(l, b_stage(t), kt);
    else load_a(l - NJB, a_stage(t), kt);
  };
  // Four-wave tiles hold 256 accumulator registers per lane, which only fit the accumulation half of the
  // register file.  Left to the builtin, the compiler keeps part of them in ordinary registers and moves
  // them back and forth inside the loop (v_accvgpr_read/write around every other MFMA); the asm form
  // pins each accumulator tile to the accumulation registers for the whole loop.
  constexpr bool kAccPinned = NWAVES == 4;
  auto mfma = [&](int buf, int m) {
    const int i = m / TN, j = m % TN;
    if constexpr (kAccPinned)
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fb[buf][j]), "v"(fa[i]));
    else
      acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[buf][j], fa[i], acc[i][j], 0, 0, 0);
  };
  // First K step of slab kt (weight stage u, token stage at a_cur): behind its MFMAs the fragments of the second
  // step, and loads: the last ones of slab kt + 1 (two-stage form), or the token panel of slab kt + 2 into the ring
  // stage at a_ld.
  // The waves leave every barrier together and run the same instructions, so a fragment read that follows the same
  // MFMA in all of them is four 1 KB requests at once against an LDS that moves 128 bytes per cycle
  // (SQ_LDS_CMD_FIFO_FULL counted the waves stalled at issue): the reads are spread over the whole step instead of
  // following the step's first MFMAs in a row (+0.5 %).  Giving each wave its own load slot within a group of LEV
  // MFMAs (one copy of the loop per wave) or holding wave w back by 16 w cycles behind the barrier measured -0.4 %
  // and -3 %: the address unit's FIFO is not filled by the waves' coincidence.
  // K-major: LDS reads that a step issues in slots strictly behind the slot of its last weight-fragment read (the
  // bound wait_b() may leave outstanding at the start of the next step).
  constexpr int G0 = BAR / TN;                        // second step: row groups ahead of the data barrier
  constexpr int BSTEP = (NM - BAR - 2 * G0 - 2) / TN; // ... spacing of the weight-fragment reads behind it
  static_assert(BSTEP >= 1, "no room for the weight fragments behind the barrier");
  constexpr int kYoungerStep0 = TM - TN + 1;          // first step: the token reads of row groups TN - 1 ... TM - 1
  constexpr int kLastB1 = BAR + 2 * G0 + (TN - 1) * BSTEP;
  constexpr int kYoungerStep1 = TM - (kLastB1 + 1) / TN;  // second step: row groups whose last MFMA lies behind slot kLastB1
  static_assert(kYoungerStep0 >= 0 && kYoungerStep1 >= 0 && kYoungerStep0 < 16 && kYoungerStep1 < 16, "lgkmcnt is four bits");
  auto step0 = [&](int u, int a_cur, int a_ld, int kt, bool next, bool next2) {
    wait_b(0, std::integral_constant<int, kYoungerStep1>{});
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      mfma(0, m);
      __builtin_amdgcn_sched_barrier(0);
      if (m % TN == TN / 2 - 1 && m / TN < TN) read_b(1, m / TN, b_stage(u), 1);   // one per row group
      if (m % TN == TN - 1) read_a(m / TN, a_cur, 1);
      if constexpr (R3) {
        if (m % LEV == LEV - 1 && m / LEV < NJA && next2) load_a(m / LEV, a_ld, kt + 2);
      } else {
        if (L1 + m / LEV < L && m % LEV == LEV - 1 && next) load(L1 + m / LEV, u ^ 1, kt + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Second K step: two row groups, the barriers, then behind the MFMAs the first-step fragments of slab kt + 1
  // (weight stage u ^ 1, token stage at a_nxt) and loads of slab kt + 2 into the stage the release barrier freed:
  // its first L1 loads (two-stage form) or its weight panel (ring form).
  auto step1 = [&](int u, int a_nxt, int kt, bool next, bool next2) {
    wait_b(1, std::integral_constant<int, kYoungerStep0>{});
    __builtin_amdgcn_sched_barrier(0);
    // Behind the barrier: the first-step fragments of slab kt + 1.  Token fragments of the row groups that ran
    // ahead of the barrier first, then one weight fragment every BSTEP MFMAs (the last one lands a dozen
    // MFMAs before its first use), token fragments of the other groups as their last MFMA issues.
#pragma unroll
    for (int m = 0; m < NM; ++m) {
      if (m == RPOS) {
        dma_wait_barrier<63>();  // every wave's reads of stage u have returned: the stage is free for slab kt + 2
        __builtin_amdgcn_sched_barrier(0);
      }
      if (m == BAR) {
        // slab kt + 1 has landed; the loads of slab kt + 2 issued since stay in flight
        if (next2) dma_wait_barrier<(R3 ? NJA : 0) + NPRE>();
        else dma_wait_barrier<0>();
        if constexpr (KM) {
          if (next && !next2 && kb.last_rows < kBK) clear_tail(b_stage(u ^ 1));  // slab kt + 1 is the last: never in the steady loop
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      mfma(1, m);
      __builtin_amdgcn_sched_barrier(0);
      if (next) {
        if (m >= BAR && m < BAR + 2 * G0 && (m - BAR) % 2 == 0) read_a((m - BAR) / 2, a_nxt, 0);
        if (m >= BAR + 2 * G0 && (m - BAR - 2 * G0) % BSTEP == 0 && (m - BAR - 2 * G0) / BSTEP < TN)
          read_b(0, (m - BAR - 2 * G0) / BSTEP, b_stage(u ^ 1), 0);
        if (m / TN >= G0 && m % TN == TN - 1) read_a(m / TN, a_nxt, 0);
      }
      if (m >= RPOS && (m - RPOS) % LEV == LEV - 1 && (m - RPOS) / LEV < L1 && next2) {
        if constexpr (R3) load_b((m - RPOS) / LEV, b_stage(u), kt + 2);
        else load((m - RPOS) / LEV, u, kt + 2);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Head of the tile: slab 0 whole and, of slab 1, what the steady schedule would have issued by now: all of it in
  // the ring form, its first L1 loads in the two-stage form.
#pragma unroll
  for (int l = 0; l < L; ++l) load(l, 0, 0);
  if (nk > 1) {
    if constexpr (R3) {  // token panel first, as the steady schedule issues them
#pragma unroll
      for (int l = 0; l < NJA; ++l) load_a(l, a_stage(1), 1);
#pragma unroll
      for (int l = 0; l < NJB; ++l) load_b(l, b_stage(1), 1);
      dma_wait_barrier<L>();
    } else {
#pragma unroll
      for (int l = 0; l < L1; ++l) load(l, 1, 1);
      dma_wait_barrier<L1>();
    }
  } else {
    dma_wait_barrier<0>();
  }
  if constexpr (KM) {
    if (nk == 1 && kb.last_rows < kBK) clear_tail(b_stage(0));
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) read_b(0, j, b_stage(0), 0);
#pragma unroll
  for (int i = 0; i < TM; ++i) read_a(i, a_stage(0), 0);

  int k0 = 0;
  if constexpr (R3) {
    // token stages of slabs k0, k0 + 1, k0 + 2 (byte offsets), rotated once per slab
    int s0 = a_stage(0), s1 = a_stage(1), s2 = a_stage(2);
    // slab kt with its weight panel in stage u
    auto slab = [&](int u, int kt, bool next, bool next2) {
      step0(u, s0, s2, kt, next, next2);
      step1(u, s1, kt, next, next2);
      const int t = s0;
      s0 = s1;
      s1 = s2;
      s2 = t;
    };
    for (; k0 + 3 < nk; k0 += 2) {  // every guard inside is true: no branches
      slab(0, k0, true, true);
      slab(1, k0 + 1, true, true);
    }
    for (; k0 < nk; k0 += 2) {
      slab(0, k0, k0 + 1 < nk, k0 + 2 < nk);
      if (k0 + 1 < nk) slab(1, k0 + 1, k0 + 2 < nk, k0 + 3 < nk);
    }
  } else {
    auto slab = [&](int u, int kt, bool next, bool next2) {
      step0(u, a_stage(u), 0, kt, next, next2);
      step1(u, a_stage(u ^ 1), kt, next, next2);
    };
    for (; k0 + 3 < nk; k0 += 2) {  // every guard inside is true: no branches
      slab(0, k0, true, true);
      slab(1, k0 + 1, true, true);
    }
    for (; k0 < nk; k0 += 2) {
      slab(0, k0, k0 + 1 < nk, k0 + 2 < nk);
      if (k0 + 1 < nk) slab(1, k0 + 1, k0 + 2 < nk, k0 + 3 < nk);
    }
  }
  // The compiler does not see that the asm statements are matrix instructions: give the last of them the
  // wait states a read of its result by an ordinary instruction needs.
  if constexpr (kAccPinned) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#endif
}

// s_waitcnt vmcnt(n) lgkmcnt(0) + s_barrier for a run-time n (the counter is an immediate).
__device__ __forceinline__ void dma_wait_barrier_n(int n) {
  switch (n) {
#define FFNK_WB(N) case N: dma_wait_barrier<N>(); break;
    FFNK_WB(0) FFNK_WB(1) FFNK_WB(2) FFNK_WB(3) FFNK_WB(4) FFNK_WB(5) FFNK_WB(6) FFNK_WB(7) FFNK_WB(8) FFNK_WB(9)
    FFNK_WB(10) FFNK_WB(11) FFNK_WB(12) FFNK_WB(13) FFNK_WB(14) FFNK_WB(15) FFNK_WB(16) FFNK_WB(17) FFNK_WB(18)
    FFNK_WB(19) FFNK_WB(20) FFNK_WB(21) FFNK_WB(22) FFNK_WB(23) FFNK_WB(24) FFNK_WB(25) FFNK_WB(26) FFNK_WB(27)
    FFNK_WB(28) FFNK_WB(29) FFNK_WB(30) FFNK_WB(31) FFNK_WB(32) FFNK_WB(33) FFNK_WB(34) FFNK_WB(35) FFNK_WB(36)
#undef FFNK_WB
    default: dma_wait_barrier<0>(); break;
  }
}

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// =============================================================================================
// Ring of S > 2 stages for the small tiles (32x32x16 MFMAs).  A 128x128 tile's slab is 512 cycles of
// MFMAs per wave, less than the latency of the loads that feed the next one: behind two stages the K loop
// runs at the memory latency (0.8 us per slab measured against 0.3 us of MFMAs).  Here slab kt + S - 1 is
// loaded while slab kt is computed: its first quarter of loads goes out behind the last K step of slab
// kt - 1 (right after the barrier that frees its stage), the other three quarters behind the first three
// K steps of slab kt - at most one load per MFMA, which is what the address unit takes.  One barrier per
// slab, before its last K step: every wave has read the last fragments of the stage before, and slab
// kt + 1 has landed (loads complete in order, so "at most (S - 2) slabs of loads outstanding").  Same
// source-order schedule as the 256-row tiles.
// =============================================================================================
template <class Cfg>
__device__ __forceinline__ void gemm_mainloop_ring(const TileLanes<Cfg>& tl,
                                                   const uint16_t* const (&baseA)[TileLanes<Cfg>::NJA],
                                                   const uint32_t (&offA)[TileLanes<Cfg>::NJA],
                                                   const uint16_t* const (&baseB)[TileLanes<Cfg>::NJB],
                                                   const uint32_t (&offB)[TileLanes<Cfg>::NJB], int k_len,
                                                   uint8_t* lds, typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN],
                                                   const KMajorB& kb = KMajorB()) {
  static_assert(Cfg::RING && !Cfg::MFMA16, "ring schedule of the small direct tiles");
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int NWAVES = Cfg::NWAVES, TM = Cfg::TM, TN = Cfg::TN, S = Cfg::STAGES, D = S - 1;
  constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
  constexpr int L = NJA + NJB;
  constexpr int STAGE = Cfg::STAGE_BYTES, A_BYTES = Cfg::A_BYTES;
  constexpr bool KM = Cfg::B_KMAJOR;     // weight panel read in place as [K, N] rows: two transposing reads per fragment
  constexpr int RB = Cfg::BN * 2;        // ... whose rows are this many bytes
  constexpr int NM = TM * TN, ND = TM + (KM ? 2 * TN : TN);
  constexpr int LQ = (L + 3) / 4;            // loads per K step (a slab's loads go out over four steps)
  constexpr int RPM = (ND + NM - 1) / NM;    // fragment reads behind each MFMA
  constexpr int LPM = (LQ + NM - 1) / NM;    // loads behind each MFMA
  static_assert((S - 1) * L + LQ <= 36, "dma_wait_barrier_n covers this many loads");
  const int wave = tl.wave_s;

  auto wave_uniform = [](const uint16_t* p) {
    if (!Cfg::DUAL) return reinterpret_cast<void*>(const_cast<uint16_t*>(p));
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<void*>(((uint64_t)hi << 32) | lo);
  };
  __amdgpu_buffer_rsrc_t rsA[NJA], rsB[NJB];
#pragma unroll
  for (int j = 0; j < NJA; ++j) rsA[j] = __builtin_amdgcn_make_buffer_rsrc(wave_uniform(baseA[j]), 0, 0xffffffff, 0x00020000);
  if constexpr (!KM) {
#pragma unroll
    for (int j = 0; j < NJB; ++j) rsB[j] = __builtin_amdgcn_make_buffer_rsrc(wave_uniform(baseB[j]), 0, 0xffffffff, 0x00020000);
  }
  // K-major: one base per weight, uniform over the wave; a slab's offset goes into its resource (see gemm_mainloop_slab_dma).
  uint64_t kw[2] = {0, 0};
  if constexpr (KM) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const uint64_t v = reinterpret_cast<uint64_t>(kb.w[q]);
      const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
      const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
      kw[q] = ((uint64_t)hi << 32) | lo;
    }
  }
  auto kmajor_rsrc = [&](int kt) {
    const int ka = kb.kt_first + kt;
    const bool second = ka >= kb.kt_switch;
    const uint64_t base = (second ? kw[1] : kw[0]) + (uint64_t)(uint32_t)(second ? ka - kb.kt_switch : ka) * kb.slab_bytes;
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(base), 0, 0xffffffff, 0x00020000);
  };
  uint32_t koff[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) koff[s] = lds_swizzle(tl.lr, 2 * s + tl.lh);
  const uint32_t a_base = (uint32_t)(tl.wm * Cfg::WTM) * kRowBytes;
  uint32_t b_base[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) b_base[tn] = A_BYTES + (uint32_t)b_frag_row<Cfg>(tl.wn, tn) * kRowBytes;
  uint32_t kaddr[KM ? S : 1][TN][2];  // K-major: LDS address of this lane's two transposing reads per stage and tile (K step: immediate)
  if constexpr (KM) {
    // As in gemm_mainloop_slab_dma: row 8 * lh + (i >> 2) of the slab, columns 16 * (group & 1) + 4 * (i & 3) ... of the tile's 32.
    const uint32_t i = tl.lane & 15, grp16 = tl.lane >> 4;
    const uint32_t row = 8 * tl.lh + (i >> 2);
    const uint32_t key = kmajor_swizzle_key<Cfg::BN>(row);
    const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>(FFNK_LDS_PTR(lds));
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const uint32_t unit = (uint32_t)b_frag_row<Cfg>(tl.wn, tn) / 32;
      const uint32_t in_stage = A_BYTES + row * RB + ((unit ^ key) << 6) + 32 * (grp16 & 1) + 8 * (i & 3);
#pragma unroll
      for (int st = 0; st < S; ++st) {
        kaddr[st][tn][0] = lds_addr + st * STAGE + in_stage;
        kaddr[st][tn][1] = kaddr[st][tn][0] + 4 * RB;
      }
    }
  }

  zero_acc<Cfg>(acc);
  const int nk = k_len / kBK;

  bf16x8_t fa[2][TM], fb[2][TN];
  bf16x4_t fb_lo[2][TN], fb_hi[2][TN];  // K-major: halves of a weight fragment as the two reads deliver them
  // Fragment read r of K step ks: the weight fragments first (K-major: two reads each), then the token fragments.
  auto read_frag = [&](int buf, int stage, auto ks_tag, int r) {
    constexpr int ks = decltype(ks_tag)::value;
    const uint8_t* st = lds + stage * STAGE;
    if constexpr (KM) {
      if (r < 2 * TN) {
        const bf16x4_t v = lds_read_tr16_b64<16 * ks * RB>(kaddr[stage][r / 2][r & 1]);
        if (r & 1) fb_hi[buf][r / 2] = v;
        else fb_lo[buf][r / 2] = v;
      } else {
        fa[buf][r - 2 * TN] = *reinterpret_cast<const bf16x8_t*>(st + a_base + (r - 2 * TN) * 32 * kRowBytes + koff[ks]);
      }
    } else {
      if (r < TN) fb[buf][r] = *reinterpret_cast<const bf16x8_t*>(st + b_base[r] + koff[ks]);
      else fa[buf][r - TN] = *reinterpret_cast<const bf16x8_t*>(st + a_base + (r - TN) * 32 * kRowBytes + koff[ks]);
    }
  };
  // K-major: the transposing reads are asm statements whose results the compiler does not wait for.
  auto frags_ready = [&](int buf) {
    if constexpr (KM) {
      kmajor_wait_frags<TN>(fb_lo[buf], fb_hi[buf]);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[buf][j] = __builtin_shufflevector(fb_lo[buf][j], fb_hi[buf][j], 0, 1, 2, 3, 4, 5, 6, 7);
    }
  };
  auto load = [&](int l, int stage, int kt) {
    uint8_t* st = lds + stage * STAGE;
    const int ko = kt * kRowBytes;
    if (l < NJB) {
      if constexpr (KM)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(kmajor_rsrc(kt), FFNK_LDS_PTR(st + A_BYTES + (l * NWAVES + wave) * 1024), 16, offB[l],
                                                 0, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsB[l], FFNK_LDS_PTR(st + A_BYTES + (l * NWAVES + wave) * 1024), 16, offB[l], ko, 0, 0);
    } else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA[l - NJB], FFNK_LDS_PTR(st + ((l - NJB) * NWAVES + wave) * 1024), 16,
                                               offA[l - NJB], ko, 0, Cfg::AUX_A);
  };
  // One K step: the MFMAs on fragment buffer `cur`; behind them the fragment reads of (stage_next, ks_next)
  // into the other buffer and loads [l0, l0 + LQ) of slab kt_dma into stage_dma.
  auto step = [&](int cur, int stage_next, auto ks_next, bool reads, bool dma, int l0, int stage_dma, int kt_dma) {
    frags_ready(cur);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < NM; ++q) {
      acc[q / TN][q % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][q % TN], fa[cur][q / TN], acc[q / TN][q % TN], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int r = q * RPM; r < (q + 1) * RPM && r < ND; ++r)
        if (reads) read_frag(cur ^ 1, stage_next, ks_next, r);
#pragma unroll
      for (int i = q * LPM; i < (q + 1) * LPM && i < LQ; ++i)
        if (dma && l0 + i < L) load(l0 + i, stage_dma, kt_dma);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Slab kt in stage U.  On entry slabs up to kt + D - 1 are issued, and the first quarter of slab kt + D.
  auto body = [&](auto stage_tag, int kt, bool steady) {
    constexpr int U = decltype(stage_tag)::value, UN = (U + 1) % S, UP = (U + S - 1) % S;
    const bool far = steady || kt + D < nk;        // slab kt + D exists
    constexpr std::integral_constant<int, 0> k0{};
    constexpr std::integral_constant<int, 1> k1{};
    constexpr std::integral_constant<int, 2> k2{};
    constexpr std::integral_constant<int, 3> k3{};
    step(0, U, k1, true, far, LQ, UP, kt + D);
    step(1, U, k2, true, far, 2 * LQ, UP, kt + D);
    step(0, U, k3, true, far, 3 * LQ, UP, kt + D);
    if (steady) {
      dma_wait_barrier<(S - 2) * L>();
    } else {
      const int last = kt + D < nk ? kt + D : nk - 1;  // last slab issued so far
      dma_wait_barrier_n(last > kt + 1 ? (last - kt - 1) * L : 0);
    }
    step(1, UN, k0, steady || kt + 1 < nk, steady || kt + S < nk, 0, U, kt + S);
  };

  // Head of the tile: slabs 0 .. D - 1 whole and the first quarter of slab D, as the steady schedule leaves them.
  int issued = 0;
#pragma unroll
  for (int j = 0; j < D; ++j)
    if (j < nk) {
#pragma unroll
      for (int l = 0; l < L; ++l) load(l, j, j);
      issued += L;
    }
  if (D < nk) {
#pragma unroll
    for (int l = 0; l < LQ && l < L; ++l) load(l, D % S, D);
    issued += LQ < L ? LQ : L;
  }
  dma_wait_barrier_n(issued - L);  // slab 0 has landed
#pragma unroll
  for (int r = 0; r < ND; ++r) read_frag(0, 0, std::integral_constant<int, 0>{}, r);

  int kt = 0;
  for (; kt + 2 * S - 1 < nk; kt += S) static_for<0, S>([&](auto u) { body(u, kt + decltype(u)::value, true); });
  for (; kt < nk; kt += S)
    static_for<0, S>([&](auto u) {
      if (kt + decltype(u)::value < nk) body(u, kt + decltype(u)::value, false);
    });
#endif
}

// Main loop of a direct-path tile, by the tile's MFMA shape.
template <class Cfg>
__device__ __forceinline__ void gemm_mainloop_direct(const TileLanes<Cfg>& tl,
                                                     const uint16_t* const (&baseA)[TileLanes<Cfg>::NJA],
                                                     const uint32_t (&offA)[TileLanes<Cfg>::NJA],
                                                     const uint16_t* const (&baseB)[TileLanes<Cfg>::NJB],
                                                     const uint32_t (&offB)[TileLanes<Cfg>::NJB], int k_len,
                                                     uint8_t* lds, typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN],
                                                     const KMajorB& kb = KMajorB()) {
  if constexpr (Cfg::MFMA16) gemm_mainloop_fixed16<Cfg>(tl, baseA, offA, baseB, offB, k_len, lds, acc, kb);
  else if constexpr (Cfg::RING) gemm_mainloop_ring<Cfg>(tl, baseA, offA, baseB, offB, k_len, lds, acc, kb);
  else gemm_mainloop_slab_dma<Cfg>(tl, baseA, offA, baseB, offB, k_len, lds, acc, kb);
}

// Map a launch-order workgroup id to a position L in the tile order such that every XCD
// (workgroup b runs on XCD b % 8) owns one contiguous range of the order: tiles that share
// A rows / B columns then meet in the same L2.  Returns -1 for a surplus workgroup.

__device__ __forceinline__ int xcd_tile_slot(int total, int bid) {
  const int per_xcd = cdiv(total, kXcds);
  const int slot = bid / kXcds;
  if (slot >= per_xcd) return -1;
  const int L = (bid % kXcds) * per_xcd + slot;
  return L < total ? L : -1;
}

// Epilogue shared by the routed kernels.  Per accumulator tile a lane holds token row lr and the output
// columns acc_col(v, lh), i.e. runs of four consecutive columns (one 8-byte store each).
template <class Cfg>
__device__ __forceinline__ void routed_epilogue(const GemmArgs& g, typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN], int row0,
                                                int row_end, int n0, int wm, int wn, uint32_t lr, uint32_t lh) {
  constexpr int TM = Cfg::TM, TN_OUT = Cfg::TN_OUT, MT = Cfg::MT, RUNS = Cfg::ACC_N / 4;
  // A tile inside the matrix on every side, with 8-byte aligned runs: no guards, one row pointer per row group and
  // the column of every store an immediate offset.  (The guarded form below costs a compare and two branches per
  // run of four outputs - as many cycles as the SwiGLU itself.)
  const bool inside = row0 + Cfg::BM <= row_end && n0 + Cfg::BN_OUT <= g.N && (reinterpret_cast<uintptr_t>(g.C) & 7) == 0 &&
                      (g.ldc & 3) == 0 && !(Cfg::DUAL && g.C_pre != nullptr);
  if (inside) {
    int64_t dst[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int p = row0 + wm * Cfg::WTM + i * MT + (int)lr;
      dst[i] = Cfg::SCATTER_C ? (int64_t)g.perm[p] : (int64_t)p;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      uint16_t* crow = g.C + dst[i] * g.ldc + (n0 + wn * Cfg::WTN_OUT + acc_col<Cfg>(0, (int)lh));
#pragma unroll
      for (int j = 0; j < TN_OUT; ++j) {
#pragma unroll
        for (int q4 = 0; q4 < RUNS; ++q4) {
          float o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (Cfg::DUAL) o[e] = swiglu(acc[i][j][4 * q4 + e], acc[i][j + TN_OUT][4 * q4 + e]);
            else o[e] = acc[i][j][4 * q4 + e];
          }
          uint2 v2;
          v2.x = pack2bf(o[0], o[1]);
          v2.y = pack2bf(o[2], o[3]);
          *reinterpret_cast<uint2*>(crow + j * MT + (acc_col<Cfg>(4 * q4, 0) - acc_col<Cfg>(0, 0))) = v2;
        }
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int p = row0 + wm * Cfg::WTM + i * MT + (int)lr;
    if (p >= row_end) continue;
    const int64_t dst = Cfg::SCATTER_C ? (int64_t)g.perm[p] : (int64_t)p;
    uint16_t* crow = g.C + dst * g.ldc;
#pragma unroll
    for (int j = 0; j < TN_OUT; ++j) {
      const int nb = n0 + wn * Cfg::WTN_OUT + j * MT;
#pragma unroll
      for (int q4 = 0; q4 < RUNS; ++q4) {
        const int n = nb + acc_col<Cfg>(4 * q4, (int)lh);
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (Cfg::DUAL) o[e] = swiglu(acc[i][j][4 * q4 + e], acc[i][j + TN_OUT][4 * q4 + e]);
          else o[e] = acc[i][j][4 * q4 + e];
        }
        if (n + 3 < g.N && ((reinterpret_cast<uintptr_t>(crow + n) & 7) == 0)) {
          uint2 v2;
          v2.x = pack2bf(o[0], o[1]);
          v2.y = pack2bf(o[2], o[3]);
          *reinterpret_cast<uint2*>(crow + n) = v2;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < g.N) crow[n + e] = f2bf(o[e]);
        }
        if (Cfg::DUAL && g.C_pre != nullptr) {  // uniform over the launch
          uint16_t* prow = g.C_pre + dst * g.ldc_pre + n;
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const typename Cfg::Acc& t = acc[i][j + half * TN_OUT];
            uint16_t* pp = prow + (int64_t)half * g.N;
            if (n + 3 < g.N && ((reinterpret_cast<uintptr_t>(pp) & 7) == 0)) {
              uint2 v2;
              v2.x = pack2bf(t[4 * q4], t[4 * q4 + 1]);
              v2.y = pack2bf(t[4 * q4 + 2], t[4 * q4 + 3]);
              *reinterpret_cast<uint2*>(pp) = v2;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < g.N) pp[e] = f2bf(t[4 * q4 + e]);
            }
          }
        }
      }
    }
  }
}

// Split-K epilogue: fp32 partial sums of one K range, no SwiGLU.  Element (routed row p, column n)
// goes to base[p * ld + n].
template <class Cfg>
__device__ __forceinline__ void routed_partial_store(float* base, int64_t ld, const GemmArgs& g,
                                                     typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN], int row0, int row_end, int n0,
                                                     int wm, int wn, uint32_t lr, uint32_t lh) {
  constexpr int MT = Cfg::MT, RUNS = Cfg::ACC_N / 4;
#pragma unroll
  for (int i = 0; i < Cfg::TM; ++i) {
    const int p = row0 + wm * Cfg::WTM + i * MT + (int)lr;
    if (p >= row_end) continue;
    float* prow = base + (int64_t)p * ld;
#pragma unroll
    for (int j = 0; j < Cfg::TN; ++j) {
#pragma unroll
      for (int q4 = 0; q4 < RUNS; ++q4) {
        const int n = n0 + wn * Cfg::WTN_OUT + j * MT + acc_col<Cfg>(4 * q4, (int)lh);
        if (n + 3 < g.N) {
          *reinterpret_cast<float4*>(prow + n) =
              make_float4(acc[i][j][4 * q4], acc[i][j][4 * q4 + 1], acc[i][j][4 * q4 + 2], acc[i][j][4 * q4 + 3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < g.N) prow[n + e] = acc[i][j][4 * q4 + e];
        }
      }
    }
  }
}

// Routed GEMM: rows in routed order, group-pure tiles.
//   GATHER_A : A row of routed position p is perm[p] (else p)
//   SCATTER_C: C row of routed position p is perm[p] (else p)
//   DUAL     : C = silu(A B0^T) * (A B1^T)   (SwiGLU epilogue in fp32 registers)
// `bid`: the workgroup's index among those of this GEMM (the launch's block index, or its offset inside a
// launch that runs several GEMMs side by side); `lds`: Cfg::LDS_BYTES, 1 KB aligned.
template <class Cfg>
__device__ __forceinline__ void routed_gemm_body(const GemmArgs& g, uint8_t* lds, const int bid) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN;
  constexpr int TM = Cfg::TM, TN = Cfg::TN;

  // ---- tile schedule (all from device-side counts; no host sync) ----
  const int SBM = g.sched_bm > 0 ? g.sched_bm : BM;
  const int SBN = g.sched_bn > 0 ? g.sched_bn : Cfg::BN_OUT;
  const int n_vis = g.counts[0];
  const int total = routed_tile_count(n_vis, g.M, g.N, SBM, SBN);
  int L, sub_m = 0, sub_n = 0, split = 0, splits = 1, tail_slot = 0;
  if (g.tail_mode == 0) {
    splits = g.splits;
    L = xcd_tile_slot(total * splits, bid);
    if (splits > 1 && L >= 0) {  // range-major: neighbours in the order share panels, not a K range
      split = L / total;
      L -= split * total;
    }
  } else {
    const int full = total / kCusPerChip * kCusPerChip;
    if (g.tail_mode == 1) {
      L = xcd_tile_slot(full, bid);
    } else if (g.tail_mode == 2) {
      const int qn = SBN / Cfg::BN_OUT, q = (SBM / BM) * qn;  // own tiles per macro tile
      if (bid >= (total - full) * q) return;
      L = full + bid / q;
      sub_m = (bid % q) / qn;
      sub_n = (bid % q) % qn;
    } else {
      const int n_tail = total - full;
      splits = tail_split_factor(n_tail, g.K / kBK);
      tail_slot = bid;
      if (tail_slot >= n_tail * splits) return;
      split = tail_slot / n_tail;
      L = full + tail_slot % n_tail;
    }
  }
  if (L < 0) return;
  const TileCoord tc = routed_tile_coord(L, n_vis, g.M, g.N, SBM, SBN, g.group_m > 0 ? g.group_m : Cfg::GROUP_M);
  const int grp = tc.grp;
  const int row0 = tc.row0 + sub_m * BM;  // routed position
  const int row_end = tc.row_end;
  const int n0 = tc.n0 + sub_n * Cfg::BN_OUT;
  if (row0 >= row_end || n0 >= g.N) return;  // a sub-tile past the edge of a partial macro tile

  typename Cfg::Acc acc[TM][TN];
  if constexpr (Cfg::DIRECT) {
    constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
    TileLanes<Cfg> rl;
    rl.init();
    // This workgroup's part of the contraction (all of it unless the launch splits K).
    const int nk = g.K / kBK;
    const int per_split = cdiv(nk, splits);
    const int kt0 = min(split * per_split, nk);
    const int k_len = (min(kt0 + per_split, nk) - kt0) * kBK;
    const int64_t k0 = (int64_t)kt0 * kBK;
    const uint16_t* baseA[NJA];
    uint32_t offA[NJA];
    const uint16_t* baseB[NJB];
    uint32_t offB[NJB];
    // Gathered rows are addressed from the start of A (the host checks that 32 bits reach every
    // row); contiguous panels from their own first row.
    const uint16_t* a0 = (Cfg::GATHER_A ? g.A : g.A + (int64_t)row0 * g.lda) + k0;
#pragma unroll
    for (int j = 0; j < NJA; ++j) {
      int p = row0 + rl.load_row(j);
      p = min(p, row_end - 1);  // rows past the group end repeat the last row; never stored
      const int64_t src = Cfg::GATHER_A ? (int64_t)g.perm[p] : (int64_t)(p - row0);
      baseA[j] = a0;
      offA[j] = (uint32_t)((src * g.lda + rl.c_log * 8) * 2);
    }
    KMajorB kb;
    if constexpr (Cfg::B_KMAJOR) {
      // Offsets inside a slab: row of the slab times the row stride, plus this lane's column chunk
      // (chunks past the last column repeat the last one; their outputs are never stored).
#pragma unroll
      for (int j = 0; j < NJB; ++j) {
        const int n = min(n0 + (int)rl.kb_chunk * 8, g.N - 8);
        baseB[j] = nullptr;
        offB[j] = (uint32_t)(((int64_t)rl.kb_group_row(j) * g.ldb + n) * 2);
      }
      kb.w[0] = g.B0[grp];
      kb.w[1] = g.k_switch > 0 ? g.B1[grp] : g.B0[grp];
      kb.kt_first = kt0;
      if (g.k_switch > 0) kb.kt_switch = g.k_switch / kBK;
      kb.slab_bytes = (uint32_t)(g.ldb * (kBK * 2));
    } else {
#pragma unroll
      for (int j = 0; j < NJB; ++j) {
        const bool up = Cfg::DUAL && rl.group_row(j) >= BN / 2;  // uniform over the wave
        const int r = rl.load_row(j) - (up ? BN / 2 : 0);
        const int n_first = min(n0, g.N - 1);
        const int n = min(n0 + r, g.N - 1);
        baseB[j] = (up ? g.B1[grp] : g.B0[grp]) + (int64_t)n_first * g.ldb + k0;
        offB[j] = (uint32_t)(((int64_t)(n - n_first) * g.ldb + rl.c_log * 8) * 2);
      }
    }
    if (k_len > 0) gemm_mainloop_direct<Cfg>(rl, baseA, offA, baseB, offB, k_len, lds, acc, kb);
    else zero_acc<Cfg>(acc);  // a range past the end of K contributes exact zeros
    if (!Cfg::DUAL && splits > 1) {
      if (g.tail_mode == 3)  // one compact fp32 tile per (tile, range) pair
        routed_partial_store<Cfg>(g.P_tail + (int64_t)tail_slot * (BM * Cfg::BN_OUT) - ((int64_t)row0 * Cfg::BN_OUT + n0),
                                  Cfg::BN_OUT, g, acc, row0, row_end, n0, rl.wm, rl.wn, rl.lr, rl.lh);
      else
        routed_partial_store<Cfg>(g.P + (int64_t)split * g.M * g.N, g.N, g, acc, row0, row_end, n0, rl.wm, rl.wn, rl.lr, rl.lh);
    } else {
      routed_epilogue<Cfg>(g, acc, row0, row_end, n0, rl.wm, rl.wn, rl.lr, rl.lh);
    }
  } else {
    constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
    TileLanes<Cfg> tl;
    tl.init();
    const uint16_t* pa[NJA];
    const uint16_t* pb[NJB];
#pragma unroll
    for (int j = 0; j < NJA; ++j) {
      int p = row0 + tl.load_row(j);
      p = min(p, row_end - 1);
      const int64_t src = Cfg::GATHER_A ? (int64_t)g.perm[p] : (int64_t)p;
      pa[j] = g.A + src * g.lda + tl.c_log * 8;
    }
#pragma unroll
    for (int j = 0; j < NJB; ++j) {
      const int r = tl.load_row(j);  // row of the LDS B panel
      const bool up = Cfg::DUAL && r >= BN / 2;
      const int n = min(n0 + (up ? r - BN / 2 : r), g.N - 1);
      pb[j] = (up ? g.B1[grp] : g.B0[grp]) + (int64_t)n * g.ldb + tl.c_log * 8;
    }
    gemm_mainloop_staged<Cfg>(tl, pa, pb, g.K, lds, acc);
    routed_epilogue<Cfg>(g, acc, row0, row_end, n0, tl.wm, tl.wn, tl.lr, tl.lh);
  }
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void routed_gemm_kernel(const GemmArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[Cfg::LDS_BYTES];
  routed_gemm_body<Cfg>(g, lds, (int)blockIdx.x);
}

// Store a weight-gradient tile: bf16 with the caller's strides when the contraction was not split, fp32 partials
// otherwise.  acc[i][j][v]: BM-panel row (= output column c) c0 + wm*WTM + i*MT + lr;
//                           BN-panel row (= output row r) r0 + wn*WTN + j*MT + acc_col(v, lh).
template <class Cfg>
__device__ __forceinline__ void splitk_store(const SplitKArgs& g, typename Cfg::Acc (&acc)[Cfg::TM][Cfg::TN], int grp, int split,
                                             int r0, int c0, const TileLanes<Cfg>& rl) {
  constexpr int TM = Cfg::TM, TN = Cfg::TN;
  constexpr int MT = Cfg::MT, RUNS = Cfg::ACC_N / 4;
  if (g.out[0] != nullptr) {
    // single split: the sums are complete, store bf16 with the caller's strides
    uint16_t* out = g.out[grp];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int c = c0 + rl.wm * Cfg::WTM + i * MT + (int)rl.lr;
      if (c >= g.Cc) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int q4 = 0; q4 < RUNS; ++q4) {
          const int r = r0 + rl.wn * Cfg::WTN_OUT + j * MT + acc_col<Cfg>(4 * q4, (int)rl.lh);
          uint16_t* dst = out + (int64_t)r * g.out_sr + (int64_t)c * g.out_sc;
          if (g.out_sr == 1 && r + 3 < g.R && (reinterpret_cast<uintptr_t>(dst) & 7) == 0) {
            uint2 v2;
            v2.x = pack2bf(acc[i][j][4 * q4], acc[i][j][4 * q4 + 1]);
            v2.y = pack2bf(acc[i][j][4 * q4 + 2], acc[i][j][4 * q4 + 3]);
            *reinterpret_cast<uint2*>(dst) = v2;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (r + e < g.R) dst[(int64_t)e * g.out_sr] = f2bf(acc[i][j][4 * q4 + e]);  // out_sc == 1: MT lanes -> 2 MT contiguous bytes
          }
        }
      }
    }
    return;
  }
  float* P = g.P + ((int64_t)(grp * g.splits + split)) * g.R * g.Cc;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int c = c0 + rl.wm * Cfg::WTM + i * MT + (int)rl.lr;
    if (c >= g.Cc) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int v = 0; v < Cfg::ACC_N; ++v) {
        const int r = r0 + rl.wn * Cfg::WTN_OUT + j * MT + acc_col<Cfg>(v, (int)rl.lh);
        if (r < g.R) P[(int64_t)r * g.Cc + c] = acc[i][j][v];  // MT lanes -> MT consecutive floats
      }
    }
  }
}

// Grouped split-K GEMM of the weight gradients (operands are padded to 64-element slabs, so
// the direct path always applies).  With Cfg::B_KMAJOR the operand A is not a padded transpose but
// the original [rows, R] matrix in routed order (see SplitKArgs).
template <class Cfg>
__device__ __forceinline__ void grouped_splitk_body(const SplitKArgs& g, uint8_t* lds, const int bid) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN;
  constexpr int TM = Cfg::TM, TN = Cfg::TN;
  constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
  static_assert(!Cfg::DUAL && Cfg::DIRECT, "split-K GEMM runs on padded, 64-aligned slabs");

  // The BM-row LDS panel holds rows of B (output columns) and the BN-row panel holds rows of A
  // (output rows): a 32-lane half wave then owns 32 consecutive output columns of one output
  // row, which makes the fp32 partial stores 128-byte contiguous.
  const int tiles_r = cdiv(g.R, BN);
  const int tiles_c = cdiv(g.Cc, BM);
  const int per_grp = tiles_r * tiles_c * g.splits;
  int L = xcd_tile_slot(2 * per_grp, bid);
  if (L < 0) return;
  const int grp = L / per_grp;
  L -= grp * per_grp;
  const int split = L % g.splits;
  const int tile = L / g.splits;
  const int tile_r = tile % tiles_r, tile_c = tile / tiles_r;

  const int n_vis = g.counts[0];
  const int vpad = (n_vis + 63) & ~63;
  const int k_begin_g = grp == 0 ? 0 : vpad;
  const int k_len_g = grp == 0 ? vpad : ((g.M - n_vis + 63) & ~63);
  const int nk_g = k_len_g / kBK;
  const int per_split = cdiv(nk_g, g.splits);
  const int kt0 = min(split * per_split, nk_g);
  const int kt1 = min(kt0 + per_split, nk_g);
  const int64_t k_begin = (int64_t)k_begin_g + (int64_t)kt0 * kBK;
  const int k_len = (kt1 - kt0) * kBK;

  TileLanes<Cfg> rl;
  rl.init();
  const int r0 = tile_r * BN, c0 = tile_c * BM;
  typename Cfg::Acc acc[TM][TN];
  if (k_len > 0) {
    const uint16_t* baseA[NJA];
    uint32_t offA[NJA];
    const uint16_t* baseB[NJB];
    uint32_t offB[NJB];
    const int c_first = min(c0, g.Cc - 1), r_first = min(r0, g.R - 1);
#pragma unroll
    for (int j = 0; j < NJA; ++j) {
      const int c = min(c0 + rl.load_row(j), g.Cc - 1);
      baseA[j] = g.B + (int64_t)c_first * g.ldb + k_begin;
      offA[j] = (uint32_t)(((int64_t)(c - c_first) * g.ldb + rl.c_log * 8) * 2);
    }
    KMajorB kb;
    if constexpr (Cfg::B_KMAJOR) {
      // A is read where it lies: contraction rows are its rows (routed order, unpadded), starting at the
      // group's first routed row.  Rows past the group's end are cleared in LDS (KMajorB::last_rows).
#pragma unroll
      for (int j = 0; j < NJB; ++j) {
        const int r = min(r0 + (int)rl.kb_chunk * 8, g.R - 8);
        baseB[j] = nullptr;
        offB[j] = (uint32_t)(((int64_t)rl.kb_group_row(j) * g.lda + r) * 2);
      }
      const int64_t row_begin = (grp == 0 ? 0 : n_vis) + (int64_t)kt0 * kBK;
      kb.w[0] = kb.w[1] = g.A + row_begin * g.lda;
      kb.slab_bytes = (uint32_t)(g.lda * (kBK * 2));
      // the group's last slab is ragged: only the range that holds it has rows to clear
      const int rows_g = grp == 0 ? n_vis : g.M - n_vis;
      if (kt1 == nk_g) kb.last_rows = rows_g - (nk_g - 1) * kBK;
    } else {
#pragma unroll
      for (int j = 0; j < NJB; ++j) {
        const int r = min(r0 + rl.load_row(j), g.R - 1);
        baseB[j] = g.A + (int64_t)r_first * g.lda + k_begin;
        offB[j] = (uint32_t)(((int64_t)(r - r_first) * g.lda + rl.c_log * 8) * 2);
      }
    }
    gemm_mainloop_direct<Cfg>(rl, baseA, offA, baseB, offB, k_len, lds, acc, kb);
  } else {
    zero_acc<Cfg>(acc);  // a split without slabs (e.g. an empty modality) contributes exact zeros
  }

  splitk_store<Cfg>(g, acc, grp, split, r0, c0, rl);
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void grouped_splitk_kernel(const SplitKArgs g) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[Cfg::LDS_BYTES];
  grouped_splitk_body<Cfg>(g, lds, (int)blockIdx.x);
}

// The MaskedLinear backward's two GEMMs in one launch, as the reference's _fused_bwd_kernel runs dA and
// dB by program-id range (ffn_kernel/linear.py:15-72): workgroups [0, dw_blocks) compute weight-gradient
// tiles (the long ones: they start first), the rest dx tiles.  The two share nothing but perm / counts,
// so the chip is filled by both at once instead of by each in turn with a partial last round.
template <class CfgDx, class CfgDw>
__global__ __launch_bounds__(CfgDx::NT) void fused_bwd_kernel(const GemmArgs gx, const SplitKArgs gw, const int dw_blocks) {
  static_assert(CfgDx::NT == CfgDw::NT, "one workgroup size for both GEMMs");
  constexpr int kLds = CfgDx::LDS_BYTES > CfgDw::LDS_BYTES ? CfgDx::LDS_BYTES : CfgDw::LDS_BYTES;
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kLds];
  if ((int)blockIdx.x < dw_blocks) grouped_splitk_body<CfgDw>(gw, lds, (int)blockIdx.x);
  else routed_gemm_body<CfgDx>(gx, lds, (int)blockIdx.x - dw_blocks);
}

// Upper bound on the number of workgroups the kernel needs, rounded so that every XCD gets the
// same number of slots.  The kernel derives the real tile count from counts[] on the device.
template <class Cfg>
inline int routed_gemm_grid(int M, int N) {
  const int tiles_m = cdiv(M, Cfg::BM) + 1;  // the two groups can each end in a partial tile
  const int tiles_n = cdiv(N, Cfg::BN_OUT);
  const int64_t total = (int64_t)tiles_m * tiles_n;
  return (int)(cdiv64(total, kXcds) * kXcds);
}

template <class Cfg>
inline hipError_t launch_routed_gemm(const GemmArgs& g, hipStream_t stream) {
  if (g.M <= 0 || g.N <= 0) return hipSuccess;
  if (g.splits > 1 && (Cfg::DUAL || !Cfg::DIRECT || g.tail_mode != 0 || g.P == nullptr)) return hipErrorInvalidValue;
  if (Cfg::B_KMAJOR && (g.N % 8 != 0 || g.K % kBK != 0 || g.k_switch % kBK != 0 || g.k_switch < 0 || g.k_switch >= g.K ||
                        g.ldb * (kBK * 2) + 2 * (int64_t)g.N >= ((int64_t)1 << 32)))
    return hipErrorInvalidValue;
  if (!Cfg::B_KMAJOR && g.k_switch != 0) return hipErrorInvalidValue;
  const int grid = routed_gemm_grid<Cfg>(g.M, g.N) * (g.splits > 1 ? g.splits : 1);
  hipLaunchKernelGGL(routed_gemm_kernel<Cfg>, dim3(grid), dim3(Cfg::NT), 0, stream, g);
  return hipGetLastError();
}

template <class Cfg>
inline hipError_t launch_grouped_splitk(const SplitKArgs& g, hipStream_t stream) {
  if (g.R <= 0 || g.Cc <= 0 || g.splits <= 0) return hipSuccess;
  if (Cfg::B_KMAJOR && (g.R % 8 != 0 || g.lda * (kBK * 2) + 2 * (int64_t)g.R >= ((int64_t)1 << 32))) return hipErrorInvalidValue;
  const int64_t total = 2LL * cdiv(g.R, Cfg::BN) * cdiv(g.Cc, Cfg::BM) * g.splits;
  const int grid = (int)(cdiv64(total, kXcds) * kXcds);
  hipLaunchKernelGGL(grouped_splitk_kernel<Cfg>, dim3(grid), dim3(Cfg::NT), 0, stream, g);
  return hipGetLastError();
}

}  // namespace ffnk
