// Routed "NT" GEMM core for gfx950: C[rows, N] = A[rows, K] * B_g[N, K]^T with both operands
// K-contiguous, bf16 in, fp32 MFMA accumulation.  Rows are processed in routed order (visual
// group first); a workgroup tile never mixes groups, so each tile multiplies by exactly one
// modality's weight.  This replaces the per-tile three-way branch of the reference kernels
// (ffn_kernel/linear.py:127-153, ffn_kernel/ffn.py:68-105), which pay two dots and a select
// on every mixed tile.
//
// Data path per workgroup: 64-column K slabs of the A and B panels go global -> LDS (directly,
// bypassing registers, or staged through registers when K has a tail), double-buffered with
// one barrier per slab; wavefronts read 16-byte MFMA fragments from an XOR-swizzled LDS
// layout and issue v_mfma_f32_32x32x16_bf16.
#pragma once
#include "common.hpp"
#include "gemm_args.hpp"

namespace ffnk {

constexpr int kBK = 64;          // K elements per LDS stage
constexpr int kRowBytes = 128;   // kBK * sizeof(bf16)
constexpr int kXcds = 8;         // MI355X: 8 XCDs, workgroups are dealt to them round-robin

// LDS byte offset of 16-byte chunk c (0..7) of tile row r.  Two rows share a 256-byte line;
// the chunk index is XORed with the row so that the 16 lanes of one ds_read_b128 phase
// (16 consecutive rows, same logical chunk) hit 16 distinct 16-byte bank groups, and any
// aligned 8 of them hit 8 distinct groups modulo 128 bytes.
__host__ __device__ constexpr uint32_t lds_swizzle(uint32_t r, uint32_t c) {
  return ((r >> 1) << 8) | (((((r & 1u) ^ ((r >> 3) & 1u)) << 3) | (c ^ (r & 7u))) << 4);
}

#define FFNK_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define FFNK_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, bool DUAL_, bool GATHER_A_, bool SCATTER_C_,
          bool DIRECT_, int GROUP_M_>
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
  static constexpr int NWAVES = WAVES_M * WAVES_N;
  static constexpr int NT = NWAVES * kWave;
  static constexpr int BN_OUT = DUAL ? BN / 2 : BN;        // output columns per tile
  static constexpr int WTM = BM / WAVES_M;                 // rows per wave
  static constexpr int WTN_OUT = BN_OUT / WAVES_N;         // output columns per wave
  static constexpr int TM = WTM / 32;                      // 32x32 MFMA tiles per wave, M direction
  static constexpr int TN_OUT = WTN_OUT / 32;
  static constexpr int TN = DUAL ? 2 * TN_OUT : TN_OUT;    // accumulator tiles per wave, N direction
  static constexpr int A_BYTES = BM * kRowBytes;
  static constexpr int B_BYTES = BN * kRowBytes;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static_assert(WTM % 32 == 0 && WTN_OUT % 32 == 0, "wave tile must be a multiple of 32x32");
  static_assert(NWAVES % 2 == 0, "direct loads need an even wave count");
  static_assert((BM / 8) % NWAVES == 0 && (BN / 8) % NWAVES == 0, "panel rows must split evenly over waves");
};

// Per-thread description of which 16-byte chunks of the A and B panels this lane moves, and
// which LDS fragments it reads.  Built once per tile by the kernels below.
template <class Cfg>
struct TileLanes {
  static constexpr int NJA = Cfg::BM / 8 / Cfg::NWAVES;  // 1 KB (8-row) groups of the A panel per wave
  static constexpr int NJB = Cfg::BN / 8 / Cfg::NWAVES;
  int lane, wave, wm, wn;
  uint32_t r_in;   // row inside the 8-row group this lane loads
  uint32_t c_log;  // logical 16-byte chunk (0..7) of that row
  uint32_t lr, lh; // MFMA fragment row (0..31) and K half (0..1)

  __device__ __forceinline__ void init() {
    const int tid = threadIdx.x;
    lane = tid & (kWave - 1);
    wave = tid / kWave;
    wm = wave / Cfg::WAVES_N;
    wn = wave % Cfg::WAVES_N;
    // The panel is moved as 1 KB groups of 8 rows; group id = j * NWAVES + wave, so the group's
    // parity (which the swizzle needs) is the wave's parity.  The lane fills physical 16-byte
    // slot `lane` of the group: lds_swizzle(group * 8 + r_in, c_log) == group * 1024 + lane * 16.
    const uint32_t q = lane & 15;
    r_in = 2 * (lane >> 4) + ((q >> 3) ^ (wave & 1));
    c_log = (q & 7) ^ r_in;
    lr = lane & 31;
    lh = lane >> 5;
  }
  // Tile row that load j of this lane covers.
  __device__ __forceinline__ int load_row(int j) const { return (j * Cfg::NWAVES + wave) * 8 + (int)r_in; }
};

// K loop of one tile.  pa[j] / pb[j] point at this lane's chunk of slab 0 for each of its rows;
// `k_len` is the contraction length from there (a multiple of 8; of 64 when Cfg::DIRECT).
// Accumulates into acc[TM][TN] (32x32 tiles, D[n][m] orientation: the weights are the MFMA "A"
// operand so that each lane ends up with runs of four consecutive output columns of one token row).
template <class Cfg>
__device__ __forceinline__ void gemm_mainloop(const TileLanes<Cfg>& tl,
                                              const uint16_t* const (&pa)[TileLanes<Cfg>::NJA],
                                              const uint16_t* const (&pb)[TileLanes<Cfg>::NJB], int k_len,
                                              uint8_t* lds0, uint8_t* lds1,
                                              f32x16_t (&acc)[Cfg::TM][Cfg::TN]) {
  constexpr int BN = Cfg::BN, NWAVES = Cfg::NWAVES;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, TN_OUT = Cfg::TN_OUT;
  constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
  const int lane = tl.lane, wave = tl.wave;

  // Fragment rows start at multiples of 32, so the swizzle terms depend on the lane only.
  uint32_t koff[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) koff[s] = lds_swizzle(tl.lr, 2 * s + tl.lh);
  const uint32_t a_base = (uint32_t)(tl.wm * Cfg::WTM) * kRowBytes;
  uint32_t b_base[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    int r;
    if (Cfg::DUAL) r = (tn < TN_OUT ? 0 : BN / 2) + tl.wn * Cfg::WTN_OUT + (tn % TN_OUT) * 32;
    else r = tl.wn * Cfg::WTN_OUT + tn * 32;
    b_base[tn] = Cfg::A_BYTES + (uint32_t)r * kRowBytes;
  }

#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int nk = cdiv(k_len, kBK);

  auto issue_direct = [&](uint8_t* stage, int kt) {
    const int64_t ko = (int64_t)kt * kBK;
#pragma unroll
    for (int j = 0; j < NJA; ++j)
      __builtin_amdgcn_global_load_lds(FFNK_GLOBAL_PTR(pa[j] + ko),
                                       FFNK_LDS_PTR(stage + (j * NWAVES + wave) * 1024), 16, 0, 0);
#pragma unroll
    for (int j = 0; j < NJB; ++j)
      __builtin_amdgcn_global_load_lds(FFNK_GLOBAL_PTR(pb[j] + ko),
                                       FFNK_LDS_PTR(stage + Cfg::A_BYTES + (j * NWAVES + wave) * 1024), 16, 0, 0);
  };

  uint4 ra[NJA], rb[NJB];  // register staging (only live when !DIRECT)
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
  if (Cfg::DIRECT) {
    issue_direct(lds0, 0);
    for (int kt = 0; kt < nk; kt += 2) {
      __syncthreads();  // slab kt has landed everywhere; everyone is done reading lds1
      if (kt + 1 < nk) issue_direct(lds1, kt + 1);
      compute(lds0);
      if (kt + 1 < nk) {
        __syncthreads();
        if (kt + 2 < nk) issue_direct(lds0, kt + 2);
        compute(lds1);
      }
    }
  } else {
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
}

// Map a launch-order workgroup id to a position L in the tile order such that every XCD
// (workgroup b runs on XCD b % 8) owns one contiguous range of the order: tiles that share
// A rows / B columns then meet in the same L2.  Returns -1 for a surplus workgroup.
__device__ __forceinline__ int xcd_tile_slot(int total) {
  const int per_xcd = cdiv(total, kXcds);
  const int slot = blockIdx.x / kXcds;
  if (slot >= per_xcd) return -1;
  const int L = (blockIdx.x % kXcds) * per_xcd + slot;
  return L < total ? L : -1;
}

// Routed GEMM: rows in routed order, group-pure tiles.
//   GATHER_A : A row of routed position p is perm[p] (else p)
//   SCATTER_C: C row of routed position p is perm[p] (else p)
//   DUAL     : C = silu(A B0^T) * (A B1^T)   (SwiGLU epilogue in fp32 registers)
template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void routed_gemm_kernel(const GemmArgs g) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN;
  constexpr int TM = Cfg::TM, TN = Cfg::TN, TN_OUT = Cfg::TN_OUT;
  constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;

  __shared__ __attribute__((aligned(1024))) uint8_t lds0[Cfg::STAGE_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t lds1[Cfg::STAGE_BYTES];

  // ---- tile schedule (all from device-side counts; no host sync) ----
  const int n_vis = g.counts[0];
  const int n_txt = g.M - n_vis;
  const int tiles_v = cdiv(n_vis, BM);
  const int tiles_m = tiles_v + cdiv(n_txt, BM);
  const int tiles_n = cdiv(g.N, Cfg::BN_OUT);
  const int L = xcd_tile_slot(tiles_m * tiles_n);
  if (L < 0) return;
  const int width = Cfg::GROUP_M * tiles_n;
  const int first_m = (L / width) * Cfg::GROUP_M;
  const int gsz = min(Cfg::GROUP_M, tiles_m - first_m);
  const int tile_m = first_m + (L % width) % gsz;
  const int tile_n = (L % width) / gsz;

  const int grp = tile_m < tiles_v ? 0 : 1;
  const int row0 = grp == 0 ? tile_m * BM : n_vis + (tile_m - tiles_v) * BM;  // routed position
  const int row_end = grp == 0 ? n_vis : g.M;
  const int n0 = tile_n * Cfg::BN_OUT;

  TileLanes<Cfg> tl;
  tl.init();

  const uint16_t* pa[NJA];
  const uint16_t* pb[NJB];
#pragma unroll
  for (int j = 0; j < NJA; ++j) {
    int p = row0 + tl.load_row(j);
    p = min(p, row_end - 1);  // rows past the group end repeat the last row; never stored
    const int64_t src = Cfg::GATHER_A ? (int64_t)g.perm[p] : (int64_t)p;
    pa[j] = g.A + src * g.lda + tl.c_log * 8;
  }
#pragma unroll
  for (int j = 0; j < NJB; ++j) {
    const int r = tl.load_row(j);  // row of the LDS B panel
    const uint16_t* base;
    int n;
    if (Cfg::DUAL) {
      const bool up = r >= BN / 2;
      base = up ? g.B1[grp] : g.B0[grp];
      n = n0 + (up ? r - BN / 2 : r);
    } else {
      base = g.B0[grp];
      n = n0 + r;
    }
    n = min(n, g.N - 1);
    pb[j] = base + (int64_t)n * g.ldb + tl.c_log * 8;
  }

  f32x16_t acc[TM][TN];
  gemm_mainloop<Cfg>(tl, pa, pb, g.K, lds0, lds1, acc);

  // ---- epilogue: lane holds, per 32x32 tile, token row (lane & 31) and output columns
  //      8 * (v / 4) + 4 * (lane >> 5) + (v % 4) ----
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int p = row0 + tl.wm * Cfg::WTM + i * 32 + (int)tl.lr;
    if (p >= row_end) continue;
    const int64_t dst = Cfg::SCATTER_C ? (int64_t)g.perm[p] : (int64_t)p;
    uint16_t* crow = g.C + dst * g.ldc;
#pragma unroll
    for (int j = 0; j < TN_OUT; ++j) {
      const int nb = n0 + tl.wn * Cfg::WTN_OUT + j * 32 + 4 * (int)tl.lh;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int n = nb + 8 * q4;
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
      }
    }
  }
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void grouped_splitk_kernel(const SplitKArgs g) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN;
  constexpr int TM = Cfg::TM, TN = Cfg::TN;
  constexpr int NJA = TileLanes<Cfg>::NJA, NJB = TileLanes<Cfg>::NJB;
  static_assert(!Cfg::DUAL && Cfg::DIRECT, "split-K GEMM runs on padded, 64-aligned slabs");

  __shared__ __attribute__((aligned(1024))) uint8_t lds0[Cfg::STAGE_BYTES];
  __shared__ __attribute__((aligned(1024))) uint8_t lds1[Cfg::STAGE_BYTES];

  // The BM-row LDS panel holds rows of B (output columns) and the BN-row panel holds rows of A
  // (output rows): a 32-lane half wave then owns 32 consecutive output columns of one output
  // row, which makes the fp32 partial stores 128-byte contiguous.
  const int tiles_r = cdiv(g.R, BN);
  const int tiles_c = cdiv(g.Cc, BM);
  const int per_grp = tiles_r * tiles_c * g.splits;
  int L = xcd_tile_slot(2 * per_grp);
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

  TileLanes<Cfg> tl;
  tl.init();
  const int r0 = tile_r * BN, c0 = tile_c * BM;
  const uint16_t* pa[NJA];
  const uint16_t* pb[NJB];
#pragma unroll
  for (int j = 0; j < NJA; ++j) {
    const int c = min(c0 + tl.load_row(j), g.Cc - 1);
    pa[j] = g.B + (int64_t)c * g.ldb + k_begin + tl.c_log * 8;
  }
#pragma unroll
  for (int j = 0; j < NJB; ++j) {
    const int r = min(r0 + tl.load_row(j), g.R - 1);
    pb[j] = g.A + (int64_t)r * g.lda + k_begin + tl.c_log * 8;
  }

  f32x16_t acc[TM][TN];
  if (k_len > 0) {
    gemm_mainloop<Cfg>(tl, pa, pb, k_len, lds0, lds1, acc);
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  }

  // acc[i][j][v]: panel-"x" row (= output column c) c0 + wm*WTM + i*32 + (lane&31);
  //               panel-"weight" row (= output row r) r0 + wn*WTN + j*32 + 8*(v/4) + 4*(lane>>5) + v%4.
  float* P = g.P + ((int64_t)(grp * g.splits + split)) * g.R * g.Cc;
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int c = c0 + tl.wm * Cfg::WTM + i * 32 + (int)tl.lr;
    if (c >= g.Cc) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int r = r0 + tl.wn * Cfg::WTN_OUT + j * 32 + 8 * (v / 4) + 4 * (int)tl.lh + (v % 4);
        if (r < g.R) P[(int64_t)r * g.Cc + c] = acc[i][j][v];  // 32 lanes -> 32 consecutive floats
      }
    }
  }
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
  const int grid = routed_gemm_grid<Cfg>(g.M, g.N);
  hipLaunchKernelGGL(routed_gemm_kernel<Cfg>, dim3(grid), dim3(Cfg::NT), 0, stream, g);
  return hipGetLastError();
}

template <class Cfg>
inline hipError_t launch_grouped_splitk(const SplitKArgs& g, hipStream_t stream) {
  if (g.R <= 0 || g.Cc <= 0 || g.splits <= 0) return hipSuccess;
  const int64_t total = 2LL * cdiv(g.R, Cfg::BN) * cdiv(g.Cc, Cfg::BM) * g.splits;
  const int grid = (int)(cdiv64(total, kXcds) * kXcds);
  hipLaunchKernelGGL(grouped_splitk_kernel<Cfg>, dim3(grid), dim3(Cfg::NT), 0, stream, g);
  return hipGetLastError();
}

}  // namespace ffnk
