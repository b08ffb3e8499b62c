// Weight-gradient GEMM of the MaskedLinear backward with BOTH operands read where they lie:
//   dW_g[r, c] = sum over the rows m of group g of  G[m, r] * X[m, c]
// The contraction runs over token rows, which is the slow axis of both matrices, and the rows of a group are
// scattered through them (perm).  The reference walks all M rows in every program and masks the other
// modality's rows out of one operand (ffn_kernel/linear.py:382-407); the transposing form of this library
// (gather_transpose_kernel + grouped_splitk_kernel) first writes routed, padded transposes of G and X.  Here a
// 64-row slab of each operand goes global -> LDS row by row, every lane fetching from the token row that perm
// names for its slab row (the 32-bit byte offsets are recomputed per slab from perm entries fetched one slab
// ahead), and ds_read_b64_tr_b16 turns both slabs into MFMA operands, as KMajorB does for one.  Rows of a group's
// last slab that lie past its end are cleared in LDS in both panels, so a non-finite value in a row of the other
// group never reaches this group's gradient.  128x128 output tile, four wavefronts of 64x64, two LDS stages,
// v_mfma_f32_32x32x16_bf16; split over the rows like grouped_splitk_kernel and stored by splitk_store.
#pragma once
#include "gemm_nt.hpp"

namespace ffnk {

using GatherDwCfg = RoutedGemmCfg<128, 128, 2, 2, false, false, false, true, 8, true, 2>;

__device__ __forceinline__ void gathered_dw_body(const GatherDwArgs& a, uint8_t* lds, const int bid) {
#if defined(__HIP_DEVICE_COMPILE__)
  using Cfg = GatherDwCfg;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, NWAVES = Cfg::NWAVES;
  constexpr int NJ = TileLanes<Cfg>::NJB;            // 1 KB loads per wave, slab and panel
  constexpr int RB = BN * 2;                         // bytes of a slab row (both panels: BM == BN)
  constexpr int STAGE = Cfg::STAGE_BYTES, PANEL = Cfg::A_BYTES;
  static_assert(BM == BN && TileLanes<Cfg>::NJA == NJ && PANEL == kBK * RB && TM == 2 && TN == 2, "square tile, 64x64 wave tiles");
  const SplitKArgs& g = a.s;

  const int tiles_r = cdiv(g.R, BN);
  const int tiles_c = cdiv(g.Cc, BM);
  const int per_grp = tiles_r * tiles_c * g.splits;
  int L = xcd_tile_slot(2 * per_grp, bid);
  if (L < 0) return;
  const int grp = L / per_grp;
  L -= grp * per_grp;
  const int split = L % g.splits;
  const int tile = L / g.splits;
  const int r0 = (tile % tiles_r) * BN, c0 = (tile / tiles_r) * BM;

  const int n_vis = a.counts[0];
  const int p_begin = grp == 0 ? 0 : n_vis;           // routed positions of the group: [p_begin, p_end)
  const int p_end = grp == 0 ? n_vis : g.M;
  const int nk_g = cdiv(p_end - p_begin, kBK);
  const int per_split = cdiv(nk_g, g.splits);
  const int kt0 = min(split * per_split, nk_g);
  const int nk = min(kt0 + per_split, nk_g) - kt0;    // slabs of this workgroup
  const int p0 = p_begin + kt0 * kBK;                 // routed position of its first slab row
  // rows of the workgroup's last slab that belong to the group (the group's last slab is ragged)
  const int last_rows = min(kBK, p_end - (p0 + (nk - 1) * kBK));

  TileLanes<Cfg> rl;
  rl.init();
  typename Cfg::Acc acc[TM][TN];
  zero_acc<Cfg>(acc);
  if (nk > 0) {
    const int wave = rl.wave_s;
    const __amdgpu_buffer_rsrc_t rsG = __builtin_amdgcn_make_buffer_rsrc((void*)a.G, 0, 0xffffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsX = __builtin_amdgcn_make_buffer_rsrc((void*)a.X, 0, 0xffffffff, 0x00020000);
    // This lane's column chunk in each operand (chunks past the last column repeat the last one; never stored).
    const uint32_t colG = (uint32_t)min(r0 + (int)rl.kb_chunk * 8, g.R - 8) * 2;
    const uint32_t colX = (uint32_t)min(c0 + (int)rl.kb_chunk * 8, g.Cc - 8) * 2;
    const uint32_t rowG = (uint32_t)(a.ldg * 2), rowX = (uint32_t)(a.ldx * 2);  // bytes per token row (host: M * ld * 2 < 2^32)

    // Token rows of this lane's NJ slab rows in slab kt (positions past the group's end repeat its last row:
    // they are loaded, then cleared in LDS).
    auto fetch_rows = [&](int kt, int (&tok)[NJ]) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) tok[j] = a.perm[min(p0 + kt * kBK + rl.kb_group_row(j), p_end - 1)];
    };
    // Slab kt -> stage: the G panel goes where the weight panel of the routed kernels sits (behind the token panel).
    auto issue = [&](int stage, const int (&tok)[NJ]) {
      uint8_t* st = lds + stage * STAGE;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsX, FFNK_LDS_PTR(st + (j * NWAVES + wave) * 1024), 16,
                                                 (uint32_t)tok[j] * rowX + colX, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsG, FFNK_LDS_PTR(st + PANEL + (j * NWAVES + wave) * 1024), 16,
                                                 (uint32_t)tok[j] * rowG + colG, 0, 0, 0);
      }
    };
    // Clear rows [last_rows, 64) of both panels of `stage` (after the slab has landed, before anyone reads it).
    auto clear_tail = [&](int stage) {
      const int bytes = (kBK - last_rows) * RB;
#pragma unroll
      for (int pnl = 0; pnl < 2; ++pnl) {
        uint8_t* first = lds + stage * STAGE + pnl * PANEL + last_rows * RB;
        for (int o = (int)threadIdx.x * 16; o < bytes; o += Cfg::NT * 16) *reinterpret_cast<uint4*>(first + o) = make_uint4(0, 0, 0, 0);
      }
      dma_wait_barrier<0>();
    };

    // Transposing reads: as KMajorB's (gemm_mainloop_slab_dma), for both panels.  [stage][panel: 0 = X, 1 = G][tile][half]
    uint32_t kaddr[2][2][2][2];
    {
      const uint32_t i = rl.lane & 15, grp16 = rl.lane >> 4;
      const uint32_t row = 8 * rl.lh + (i >> 2);
      const uint32_t key = kmajor_swizzle_key<BN>(row);
      const uint32_t lds_addr = (uint32_t)reinterpret_cast<uintptr_t>(FFNK_LDS_PTR(lds));
#pragma unroll
      for (int pnl = 0; pnl < 2; ++pnl)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const uint32_t unit = (uint32_t)((pnl == 0 ? rl.wm : rl.wn) * 64 + t * 32) / 32;
          const uint32_t in_stage = pnl * PANEL + row * RB + ((unit ^ key) << 6) + 32 * (grp16 & 1) + 8 * (i & 3);
#pragma unroll
          for (int st = 0; st < 2; ++st) {
            kaddr[st][pnl][t][0] = lds_addr + st * STAGE + in_stage;
            kaddr[st][pnl][t][1] = kaddr[st][pnl][t][0] + 4 * RB;
          }
        }
    }
    bf16x4_t lo[2][2][2], hi[2][2][2];  // [buffer][panel][tile]
    auto reads = [&](int buf, int stage, auto ks_tag, int n0, int n1) {  // reads [n0, n1) of the 8 of a K step
      constexpr int ks = decltype(ks_tag)::value;
#pragma unroll
      for (int n = 0; n < 8; ++n) {
        if (n < n0 || n >= n1) continue;
        const int pnl = n >> 2, t = (n >> 1) & 1, half = n & 1;
        const bf16x4_t v = lds_read_tr16_b64<16 * ks * RB>(kaddr[stage][pnl][t][half]);
        if (half) hi[buf][pnl][t] = v;
        else lo[buf][pnl][t] = v;
      }
    };
    // One K step: wait for its fragments, then its four MFMAs with the next step's reads behind the first two and
    // (last step of a slab) the next slab's loads behind the others.
    auto step = [&](int cur, int stage_next, auto ks_next, bool rd, bool dma, int stage_dma, const int (&tok)[NJ]) {
      asm volatile("s_waitcnt lgkmcnt(0)"
                   : "+v"(lo[cur][0][0]), "+v"(hi[cur][0][0]), "+v"(lo[cur][0][1]), "+v"(hi[cur][0][1]), "+v"(lo[cur][1][0]),
                     "+v"(hi[cur][1][0]), "+v"(lo[cur][1][1]), "+v"(hi[cur][1][1]));
      bf16x8_t fx[2], fg[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        fx[t] = __builtin_shufflevector(lo[cur][0][t], hi[cur][0][t], 0, 1, 2, 3, 4, 5, 6, 7);
        fg[t] = __builtin_shufflevector(lo[cur][1][t], hi[cur][1][t], 0, 1, 2, 3, 4, 5, 6, 7);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[q / 2][q % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fg[q % 2], fx[q / 2], acc[q / 2][q % 2], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (q < 2) {
          if (rd) reads(cur ^ 1, stage_next, ks_next, q * 4, q * 4 + 4);
        } else if (dma) {
          uint8_t* st = lds + stage_dma * STAGE;
#pragma unroll
          for (int j = (q - 2) * (NJ / 2); j < (q - 1) * (NJ / 2); ++j) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsX, FFNK_LDS_PTR(st + (j * NWAVES + wave) * 1024), 16,
                                                     (uint32_t)tok[j] * rowX + colX, 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsG, FFNK_LDS_PTR(st + PANEL + (j * NWAVES + wave) * 1024), 16,
                                                     (uint32_t)tok[j] * rowG + colG, 0, 0, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    static_assert(NJ % 2 == 0, "a slab's loads go out behind two MFMAs");
    constexpr std::integral_constant<int, 0> k0{};
    constexpr std::integral_constant<int, 1> k1{};
    constexpr std::integral_constant<int, 2> k2{};
    constexpr std::integral_constant<int, 3> k3{};

    // Head: slabs 0 and 1 issued, the token rows of slab 2 under way.
    int tok[NJ];
    fetch_rows(0, tok);
    issue(0, tok);
    if (nk > 1) {
      fetch_rows(1, tok);
      issue(1, tok);
    }
    if (nk > 2) fetch_rows(2, tok);
    dma_wait_barrier<0>();
    if (nk == 1 && last_rows < kBK) clear_tail(0);
    reads(0, 0, k0, 0, 8);
    // Slab kt in stage u; on entry slab kt + 1 is issued and tok holds the token rows of slab kt + 2.
    auto body = [&](int u, int kt) {
      step(0, u, k1, true, false, 0, tok);
      step(1, u, k2, true, false, 0, tok);
      step(0, u, k3, true, false, 0, tok);
      dma_wait_barrier<0>();  // every wave has read the last of stage u; slab kt + 1 has landed in the other stage
      if (kt + 2 == nk && last_rows < kBK) clear_tail(u ^ 1);
      step(1, u ^ 1, k0, kt + 1 < nk, kt + 2 < nk, u, tok);
      if (kt + 3 < nk) fetch_rows(kt + 3, tok);
    };
    for (int kt = 0; kt < nk; kt += 2) {
      body(0, kt);
      if (kt + 1 < nk) body(1, kt + 1);
    }
  }
  splitk_store<Cfg>(g, acc, grp, split, r0, c0, rl);
#endif
}

// Workgroups of a launch that runs the gathered weight-gradient GEMM: a multiple of the XCD count.
inline int gathered_dw_blocks(int R, int Cc, int splits) {
  const int64_t total = 2LL * cdiv(R, GatherDwCfg::BN) * cdiv(Cc, GatherDwCfg::BM) * splits;
  return (int)(cdiv64(total, kXcds) * kXcds);
}

}  // namespace ffnk
