// The tile shapes every GEMM kind is instantiated for, and the switch that picks one at run time.
#pragma once
#include "gemm_nt.hpp"
#include "launch.hpp"

namespace ffnk {

// LDS stages of the 256x256 single-weight tiles on the direct path: 3 = token panel in a ring of three stages, weight
// panel in two (gemm_mainloop_fixed16).  Measured on the same box against two stages of both: down projection at
// M = 32768, K = 14336 -3.5 to -4.2 % (2.66 -> 2.55 ms), at M = 1024 -9 % (159 -> 145 us), at M = 4096 -2.3 %.  The
// SwiGLU tiles keep two stages: the ring measured between -0.8 % and +1.3 % there over three boxes (a tile's head
// issues two slabs of loads in one burst, which weighs more on a 64-slab contraction than on a 224-slab one), and
// so did the weight panel in the ring instead of the token panel.
constexpr int kBigStagesPlain = 3;
constexpr int kGroupM = 8;       // M-tiles per L2 super-group in the tile order of the SwiGLU GEMM (4: the same, 16 costs 6 % at d=4096, h=14336)
constexpr int kGroupMPlain = 4;  // single-weight GEMMs: long contractions make wide token panels, 4 x 8 tiles per XCD round re-read fewer of them (1-2 % at K=14336)

// Plain (single-weight) tiles: BN = output columns.
template <bool GATHER, bool SCATTER, bool DIRECT>
struct PlainTiles {
  using T0 = RoutedGemmCfg<256, 256, 2, 4, false, GATHER, SCATTER, DIRECT, kGroupMPlain, false, DIRECT ? kBigStagesPlain : 2>;
  using T1 = RoutedGemmCfg<256, 256, 2, 2, false, GATHER, SCATTER, DIRECT, kGroupMPlain, false, DIRECT ? kBigStagesPlain : 2>;
  using T2 = RoutedGemmCfg<128, 128, 2, 2, false, GATHER, SCATTER, DIRECT, kGroupMPlain>;
  using T3 = RoutedGemmCfg<128, 64, 2, 2, false, GATHER, SCATTER, DIRECT, kGroupMPlain>;
  // 128x128 behind a ring of four LDS stages (direct path; otherwise the two-stage tile)
  using T4 = RoutedGemmCfg<128, 128, 2, 2, false, GATHER, SCATTER, DIRECT, kGroupMPlain, false, DIRECT ? 4 : 2>;
};

// The same tiles over K-major weights ([K, N] rows, N contiguous; direct path only).
template <bool GATHER, bool SCATTER>
struct KMajorTiles {
  using T0 = RoutedGemmCfg<256, 256, 2, 4, false, GATHER, SCATTER, true, kGroupM, true, kBigStagesPlain>;
  using T1 = RoutedGemmCfg<256, 256, 2, 2, false, GATHER, SCATTER, true, kGroupM, true, kBigStagesPlain>;
  using T2 = RoutedGemmCfg<128, 128, 2, 2, false, GATHER, SCATTER, true, kGroupM, true>;
  using T3 = RoutedGemmCfg<128, 64, 2, 2, false, GATHER, SCATTER, true, kGroupM, true>;
  // 128x128 behind a ring of four LDS stages, for the routed GEMMs (the weight-gradient GEMMs, whose last slab is
  // ragged and cleared in LDS, stay on the two-stage tile)
  using T4 = RoutedGemmCfg<128, 128, 2, 2, false, GATHER, SCATTER, true, kGroupM, true, 4>;
};

// SwiGLU tiles: BN = gate rows + up rows held in LDS, i.e. BN / 2 output columns.
template <bool DIRECT>
struct DualTiles {
  using T0 = RoutedGemmCfg<256, 256, 2, 4, true, true, false, DIRECT, kGroupM>;
  using T1 = RoutedGemmCfg<256, 256, 2, 2, true, true, false, DIRECT, kGroupM>;
  using T2 = RoutedGemmCfg<128, 128, 2, 2, true, true, false, DIRECT, kGroupM>;
  using T3 = RoutedGemmCfg<64, 128, 2, 2, true, true, false, DIRECT, kGroupM>;
  using T4 = RoutedGemmCfg<128, 128, 2, 2, true, true, false, DIRECT, kGroupM, false, DIRECT ? 4 : 2>;
};

template <class Tiles>
inline hipError_t dispatch_tile(int tile, const GemmArgs& g, hipStream_t stream) {
  switch (tile) {
    case TILE_256x256_W8: return launch_routed_gemm<typename Tiles::T0>(g, stream);
    case TILE_256x256_W4:
      // The four-wave tile exists on the direct path only: staged through registers its 256 accumulators and the
      // staging registers do not fit (the compiler spills some 430 of them); the eight-wave tile covers the same
      // macro tile with half the accumulators per lane.
      if constexpr (Tiles::T1::DIRECT) return launch_routed_gemm<typename Tiles::T1>(g, stream);
      else return launch_routed_gemm<typename Tiles::T0>(g, stream);
    case TILE_128x128_W4: return launch_routed_gemm<typename Tiles::T2>(g, stream);
    case TILE_SMALL_W4: return launch_routed_gemm<typename Tiles::T3>(g, stream);
    case TILE_128x128_R4: return launch_routed_gemm<typename Tiles::T4>(g, stream);
    default: return hipErrorInvalidValue;
  }
}

// GEMMs on the 256x256 tile: when the tile count is not a multiple of the CU count, the last
// round would run a few tiles on a few CUs for a full tile time (2064 tiles at M = 32768, N = 4096:
// 8 rounds + 16 tiles).  Run the whole rounds with the big tile and the remainder in a second
// launch: as 128x128 tiles (128 rows x 64 gate + 64 up columns for the SwiGLU kernel), or, with
// GemmArgs::P_tail, on the big tile cut into K ranges plus a reduce pass (a shorter tail: 0.20 -> 0.05 ms
// at the shape above).  Either way the rows of the remainder's tiles are summed in another fp32 order than
// the rows of the whole rounds (32x32x16 MFMAs over 16-element K steps, or partial sums per K range,
// against 16x16x32 MFMAs over 32-element steps): which launch a row falls into depends on the mask and on
// the batch, so a row's result is reproducible for a given call but agrees between differently composed
// calls only to fp32 summation accuracy - far inside the bf16 rounding of the output, and the bound the
// batch-composition test states.
template <class Tiles, class Big>
inline hipError_t dispatch_big_tile_with_tail(const GemmArgs& g, hipStream_t stream) {
  using Small = typename Tiles::T2;
  GemmArgs a = g;
  a.tail_mode = 1;
  if (hipError_t e = launch_routed_gemm<Big>(a, stream)) return e;
  if (!Big::DUAL && Big::SCATTER_C && g.P_tail != nullptr) {
    // Split tail: the remaining tiles on the big tile, each cut into K ranges (at most kTailSlots
    // (tile, range) pairs), then the reduce pass.
    a.tail_mode = 3;
    hipLaunchKernelGGL(routed_gemm_kernel<Big>, dim3(kTailSlots), dim3(Big::NT), 0, stream, a);
    if (hipError_t e = hipGetLastError()) return e;
    return launch_routed_tail_reduce(g.P_tail, g.M, g.N, g.K, g.counts, g.perm, Big::BM, Big::BN_OUT, g.group_m > 0 ? g.group_m : Big::GROUP_M, g.C,
                                     g.ldc, stream);
  }
  a.tail_mode = 2;
  a.sched_bm = Big::BM;
  a.sched_bn = Big::BN_OUT;
  constexpr int q = (Big::BM / Small::BM) * (Big::BN_OUT / Small::BN_OUT);
  hipLaunchKernelGGL(routed_gemm_kernel<Small>, dim3((kCusPerChip - 1) * q), dim3(Small::NT), 0, stream, a);
  return hipGetLastError();
}

template <class Tiles>
inline hipError_t dispatch_tile_with_tail(int tile, const GemmArgs& g, hipStream_t stream) {
  if (!is_big_tile(tile) || g.splits > 1 || g.M <= 0 || g.N <= 0) return dispatch_tile<Tiles>(tile, g, stream);
  // At most one round of big tiles: nothing to split off (every tile would land in the remainder).
  if ((int64_t)(cdiv(g.M, Tiles::T0::BM) + 1) * cdiv(g.N, Tiles::T0::BN_OUT) <= kCusPerChip)
    return dispatch_tile<Tiles>(tile, g, stream);
  return tile == TILE_256x256_W8 ? dispatch_big_tile_with_tail<Tiles, typename Tiles::T0>(g, stream)
                                 : dispatch_big_tile_with_tail<Tiles, typename Tiles::T1>(g, stream);
}

}  // namespace ffnk
