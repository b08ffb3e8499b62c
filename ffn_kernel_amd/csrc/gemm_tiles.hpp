// The tile shapes every GEMM kind is instantiated for, and the switch that picks one at run time.
#pragma once
#include "gemm_nt.hpp"
#include "launch.hpp"

namespace ffnk {

constexpr int kGroupM = 8;  // M-tiles per L2 super-group in the tile order

// Plain (single-weight) tiles: BN = output columns.
template <bool GATHER, bool SCATTER, bool DIRECT>
struct PlainTiles {
  using T0 = RoutedGemmCfg<256, 256, 2, 4, false, GATHER, SCATTER, DIRECT, kGroupM>;
  using T1 = RoutedGemmCfg<256, 256, 2, 2, false, GATHER, SCATTER, DIRECT, kGroupM>;
  using T2 = RoutedGemmCfg<128, 128, 2, 2, false, GATHER, SCATTER, DIRECT, kGroupM>;
  using T3 = RoutedGemmCfg<128, 64, 2, 2, false, GATHER, SCATTER, DIRECT, kGroupM>;
};

// SwiGLU tiles: BN = gate rows + up rows held in LDS, i.e. BN / 2 output columns.
template <bool DIRECT>
struct DualTiles {
  using T0 = RoutedGemmCfg<256, 256, 2, 4, true, true, false, DIRECT, kGroupM>;
  using T1 = RoutedGemmCfg<256, 256, 2, 2, true, true, false, DIRECT, kGroupM>;
  using T2 = RoutedGemmCfg<128, 128, 2, 2, true, true, false, DIRECT, kGroupM>;
  using T3 = RoutedGemmCfg<64, 128, 2, 2, true, true, false, DIRECT, kGroupM>;
};

template <class Tiles>
inline hipError_t dispatch_tile(int tile, const GemmArgs& g, hipStream_t stream) {
  switch (tile) {
    case TILE_256x256_W8: return launch_routed_gemm<typename Tiles::T0>(g, stream);
    case TILE_256x256_W4: return launch_routed_gemm<typename Tiles::T1>(g, stream);
    case TILE_128x128_W4: return launch_routed_gemm<typename Tiles::T2>(g, stream);
    case TILE_SMALL_W4: return launch_routed_gemm<typename Tiles::T3>(g, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace ffnk
