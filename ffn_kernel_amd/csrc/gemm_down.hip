// MaskedFFN down-projection (A = H in routed order, C scattered to token order) and the
// grouped split-K GEMM of the weight gradients.
#include "gemm_tiles.hpp"

namespace ffnk {

hipError_t launch_down_gemm(int tile, bool direct, const GemmArgs& g, hipStream_t stream) {
  return direct ? dispatch_tile_with_tail<PlainTiles<false, true, true>>(tile, g, stream)
                : dispatch_tile<PlainTiles<false, true, false>>(tile, g, stream);
}

hipError_t launch_splitk_gemm(int tile, const SplitKArgs& g, hipStream_t stream) {
  using Tiles = PlainTiles<false, false, true>;
  switch (tile) {
    case TILE_256x256_W8: return launch_grouped_splitk<Tiles::T0>(g, stream);
    case TILE_256x256_W4: return launch_grouped_splitk<Tiles::T1>(g, stream);
    case TILE_128x128_W4: return launch_grouped_splitk<Tiles::T2>(g, stream);
    case TILE_SMALL_W4: return launch_grouped_splitk<Tiles::T3>(g, stream);
    case TILE_128x128_R4: return launch_grouped_splitk<Tiles::T4>(g, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace ffnk
