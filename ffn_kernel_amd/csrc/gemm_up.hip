// MaskedFFN up-projection with the SwiGLU epilogue: gathered A rows, H written in routed order.
#include "gemm_tiles.hpp"

namespace ffnk {

hipError_t launch_up_gemm(int tile, bool direct, const GemmArgs& g, hipStream_t stream) {
  return direct ? dispatch_tile_with_tail<DualTiles<true>>(tile, g, stream)
                : dispatch_tile<DualTiles<false>>(tile, g, stream);
}

TileGeom tile_geom(int tile, bool dual) {
  switch (tile) {
    case TILE_256x256_W8: return {256, dual ? 128 : 256, 2, 4};
    case TILE_256x256_W4: return {256, dual ? 128 : 256, 2, 2};
    case TILE_128x128_W4:
    case TILE_128x128_R4: return {128, dual ? 64 : 128, 2, 2};
    default: return dual ? TileGeom{64, 64, 2, 2} : TileGeom{128, 64, 2, 2};
  }
}

}  // namespace ffnk
