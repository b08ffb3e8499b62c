// MaskedLinear forward / dx GEMM: gathered A rows, scattered C rows, one weight per group.
#include "gemm_tiles.hpp"

namespace ffnk {

hipError_t launch_linear_gemm(int tile, bool direct, const GemmArgs& g, hipStream_t stream) {
  return direct ? dispatch_tile_with_tail<PlainTiles<true, true, true>>(tile, g, stream)
                : dispatch_tile<PlainTiles<true, true, false>>(tile, g, stream);
}

}  // namespace ffnk
