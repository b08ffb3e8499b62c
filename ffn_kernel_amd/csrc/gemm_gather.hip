// Routed GEMM with gathered A rows and routed-order C rows, one weight per group: the pre-activations
// and the intermediate's gradient in the MaskedFFN backward (the up-projection kernel without its
// SwiGLU epilogue).
#include "gemm_tiles.hpp"

namespace ffnk {

hipError_t launch_gather_gemm(int tile, bool direct, const GemmArgs& g, hipStream_t stream) {
  return direct ? dispatch_tile_with_tail<PlainTiles<true, false, true>>(tile, g, stream)
                : dispatch_tile<PlainTiles<true, false, false>>(tile, g, stream);
}

}  // namespace ffnk
