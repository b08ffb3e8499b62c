// MaskedFFN backward dH GEMM over the down-projection weight as stored: gathered A rows, C in routed
// order.
#include "gemm_tiles.hpp"

namespace ffnk {

hipError_t launch_gather_gemm_kmajor(int tile, const GemmArgs& g, hipStream_t stream) {
  return dispatch_tile_with_tail<KMajorTiles<true, false>>(tile, g, stream);
}

}  // namespace ffnk
