// MaskedFFN backward dx GEMM over the up-projection weights as stored: A in routed order, C scattered
// to token order, the contraction running through the gate weight and on into the up weight.
#include "gemm_tiles.hpp"

namespace ffnk {

hipError_t launch_down_gemm_kmajor(int tile, const GemmArgs& g, hipStream_t stream) {
  return dispatch_tile_with_tail<KMajorTiles<false, true>>(tile, g, stream);
}

}  // namespace ffnk
