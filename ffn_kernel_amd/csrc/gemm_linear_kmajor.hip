// MaskedLinear dx GEMM over the weight as stored ([K, N] rows of the contraction, N contiguous):
// gathered A rows, scattered C rows.
#include "gemm_tiles.hpp"

namespace ffnk {

hipError_t launch_linear_gemm_kmajor(int tile, const GemmArgs& g, hipStream_t stream) {
  return dispatch_tile_with_tail<KMajorTiles<true, true>>(tile, g, stream);
}

}  // namespace ffnk
