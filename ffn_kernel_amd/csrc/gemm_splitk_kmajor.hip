// Weight-gradient GEMM of the MaskedFFN backward with one operand read where it lies: the rows of
// H, dt1 or dt3 (routed order) are the contraction rows, turned into MFMA operands by the transposing
// LDS read; the other operand is the 64-padded transpose of the gathered x or g.
#include "gemm_tiles.hpp"

namespace ffnk {

hipError_t launch_splitk_gemm_kmajor(int tile, const SplitKArgs& g, hipStream_t stream) {
  using Tiles = KMajorTiles<false, false>;
  switch (tile) {
    case TILE_256x256_W8: return launch_grouped_splitk<Tiles::T0>(g, stream);
    case TILE_256x256_W4: return launch_grouped_splitk<Tiles::T1>(g, stream);
    case TILE_128x128_W4: return launch_grouped_splitk<Tiles::T2>(g, stream);
    case TILE_SMALL_W4: return launch_grouped_splitk<Tiles::T3>(g, stream);
    case TILE_128x128_R4: return launch_grouped_splitk<Tiles::T2>(g, stream);  // no ring here: the group's last slab is cleared in LDS
    default: return hipErrorInvalidValue;
  }
}

}  // namespace ffnk
