// MaskedLinear backward: the dx GEMM (on the weights where they lie, K-major) and the weight-gradient
// GEMM in one launch (fused_bwd_kernel), both on 128x128 tiles: two LDS stages and two workgroups per CU,
// or (ring) four stages and one workgroup per CU.
#include "gemm_tiles.hpp"

namespace ffnk {

using FusedDx = KMajorTiles<true, true>::T2;
using FusedDw = PlainTiles<false, false, true>::T2;
using RingDx = KMajorTiles<true, true>::T4;
using RingDw = PlainTiles<false, false, true>::T4;
static_assert(FusedDx::BM == RingDx::BM && FusedDx::BN_OUT == RingDx::BN_OUT && FusedDw::BM == RingDw::BM && FusedDw::BN == RingDw::BN,
              "both forms of the fused launch cut the same tiles");

int fused_bwd_dw_blocks(int R, int Cc, int splits) {
  const int64_t total = 2LL * cdiv(R, FusedDw::BN) * cdiv(Cc, FusedDw::BM) * splits;
  return (int)(cdiv64(total, kXcds) * kXcds);  // a multiple of the XCD count: the dx tiles keep their XCD mapping
}

hipError_t launch_fused_bwd(const GemmArgs& gx, const SplitKArgs& gw, bool ring, hipStream_t stream) {
  if (gx.M <= 0 || gx.N <= 0 || gw.R <= 0 || gw.Cc <= 0 || gw.splits <= 0) return hipErrorInvalidValue;
  if (gx.splits != 1 || gx.tail_mode != 0 || gx.k_switch != 0) return hipErrorInvalidValue;
  if (gx.N % 8 != 0 || gx.K % kBK != 0 || gx.ldb * (kBK * 2) + 2 * (int64_t)gx.N >= ((int64_t)1 << 32)) return hipErrorInvalidValue;
  const int dw_blocks = fused_bwd_dw_blocks(gw.R, gw.Cc, gw.splits);
  const int dx_blocks = routed_gemm_grid<FusedDx>(gx.M, gx.N);
  if (ring)
    hipLaunchKernelGGL((fused_bwd_kernel<RingDx, RingDw>), dim3(dw_blocks + dx_blocks), dim3(RingDx::NT), 0, stream, gx, gw,
                       dw_blocks);
  else
    hipLaunchKernelGGL((fused_bwd_kernel<FusedDx, FusedDw>), dim3(dw_blocks + dx_blocks), dim3(FusedDx::NT), 0, stream, gx, gw,
                       dw_blocks);
  return hipGetLastError();
}

}  // namespace ffnk
