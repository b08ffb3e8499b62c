// MaskedLinear backward: the dx GEMM (on the weights where they lie, K-major) and the weight-gradient
// GEMM in one launch (fused_bwd_kernel), both on 128x128 tiles: two LDS stages and two workgroups per CU,
// or (ring) four stages and one workgroup per CU.
#include "gemm_tiles.hpp"
#include "gemm_dw_gather.hpp"

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

// The same launch with the weight-gradient workgroups reading g and x where they lie (gathered_dw_body): no
// transposes, so the backward is this one launch behind the row partition.
template <class CfgDx>
__global__ __launch_bounds__(CfgDx::NT) void fused_bwd_gather_kernel(const GemmArgs gx, const GatherDwArgs gw, const int dw_blocks) {
  static_assert(CfgDx::NT == GatherDwCfg::NT, "one workgroup size for both GEMMs");
  constexpr int kLds = CfgDx::LDS_BYTES > GatherDwCfg::LDS_BYTES ? CfgDx::LDS_BYTES : GatherDwCfg::LDS_BYTES;
  __shared__ __attribute__((aligned(1024))) uint8_t lds[kLds];
  if ((int)blockIdx.x < dw_blocks) gathered_dw_body(gw, lds, (int)blockIdx.x);
  else routed_gemm_body<CfgDx>(gx, lds, (int)blockIdx.x - dw_blocks);
}

__global__ __launch_bounds__(GatherDwCfg::NT) void gathered_dw_kernel(const GatherDwArgs gw) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[GatherDwCfg::LDS_BYTES];
  gathered_dw_body(gw, lds, (int)blockIdx.x);
}

static bool gather_dw_args_ok(const GatherDwArgs& w) {
  constexpr int64_t k4g = (int64_t)1 << 32;
  const SplitKArgs& s = w.s;
  return s.R >= 8 && s.Cc >= 8 && s.R % 8 == 0 && s.Cc % 8 == 0 && s.splits >= 1 && s.M > 0 && w.ldg % 8 == 0 && w.ldx % 8 == 0 &&
         (int64_t)s.M * w.ldg * 2 + 2 * (int64_t)s.R < k4g && (int64_t)s.M * w.ldx * 2 + 2 * (int64_t)s.Cc < k4g &&
         (reinterpret_cast<uintptr_t>(w.G) & 15) == 0 && (reinterpret_cast<uintptr_t>(w.X) & 15) == 0;
}

hipError_t launch_gathered_dw(const GatherDwArgs& gw, hipStream_t stream) {
  if (!gather_dw_args_ok(gw)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(gathered_dw_kernel, dim3(gathered_dw_blocks(gw.s.R, gw.s.Cc, gw.s.splits)), dim3(GatherDwCfg::NT), 0, stream, gw);
  return hipGetLastError();
}

hipError_t launch_fused_bwd_gather(const GemmArgs& gx, const GatherDwArgs& gw, hipStream_t stream) {
  if (gx.M <= 0 || gx.N <= 0 || !gather_dw_args_ok(gw)) return hipErrorInvalidValue;
  if (gx.splits != 1 || gx.tail_mode != 0 || gx.k_switch != 0) return hipErrorInvalidValue;
  if (gx.N % 8 != 0 || gx.K % kBK != 0 || gx.ldb * (kBK * 2) + 2 * (int64_t)gx.N >= ((int64_t)1 << 32)) return hipErrorInvalidValue;
  const int dw_blocks = gathered_dw_blocks(gw.s.R, gw.s.Cc, gw.s.splits);
  const int dx_blocks = routed_gemm_grid<FusedDx>(gx.M, gx.N);
  hipLaunchKernelGGL((fused_bwd_gather_kernel<FusedDx>), dim3(dw_blocks + dx_blocks), dim3(FusedDx::NT), 0, stream, gx, gw, dw_blocks);
  return hipGetLastError();
}

}  // namespace ffnk
