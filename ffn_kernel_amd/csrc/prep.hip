// Layout passes around the backward GEMMs.  The reference README (README.md:159-172) splits a
// backward into "an elementwise pass, then a fused GEMM"; for MaskedLinear the elementwise pass
// is the routed gather/transpose below, which turns every contraction of the backward into the
// K-contiguous form the MFMA core wants.
#include "common.hpp"
#include "launch.hpp"

namespace ffnk {

constexpr int kTt = 64;  // transpose tile edge

// dst[r, c] = src[r * sr + c * sc].  One 64x64 tile per block, staged through LDS so that both
// the reads (along whichever source axis has the smaller stride) and the writes are contiguous.
__global__ __launch_bounds__(256) void strided_copy2d_kernel(const uint16_t* __restrict__ src, int64_t sr,
                                                             int64_t sc, uint16_t* __restrict__ dst,
                                                             int64_t ld_dst, int rows, int cols) {
  __shared__ uint16_t tile[kTt][kTt + 2];
  const int r0 = blockIdx.y * kTt, c0 = blockIdx.x * kTt;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 64 x 4
  const bool col_fast = (sc <= sr);  // read with tx along the faster source axis
  for (int i = ty; i < kTt; i += 4) {
    const int r = col_fast ? r0 + i : r0 + tx;
    const int c = col_fast ? c0 + tx : c0 + i;
    if (r < rows && c < cols) tile[r - r0][c - c0] = src[(int64_t)r * sr + (int64_t)c * sc];
  }
  __syncthreads();
  for (int i = ty; i < kTt; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    if (r < rows && c < cols) dst[(int64_t)r * ld_dst + c] = tile[i][tx];
  }
}

hipError_t launch_strided_copy2d(const uint16_t* src, int64_t sr, int64_t sc, uint16_t* dst, int64_t ld_dst,
                                 int rows, int cols, hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return hipSuccess;
  dim3 grid(cdiv(cols, kTt), cdiv(rows, kTt));
  hipLaunchKernelGGL(strided_copy2d_kernel, grid, dim3(256), 0, stream, src, sr, sc, dst, ld_dst, rows, cols);
  return hipGetLastError();
}

// dst[c, pos] = src[perm[p], c] over padded routed positions pos in [0, pad64(nv) + pad64(nt));
// padding positions are written as zero so that they add nothing to a contraction over pos.
__global__ __launch_bounds__(256) void gather_transpose_kernel(const uint16_t* __restrict__ src, int64_t ld_src,
                                                               const int32_t* __restrict__ perm,
                                                               const int32_t* __restrict__ counts,
                                                               uint16_t* __restrict__ dst, int64_t ld_dst, int M,
                                                               int cols) {
  __shared__ uint16_t tile[kTt][kTt + 2];  // [routed position][column]
  const int n_vis = counts[0];
  const int vpad = (n_vis + 63) & ~63;
  const int tpad = (M - n_vis + 63) & ~63;
  const int pos0 = blockIdx.x * kTt;
  if (pos0 >= vpad + tpad) return;  // grid is sized for the worst-case padding
  const int c0 = blockIdx.y * kTt;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  // A 64-position block lies entirely inside one group because vpad is a multiple of 64.
  const bool text = pos0 >= vpad;
  for (int i = ty; i < kTt; i += 4) {
    const int pos = pos0 + i;
    const int p = text ? n_vis + (pos - vpad) : pos;
    const bool valid = text ? p < M : p < n_vis;
    uint16_t v = 0;
    const int c = c0 + tx;
    if (valid && c < cols) v = src[(int64_t)perm[p] * ld_src + c];
    tile[i][tx] = v;
  }
  __syncthreads();
  for (int i = ty; i < kTt; i += 4) {
    const int c = c0 + i;
    if (c < cols) dst[(int64_t)c * ld_dst + pos0 + tx] = tile[tx][i];
  }
}

hipError_t launch_gather_transpose(const uint16_t* src, int64_t ld_src, const int32_t* perm,
                                   const int32_t* counts, uint16_t* dst, int64_t ld_dst, int M, int cols,
                                   hipStream_t stream) {
  if (M <= 0 || cols <= 0) return hipSuccess;
  const int max_pos = (int)round_up64(M, 64) + 64;  // >= pad64(nv) + pad64(nt) for every split of M
  dim3 grid(cdiv(max_pos, kTt), cdiv(cols, kTt));
  hipLaunchKernelGGL(gather_transpose_kernel, grid, dim3(256), 0, stream, src, ld_src, perm, counts, dst, ld_dst,
                     M, cols);
  return hipGetLastError();
}

// out_g[r * sr + c * sc] = bf16(P[g][0][r][c] + P[g][1][r][c] + ...), summed in split order so
// that the result does not depend on scheduling.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ P, int splits, int R, int Cc,
                                                            uint16_t* __restrict__ out0,
                                                            uint16_t* __restrict__ out1, int64_t sr, int64_t sc) {
  const int64_t plane = (int64_t)R * Cc;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= plane) return;
  const int g = blockIdx.y;
  const float* p = P + (int64_t)g * splits * plane + idx;
  float s = 0.f;
  for (int k = 0; k < splits; ++k) s += p[(int64_t)k * plane];
  const int r = (int)(idx / Cc), c = (int)(idx % Cc);
  uint16_t* out = g == 0 ? out0 : out1;
  out[(int64_t)r * sr + (int64_t)c * sc] = f2bf(s);
}

hipError_t launch_splitk_reduce(const float* P, int splits, int R, int Cc, uint16_t* out0, uint16_t* out1,
                                int64_t sr, int64_t sc, hipStream_t stream) {
  if (R <= 0 || Cc <= 0) return hipSuccess;
  const int64_t plane = (int64_t)R * Cc;
  dim3 grid((unsigned)cdiv64(plane, 256), 2);
  hipLaunchKernelGGL(splitk_reduce_kernel, grid, dim3(256), 0, stream, P, splits, R, Cc, out0, out1, sr, sc);
  return hipGetLastError();
}

}  // namespace ffnk
