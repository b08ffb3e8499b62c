// Any-stride scalar kernels.  The reference passes strides straight through to its kernels
// (ffn_kernel/linear.py:441-444) and masks every load, so it accepts operands the MFMA path
// cannot address with 16-byte loads (K not a multiple of 8, odd row strides, unaligned views).
// These kernels cover those calls: one thread per output element, fp32 accumulation, the mask
// tested per row exactly as the reference does.  They are a completeness path, not a fast one.
#include "common.hpp"
#include "launch.hpp"

namespace ffnk {

inline int grid_y(int blocks) { return blocks < 65535 ? blocks : 65535; }  // the launch limit of grid.y

__global__ __launch_bounds__(256) void generic_linear_kernel(const GenericLinearArgs a) {
  const int m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= a.M) return;
  const uint16_t* w = a.mask[m] ? a.W[0] : a.W[1];
  const uint16_t* xr = a.x + (int64_t)m * a.sxm;
  for (int n = blockIdx.y * 64 + (threadIdx.x & 63); n < a.N; n += gridDim.y * 64) {
    float acc = 0.f;
    for (int k = 0; k < a.K; ++k) acc += bf2f(xr[(int64_t)k * a.sxk]) * bf2f(w[(int64_t)k * a.swk + (int64_t)n * a.swn]);
    a.y[(int64_t)m * a.sym + (int64_t)n * a.syn] = f2bf(acc);
  }
}

hipError_t launch_generic_linear(const GenericLinearArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0) return hipSuccess;
  dim3 grid(cdiv(a.M, 4), grid_y(cdiv(a.N, 64)));  // rows on x; the kernel walks column blocks gridDim.y apart
  hipLaunchKernelGGL(generic_linear_kernel, grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

__global__ __launch_bounds__(256) void generic_up_kernel(const GenericUpArgs a) {
  const int m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= a.M) return;
  const int grp = a.mask[m] ? 0 : 1;
  const uint16_t* wg = a.G[grp];
  const uint16_t* wu = a.U[grp];
  const uint16_t* xr = a.x + (int64_t)m * a.sxm;
  for (int n = blockIdx.y * 64 + (threadIdx.x & 63); n < a.N; n += gridDim.y * 64) {
    float g = 0.f, u = 0.f;
    for (int k = 0; k < a.K; ++k) {
      const float xv = bf2f(xr[k]);
      const int64_t o = (int64_t)k * a.swk + (int64_t)n * a.swn;
      g += xv * bf2f(wg[o]);
      u += xv * bf2f(wu[o]);
    }
    a.H[(int64_t)m * a.ldh + n] = f2bf(swiglu(g, u));
  }
}

hipError_t launch_generic_up(const GenericUpArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0) return hipSuccess;
  dim3 grid(cdiv(a.M, 4), grid_y(cdiv(a.N, 64)));  // rows on x; the kernel walks column blocks gridDim.y apart
  hipLaunchKernelGGL(generic_up_kernel, grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

// dx[m, k] = sum_n g[m, n] * W_mask[m][k, n]
__global__ __launch_bounds__(256) void generic_bwd_dx_kernel(const GenericBwdArgs a) {
  const int m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= a.M) return;
  const uint16_t* w = a.mask[m] ? a.W[0] : a.W[1];
  const uint16_t* gr = a.g + (int64_t)m * a.sgm;
  for (int k = blockIdx.y * 64 + (threadIdx.x & 63); k < a.K; k += gridDim.y * 64) {
    float acc = 0.f;
    for (int n = 0; n < a.N; ++n) acc += bf2f(gr[n]) * bf2f(w[(int64_t)k * a.swk + (int64_t)n * a.swn]);
    a.dx[(int64_t)m * a.sdxm + k] = f2bf(acc);
  }
}

// dW_v[k, n] = sum over visual rows of x[m, k] g[m, n]; dW_t likewise over text rows.  Rows are
// visited in ascending order by a single thread: deterministic, and a modality without rows
// gets exact zeros (the reference stores both accumulators unconditionally, linear.py:414-415).
__global__ __launch_bounds__(256) void generic_bwd_dw_kernel(const GenericBwdArgs a) {
  // K / 4 (up to 2^22 blocks) on grid.x; the 64-column blocks of N on grid.y, which is limited to
  // 65535 blocks: each block walks the column blocks gridDim.y apart
  const int k = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (k >= a.K) return;
  for (int n = blockIdx.y * 64 + (threadIdx.x & 63); n < a.N; n += gridDim.y * 64) {
    float av = 0.f, at = 0.f;
    for (int m = 0; m < a.M; ++m) {
      const float p = bf2f(a.x[(int64_t)m * a.sxm + k]) * bf2f(a.g[(int64_t)m * a.sgm + n]);
      if (a.mask[m]) av += p;
      else at += p;
    }
    const int64_t o = (int64_t)k * a.sdk + (int64_t)n * a.sdn;
    a.dW[0][o] = f2bf(av);
    a.dW[1][o] = f2bf(at);
  }
}

hipError_t launch_generic_bwd(const GenericBwdArgs& a, hipStream_t stream) {
  if (a.M > 0 && a.K > 0) {
    dim3 grid(cdiv(a.M, 4), grid_y(cdiv(a.K, 64)));
    hipLaunchKernelGGL(generic_bwd_dx_kernel, grid, dim3(256), 0, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  if (a.K > 0 && a.N > 0) {
    dim3 grid(cdiv(a.K, 4), grid_y(cdiv(a.N, 64)));
    hipLaunchKernelGGL(generic_bwd_dw_kernel, grid, dim3(256), 0, stream, a);
    return hipGetLastError();
  }
  return hipSuccess;
}

}  // namespace ffnk
