// Layout passes around the backward GEMMs.  The reference README (README.md:159-172) splits a
// backward into "an elementwise pass, then a fused GEMM"; for MaskedLinear the elementwise pass
// is the routed gather/transpose below, which turns every contraction of the backward into the
// K-contiguous form the MFMA core wants.
#include "common.hpp"
#include "launch.hpp"
#include "gemm_sched.hpp"

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

// dst[r, c] = src[c * sc + r] (a transpose: the source is contiguous along r).  64x64 tile per block:
// 16-byte reads along r, scalar transposing LDS writes, 16-byte reads of the transposed tile, 16-byte
// stores along c.  rows, cols, sc, ld_dst multiples of 8; 16-byte aligned bases.
__global__ __launch_bounds__(256) void transpose_copy_kernel(const uint16_t* __restrict__ src, int64_t sc,
                                                             uint16_t* __restrict__ dst, int64_t ld_dst, int rows,
                                                             int cols) {
  __shared__ __attribute__((aligned(16))) uint16_t tile[kTt][kTt + 8];  // [r][c]
  const int r0 = blockIdx.y * kTt, c0 = blockIdx.x * kTt;
  const int t = threadIdx.x, ch = t & 7;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int ci = (t >> 3) + pass * 32;
    uint16_t v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (c0 + ci < cols && r0 + ch * 8 < rows)
      *reinterpret_cast<uint4*>(v) = *reinterpret_cast<const uint4*>(src + (int64_t)(c0 + ci) * sc + r0 + ch * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) tile[ch * 8 + e][ci] = v[e];
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int rr = (t >> 3) + pass * 32;
    if (r0 + rr < rows && c0 + ch * 8 < cols)
      *reinterpret_cast<uint4*>(dst + (int64_t)(r0 + rr) * ld_dst + c0 + ch * 8) =
          *reinterpret_cast<const uint4*>(&tile[rr][ch * 8]);
  }
}

hipError_t launch_strided_copy2d(const uint16_t* src, int64_t sr, int64_t sc, uint16_t* dst, int64_t ld_dst,
                                 int rows, int cols, hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return hipSuccess;
  if (sr == 1 && sc % 8 == 0 && ld_dst % 8 == 0 && rows % 8 == 0 && cols % 8 == 0 &&
      (reinterpret_cast<uintptr_t>(src) & 15) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
    dim3 grid(cdiv(cols, kTt), cdiv(rows, kTt));
    hipLaunchKernelGGL(transpose_copy_kernel, grid, dim3(256), 0, stream, src, sc, dst, ld_dst, rows, cols);
    return hipGetLastError();
  }
  dim3 grid(cdiv(cols, kTt), cdiv(rows, kTt));
  hipLaunchKernelGGL(strided_copy2d_kernel, grid, dim3(256), 0, stream, src, sr, sc, dst, ld_dst, rows, cols);
  return hipGetLastError();
}

// dst[c, pos] = src[perm[p], c] over padded routed positions pos in [0, pad64(nv) + pad64(nt));
// padding positions are written as zero so that they add nothing to a contraction over pos.
// blockIdx.z selects one of two (src, dst) pairs so that g and x are transposed in one launch.
// 64 positions x 64 columns per block: 16-byte row reads (two positions per thread), transposing LDS writes of
// one dword per pair of positions, 16-byte reads of the transposed tile, 16-byte stores (8 consecutive positions
// of one column).
struct GatherTransposeArgs {
  const uint16_t* src[2]; int64_t ld_src[2];
  uint16_t* dst[2]; int64_t ld_dst;
  int cols[2];
  const int32_t* perm; const int32_t* counts;
  int M;
  int routed[2];  // source rows already in routed order: row p instead of row perm[p]
};

__global__ __launch_bounds__(256) void gather_transpose_kernel(const GatherTransposeArgs a) {
  // [column][pair of positions], one dword per pair; the pair index is XORed with 4 * (column / 8 % 8), which keeps
  // the transposing writes (a half wave: 8 column chunks x 4 pairs) and the 16-byte reads free of bank conflicts.
  __shared__ __attribute__((aligned(16))) uint32_t tile[kTt][kTt / 2];
  static_assert(kTt == 64, "one pass of 256 threads: 32 position pairs x 8 column chunks");
  const int z = blockIdx.z;
  const int cols = a.cols[z];
  const int c0 = blockIdx.y * kTt;
  if (c0 >= cols) return;  // grid.y is sized for the wider of the two operands
  const int n_vis = a.counts[0];
  const int vpad = (n_vis + 63) & ~63;
  const int tpad = (a.M - n_vis + 63) & ~63;
  const int pos0 = blockIdx.x * kTt;
  if (pos0 >= vpad + tpad) return;  // grid.x is sized for the worst-case padding
  // A 64-position block lies entirely inside one group because vpad is a multiple of 64.
  const bool text = pos0 >= vpad;
  const uint16_t* src = a.src[z];
  const int64_t ld_src = a.ld_src[z];
  const int t = threadIdx.x;
  const int ch = t & 7;   // 8-column chunk of the 64-column tile
  const int pr = t >> 3;  // position pair inside the tile
  const int c = c0 + ch * 8;
  uint16_t v[2][8];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int pos = pos0 + 2 * pr + h;
    const int p = text ? n_vis + (pos - vpad) : pos;
    const bool valid = text ? p < a.M : p < n_vis;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[h][e] = 0;
    if (valid) {
      const uint16_t* row = src + (int64_t)(a.routed[z] ? p : a.perm[p]) * ld_src;
      if (c + 8 <= cols) {
        *reinterpret_cast<uint4*>(v[h]) = *reinterpret_cast<const uint4*>(row + c);  // cols % 8 == 0, 16-byte aligned rows
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (c + e < cols) v[h][e] = row[c + e];
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) tile[ch * 8 + e][pr ^ (ch << 2)] = (uint32_t)v[0][e] | ((uint32_t)v[1][e] << 16);
  __syncthreads();
  uint16_t* dst = a.dst[z];
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int cc = (t >> 3) + pass * 32;  // column inside the tile
    if (c0 + cc < cols)
      *reinterpret_cast<uint4*>(dst + (int64_t)(c0 + cc) * a.ld_dst + pos0 + ch * 8) =
          *reinterpret_cast<const uint4*>(&tile[cc][(ch ^ ((cc >> 3) & 7)) << 2]);
  }
}

hipError_t launch_gather_transpose2(const uint16_t* src0, int64_t ld0, int cols0, uint16_t* dst0,
                                    const uint16_t* src1, int64_t ld1, int cols1, uint16_t* dst1, int64_t ld_dst,
                                    const int32_t* perm, const int32_t* counts, int M, hipStream_t stream,
                                    bool routed0, bool routed1) {
  if (M <= 0 || (cols0 <= 0 && cols1 <= 0)) return hipSuccess;
  GatherTransposeArgs a;
  a.src[0] = src0; a.ld_src[0] = ld0; a.dst[0] = dst0; a.cols[0] = cols0;
  a.src[1] = src1; a.ld_src[1] = ld1; a.dst[1] = dst1; a.cols[1] = cols1;
  a.ld_dst = ld_dst; a.perm = perm; a.counts = counts; a.M = M;
  a.routed[0] = routed0; a.routed[1] = routed1;
  const int max_pos = (int)round_up64(M, 64) + 64;  // >= pad64(nv) + pad64(nt) for every split of M
  const int max_cols = cols0 > cols1 ? cols0 : cols1;
  dim3 grid(cdiv(max_pos, kTt), cdiv(max_cols, kTt), 2);
  hipLaunchKernelGGL(gather_transpose_kernel, grid, dim3(256), 0, stream, a);
  return hipGetLastError();
}

// SwiGLU backward in place (see launch.hpp); 8 columns per thread, fp32 maths, bf16 storage.  The
// derivative is the textbook one, silu'(t) = s + t s (1 - s) with s = sigmoid(t) (the reference's
// README.md:159-172 sketches this pass; its derivative term there is not this one and is not used).
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const uint16_t* pre, int64_t ld_pre, uint16_t* T13, int64_t ld13,
                                                         uint16_t* __restrict__ DH, int64_t ldh, int M, int h) {
  const int h8 = h >> 3;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)M * h8) return;
  const int p = (int)(idx / h8), j = (int)(idx % h8) * 8;
  const uint16_t* ps1 = pre + (int64_t)p * ld_pre + j;  // may be T13 itself (in place)
  uint16_t* pt1 = T13 + (int64_t)p * ld13 + j;
  uint16_t* pt3 = pt1 + h;
  uint16_t* pdh = DH + (int64_t)p * ldh + j;
  uint16_t t1[8], t3[8], dh[8];
  *reinterpret_cast<uint4*>(t1) = *reinterpret_cast<const uint4*>(ps1);
  *reinterpret_cast<uint4*>(t3) = *reinterpret_cast<const uint4*>(ps1 + h);
  *reinterpret_cast<uint4*>(dh) = *reinterpret_cast<const uint4*>(pdh);
  uint16_t o1[8], o3[8], oh[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float a = bf2f(t1[e]), b = bf2f(t3[e]), g = bf2f(dh[e]);
    const float s = 1.0f / (1.0f + __expf(-a));
    const float silu = a * s;
    o1[e] = f2bf(g * b * (s + silu * (1.0f - s)));
    o3[e] = f2bf(g * silu);
    oh[e] = f2bf(silu * b);
  }
  *reinterpret_cast<uint4*>(pt1) = *reinterpret_cast<const uint4*>(o1);
  *reinterpret_cast<uint4*>(pt3) = *reinterpret_cast<const uint4*>(o3);
  *reinterpret_cast<uint4*>(pdh) = *reinterpret_cast<const uint4*>(oh);
}

hipError_t launch_swiglu_bwd(const uint16_t* pre, int64_t ld_pre, uint16_t* T13, int64_t ld13, uint16_t* DH, int64_t ldh,
                             int M, int h, hipStream_t stream) {
  if (M <= 0 || h <= 0) return hipSuccess;
  if (h % 8 != 0 || ld13 % 8 != 0 || ldh % 8 != 0 || ld_pre % 8 != 0) return hipErrorInvalidValue;
  const int64_t n = (int64_t)M * (h / 8);
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3((unsigned)cdiv64(n, 256)), dim3(256), 0, stream, pre, ld_pre, T13, ld13, DH,
                     ldh, M, h);
  return hipGetLastError();
}

// out_g[r * sr + c * sc] = bf16(P[g][0][r][c] + P[g][1][r][c] + ...), summed in split order so
// that the result does not depend on scheduling.  VEC: four consecutive columns per thread (16-byte loads of the
// partials, one 8-byte store), for outputs whose columns are contiguous (sc == 1) and Cc % 4 == 0.
template <bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ P, int splits, int R, int Cc,
                                                            uint16_t* __restrict__ out0,
                                                            uint16_t* __restrict__ out1, int64_t sr, int64_t sc) {
  const int64_t plane = (int64_t)R * Cc;
  const int64_t idx = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * (VEC ? 4 : 1);
  if (idx >= plane) return;
  const int g = blockIdx.y;
  const float* p = P + (int64_t)g * splits * plane + idx;
  uint16_t* out = g == 0 ? out0 : out1;
  const int r = (int)(idx / Cc), c = (int)(idx % Cc);
  if constexpr (VEC) {
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = 0; k < splits; ++k) {
      const float4 v = *reinterpret_cast<const float4*>(p + (int64_t)k * plane);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    uint2 v2;
    v2.x = pack2bf(s.x, s.y);
    v2.y = pack2bf(s.z, s.w);
    *reinterpret_cast<uint2*>(out + (int64_t)r * sr + c) = v2;
  } else {
    float s = 0.f;
    for (int k = 0; k < splits; ++k) s += p[(int64_t)k * plane];
    out[(int64_t)r * sr + (int64_t)c * sc] = f2bf(s);
  }
}

hipError_t launch_splitk_reduce(const float* P, int splits, int R, int Cc, uint16_t* out0, uint16_t* out1,
                                int64_t sr, int64_t sc, hipStream_t stream) {
  if (R <= 0 || Cc <= 0) return hipSuccess;
  const int64_t plane = (int64_t)R * Cc;
  const bool vec = sc == 1 && Cc % 4 == 0 && sr % 4 == 0 && ((reinterpret_cast<uintptr_t>(out0) | reinterpret_cast<uintptr_t>(out1)) & 7) == 0 &&
                   (reinterpret_cast<uintptr_t>(P) & 15) == 0;
  if (vec) {
    dim3 grid((unsigned)cdiv64(plane / 4, 256), 2);
    hipLaunchKernelGGL(splitk_reduce_kernel<true>, grid, dim3(256), 0, stream, P, splits, R, Cc, out0, out1, sr, sc);
  } else {
    dim3 grid((unsigned)cdiv64(plane, 256), 2);
    hipLaunchKernelGGL(splitk_reduce_kernel<false>, grid, dim3(256), 0, stream, P, splits, R, Cc, out0, out1, sr, sc);
  }
  return hipGetLastError();
}

// out[perm[p], n] = bf16(P[0][p][n] + P[1][p][n] + ...) in split order: the reduce pass of a split-K
// routed GEMM.  One workgroup per (routed row, 1024 columns); N % 4 == 0.
__global__ __launch_bounds__(256) void routed_reduce_kernel(const float* __restrict__ P, int splits, int M, int N,
                                                            const int32_t* __restrict__ perm,
                                                            uint16_t* __restrict__ out, int64_t ldo) {
  const int p = blockIdx.y;
  const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (n >= N) return;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = 0; k < splits; ++k) {
    const float4 v = *reinterpret_cast<const float4*>(P + ((int64_t)k * M + p) * N + n);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  uint16_t* o = out + (int64_t)perm[p] * ldo + n;
  if ((reinterpret_cast<uintptr_t>(o) & 7) == 0) {
    uint2 v2;
    v2.x = pack2bf(s.x, s.y);
    v2.y = pack2bf(s.z, s.w);
    *reinterpret_cast<uint2*>(o) = v2;
  } else {
    o[0] = f2bf(s.x); o[1] = f2bf(s.y); o[2] = f2bf(s.z); o[3] = f2bf(s.w);
  }
}

hipError_t launch_routed_reduce(const float* P, int splits, int M, int N, const int32_t* perm, uint16_t* out,
                                int64_t ldo, hipStream_t stream) {
  if (M <= 0 || N <= 0) return hipSuccess;
  dim3 grid((unsigned)cdiv(N, 1024), (unsigned)M);
  hipLaunchKernelGGL(routed_reduce_kernel, grid, dim3(256), 0, stream, P, splits, M, N, perm, out, ldo);
  return hipGetLastError();
}

// Reduce pass of a split tail (see GemmArgs::P_tail): workgroups (i, 0 .. kTailRowChunks - 1) add the K
// ranges of tail tile i, one band of rows each, and scatter the rows, C[perm[p], n] = bf16(sum_k P_tail[k * n_tail + i][p - row0][n - n0]).
// Recomputes the GEMM kernel's schedule from counts[]; exits when the tail was not split.
constexpr int kTailRowChunks = 16;  // row bands per tile in the tail reduce: enough workgroups to fill the chip from 16 tiles

__global__ __launch_bounds__(256) void routed_tail_reduce_kernel(const float* __restrict__ P_tail, int M, int N, int K,
                                                                 const int32_t* __restrict__ counts,
                                                                 const int32_t* __restrict__ perm, int bm, int bn,
                                                                 int group_m, uint16_t* __restrict__ C, int64_t ldc) {
  const int n_vis = counts[0];
  const int total = routed_tile_count(n_vis, M, N, bm, bn);
  const int full = total / kCusPerChip * kCusPerChip;
  const int n_tail = total - full;
  const int tile_i = blockIdx.x;
  if (tile_i >= n_tail) return;
  const int splits = tail_split_factor(n_tail, K / 64);
  if (splits == 1) return;  // the GEMM stored this tile itself
  const TileCoord tc = routed_tile_coord(full + tile_i, n_vis, M, N, bm, bn, group_m);
  const int quads = bn / 4;                   // float4 columns per tile row
  const int rows_per_pass = 256 / quads;
  const int q = threadIdx.x % quads;
  const int n = tc.n0 + 4 * q;
  if (n >= N) return;
  const int64_t tile_elems = (int64_t)bm * bn;
  const int band = bm / kTailRowChunks;
  for (int r = blockIdx.y * band + threadIdx.x / quads; r < (blockIdx.y + 1) * band; r += rows_per_pass) {
    const int p = tc.row0 + r;
    if (p >= tc.row_end) break;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = 0; k < splits; ++k) {
      const float4 v = *reinterpret_cast<const float4*>(P_tail + ((int64_t)k * n_tail + tile_i) * tile_elems + (int64_t)r * bn + 4 * q);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    uint16_t* o = C + (int64_t)perm[p] * ldc + n;
    if (n + 3 < N && (reinterpret_cast<uintptr_t>(o) & 7) == 0) {
      uint2 v2;
      v2.x = pack2bf(s.x, s.y);
      v2.y = pack2bf(s.z, s.w);
      *reinterpret_cast<uint2*>(o) = v2;
    } else {
      const float e[4] = {s.x, s.y, s.z, s.w};
      for (int i = 0; i < 4; ++i)
        if (n + i < N) o[i] = f2bf(e[i]);
    }
  }
}

hipError_t launch_routed_tail_reduce(const float* P_tail, int M, int N, int K, const int32_t* counts,
                                     const int32_t* perm, int bm, int bn, int group_m, uint16_t* C, int64_t ldc,
                                     hipStream_t stream) {
  if (M <= 0 || N <= 0 || bn % 4 != 0 || 256 % (bn / 4) != 0 || bm % kTailRowChunks != 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(routed_tail_reduce_kernel, dim3(kTailSlots, kTailRowChunks), dim3(256), 0, stream, P_tail, M, N, K, counts, perm, bm,
                     bn, group_m, C, ldc);
  return hipGetLastError();
}

}  // namespace ffnk
