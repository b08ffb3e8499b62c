// Host-side launch interface between the C ABI (capi.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "gemm_args.hpp"

namespace ffnk {

// ---- route.hip ----
hipError_t launch_route(const uint8_t* mask, int M, int32_t* perm, int32_t* counts, hipStream_t stream);

// ---- gemm_*.hip: LDS-tiled MFMA kernels ----
enum TileId : int {
  TILE_256x256_W8 = 0,  // 256x256 macro tile, 8 waves (2x4), wave tile 128x64
  TILE_256x256_W4 = 1,  // 256x256 macro tile, 4 waves (2x2), wave tile 128x128
  TILE_128x128_W4 = 2,  // 128x128 macro tile, 4 waves (2x2), wave tile 64x64
  TILE_SMALL_W4 = 3,    // 128x64 (plain) or 64x128 holding 64 gate + 64 up rows (SwiGLU), 4 waves
  TILE_128x128_R4 = 4,  // 128x128, 4 waves, ring of four LDS stages (one workgroup per CU; long contractions, few tiles)
  TILE_COUNT = 5
};

// The two 256x256 tiles: past one round of the chip they run whole rounds first and the remainder apart.
inline bool is_big_tile(int tile) { return tile == TILE_256x256_W8 || tile == TILE_256x256_W4; }

// Geometry of a tile id, as reported through ffnk_tile_config().
struct TileGeom {
  int block_m, block_n_out, waves_m, waves_n;
};
TileGeom tile_geom(int tile, bool dual);

// y = route-gather(x) @ W_g^T, scattered back to token order (MaskedLinear forward, and dx).
hipError_t launch_linear_gemm(int tile, bool direct, const GemmArgs& g, hipStream_t stream);
// H(routed order) = silu(gather(x) @ W1_g^T) * (gather(x) @ W3_g^T)
hipError_t launch_up_gemm(int tile, bool direct, const GemmArgs& g, hipStream_t stream);
// out(token order) = H(routed order) @ W2_g^T
hipError_t launch_down_gemm(int tile, bool direct, const GemmArgs& g, hipStream_t stream);
// C(routed order) = route-gather(A) @ B_g^T (MaskedFFN backward: pre-activations, dH)
hipError_t launch_gather_gemm(int tile, bool direct, const GemmArgs& g, hipStream_t stream);
// The three single-weight GEMMs above over K-major weights: B0[g] (and B1[g] past GemmArgs::k_switch)
// is [K, N] rows with N contiguous.  K % 64 == 0 and N % 8 == 0 are required.
hipError_t launch_linear_gemm_kmajor(int tile, const GemmArgs& g, hipStream_t stream);
hipError_t launch_down_gemm_kmajor(int tile, const GemmArgs& g, hipStream_t stream);
hipError_t launch_gather_gemm_kmajor(int tile, const GemmArgs& g, hipStream_t stream);
// P[grp][split] = A[:, kslice] @ B[:, kslice]^T (fp32 partials; weight gradients)
hipError_t launch_splitk_gemm(int tile, const SplitKArgs& g, hipStream_t stream);
// The same with A read in place: [rows, R] in routed order instead of a padded transpose (SplitKArgs).
hipError_t launch_splitk_gemm_kmajor(int tile, const SplitKArgs& g, hipStream_t stream);

// The MaskedLinear backward's dx GEMM (K-major weights, as launch_linear_gemm_kmajor on the 128x128 tile)
// and its weight-gradient GEMM (as launch_splitk_gemm on the 128x128 tile) in ONE launch: weight-gradient
// workgroups first, dx workgroups behind them.
// ring: both on the 128x128 tile behind four LDS stages (one workgroup per CU) instead of two stages (two per CU).
hipError_t launch_fused_bwd(const GemmArgs& gx, const SplitKArgs& gw, bool ring, hipStream_t stream);

// The weight-gradient GEMM of the MaskedLinear backward on g and x as they lie (no transposes; rows found through
// perm), alone or in one launch with the dx GEMM on the two-stage 128x128 tile.  hipErrorInvalidValue where the
// operands do not qualify (see GatherDwArgs).
hipError_t launch_gathered_dw(const GatherDwArgs& gw, hipStream_t stream);
hipError_t launch_fused_bwd_gather(const GemmArgs& gx, const GatherDwArgs& gw, hipStream_t stream);

// ---- prep.hip: layout passes around the GEMMs ----
// dst[r, c] (row-major, ld_dst) = src[r * sr + c * sc] for r < rows, c < cols.
hipError_t launch_strided_copy2d(const uint16_t* src, int64_t sr, int64_t sc, uint16_t* dst, int64_t ld_dst,
                                 int rows, int cols, hipStream_t stream);
// For both (src, dst) pairs: dst[c, pos(p)] = src[perm[p], c]; routed columns padded per group to a
// multiple of 64 with zeros: pos(p) = p for visual p, pad64(n_vis) + (p - n_vis) for text p.  dst is
// [cols, ld_dst]; cols % 8 == 0 and 16-byte aligned source rows are required.
hipError_t launch_gather_transpose2(const uint16_t* src0, int64_t ld0, int cols0, uint16_t* dst0,
                                    const uint16_t* src1, int64_t ld1, int cols1, uint16_t* dst1, int64_t ld_dst,
                                    const int32_t* perm, const int32_t* counts, int M, hipStream_t stream,
                                    bool routed0 = false, bool routed1 = false);
// routedN: source N's rows are already in routed order (row p instead of row perm[p]).

// SwiGLU backward, elementwise over routed-order rows (MaskedFFN backward):
//   t1 = pre[p, j], t3 = pre[p, h + j], dh = DH[p, j]
//   T13[p, j] <- dh * t3 * silu'(t1),  T13[p, h + j] <- dh * silu(t1),  DH[p, j] <- silu(t1) * t3
// pre, T13: [M, 2h] with row strides ld_pre, ld13 (pre may be T13: in place); DH: [M, h] row stride ldh;
// h % 8 == 0.
hipError_t launch_swiglu_bwd(const uint16_t* pre, int64_t ld_pre, uint16_t* T13, int64_t ld13, uint16_t* DH, int64_t ldh,
                             int M, int h, hipStream_t stream);
// out_g[r * sr + c * sc] = bf16(sum_s P[g][s][r][c]) for g in {0, 1}.
hipError_t launch_splitk_reduce(const float* P, int splits, int R, int Cc, uint16_t* out0, uint16_t* out1,
                                int64_t sr, int64_t sc, hipStream_t stream);

// out[perm[p], n] = bf16(sum_s P[s][p][n]): reduce pass of a split-K routed GEMM (N % 4 == 0, M < 65536).
hipError_t launch_routed_reduce(const float* P, int splits, int M, int N, const int32_t* perm, uint16_t* out,
                                int64_t ldo, hipStream_t stream);

// Reduce pass of a split tail (GemmArgs::P_tail) of a GEMM on bm x bn tiles with scatter epilogue.
hipError_t launch_routed_tail_reduce(const float* P_tail, int M, int N, int K, const int32_t* counts,
                                     const int32_t* perm, int bm, int bn, int group_m, uint16_t* C, int64_t ldc,
                                     hipStream_t stream);

// ---- stream.hip: weight-streaming kernels for M <= 64 ----
struct StreamArgs {
  const uint16_t* X; int64_t ldx;  // token rows: x [M, K] (gather_x = 1, token order) or H [M, K] (routed order)
  int gather_x;
  const uint8_t* mask; int M;      // M <= 64
  const uint16_t* W0[2];           // per group: weight rows [Nrows, K], K contiguous
  const uint16_t* W1[2];           // up-projection only: the second ("up") weight
  int64_t ldw;
  int Nrows, K, splits;            // K % 256 == 0; splits > 1 only for the down projection
  uint16_t* H; int64_t ldh;        // up-projection output, routed order [M, Nrows]
  float* P;                        // down-projection partials [splits][M][Nrows] (routed order), or NULL:
  uint16_t* out; int64_t ldo;      // ... splits == 1 and the result goes straight to out (token order)
};
// Shape of the streaming kernels for M rows (reported through ffnk_tile_config).
int stream_rows_per_block(int M, bool dual);  // weight rows (of each matrix) per workgroup
int stream_chunk_k(int M, bool dual);         // K elements per streamed chunk
int stream_waves_per_block(int M, bool dual); // wavefronts sharing one workgroup's K range
hipError_t launch_stream_up(const StreamArgs& a, hipStream_t stream);
hipError_t launch_stream_down(const StreamArgs& a, hipStream_t stream);
// stream_dot.hip: M <= 8, contiguous-row dot-product kernels (splits == 1, P unused, no reduce pass).
bool stream_dot_ok(int M, int K);
int stream_dot_slices_per_wave(int K);
int stream_dot_rows_per_block(int Nrows, bool dual, int K);
hipError_t launch_stream_dot_up(const StreamArgs& a, hipStream_t stream);
hipError_t launch_stream_dot_down(const StreamArgs& a, hipStream_t stream);
// stream_tile.hip: 9 <= M <= 64, contiguous loads + LDS transpose + shared token-row slab.
bool stream_tile_ok(int M, int d, int h);
bool stream_tile_down_ok(int M, int Nrows, int K);  // single-weight projection alone (MaskedLinear forward)
int stream_tile_rows_per_block(int M, bool dual);
int stream_tile_depth(int M, bool dual);
int stream_tile_direct(int M, bool dual);  // 1: the token-row slab is filled by direct global->LDS loads
int stream_tile_down_splits(int M, int d, int h);
hipError_t launch_stream_tile_up(const StreamArgs& a, hipStream_t stream);
hipError_t launch_stream_tile_down(const StreamArgs& a, hipStream_t stream);
// out[token row of p, n] = bf16(sum_s P[s][p][n])
hipError_t launch_stream_reduce(const float* P, int splits, int M, int N, const uint8_t* mask, uint16_t* out,
                                int64_t ldo, hipStream_t stream);

// ---- generic.hip: any-stride scalar kernels ----
struct GenericLinearArgs {
  const uint16_t* x; int64_t sxm, sxk;
  const uint16_t* W[2]; int64_t swk, swn;  // [visual, text]
  const uint8_t* mask;
  uint16_t* y; int64_t sym, syn;
  int M, K, N;
};
hipError_t launch_generic_linear(const GenericLinearArgs& a, hipStream_t stream);
struct GenericUpArgs {
  const uint16_t* x; int64_t sxm;
  const uint16_t* G[2]; const uint16_t* U[2]; int64_t swk, swn;  // gate = W1/U1, up = W3/U3
  const uint8_t* mask;
  uint16_t* H; int64_t ldh;
  int M, K, N;
};
hipError_t launch_generic_up(const GenericUpArgs& a, hipStream_t stream);
struct GenericBwdArgs {
  const uint16_t* g; int64_t sgm;
  const uint16_t* x; int64_t sxm;
  const uint16_t* W[2]; int64_t swk, swn;
  const uint8_t* mask;
  uint16_t* dx; int64_t sdxm;
  uint16_t* dW[2]; int64_t sdk, sdn;
  int M, K, N;
};
hipError_t launch_generic_bwd(const GenericBwdArgs& a, hipStream_t stream);

}  // namespace ffnk
