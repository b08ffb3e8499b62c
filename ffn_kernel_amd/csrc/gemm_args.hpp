// Plain argument blocks of the tiled GEMM kernels (shared by host launch code and device code).
#pragma once
#include <stdint.h>

namespace ffnk {

struct GemmArgs {
  const uint16_t* A;     // [*, K] rows, K contiguous
  int64_t lda;
  const uint16_t* B0[2]; // per group (0 = visual, 1 = text): [N, K] rows, K contiguous
  const uint16_t* B1[2]; // SwiGLU kernels only: second weight (the "up" projection), same shape
  int64_t ldb;
  // K-major kernels (weights where the backward finds them): B0[g] is [K, N] rows, N contiguous, row
  // stride ldb.  With k_switch > 0 (a multiple of 64) the contraction continues in B1[g]: row k of the
  // operand is B0[g] row k for k < k_switch and B1[g] row k - k_switch after it (two weights that
  // share the output axis, contracted in one pass).  0: B0 all the way.
  int k_switch = 0;
  uint16_t* C;           // [*, N] rows
  int64_t ldc;
  // SwiGLU kernels only, optional: the two pre-activations, bf16, rows like C (routed order):
  // C_pre[row, n] = A B0^T, C_pre[row, N + n] = A B1^T.  Saved by a training forward so that the
  // backward need not recompute them.  NULL: not stored.
  uint16_t* C_pre = nullptr;
  int64_t ldc_pre = 0;
  const int32_t* perm;   // routed position -> token row
  const int32_t* counts; // counts[0] = visual rows (device memory)
  int M, N, K;           // N = output columns
  // Tile schedule.  The order of macro tiles is computed on a grid of sched_bm x sched_bn output
  // tiles (0 = the kernel's own tile).  tail_mode 0: the launch covers every tile.  1: only the tiles
  // that fill whole rounds of the chip (the first floor(tiles / 256) * 256 of the order).  2: only the
  // remaining tiles, each cut into the kernel's own (smaller) tiles - launched with a smaller tile
  // config, this spreads the last, partial round over all CUs instead of leaving most of them idle.
  // 3: only the remaining tiles, on the kernel's own tile, each cut into K ranges (split tail, see
  // P_tail below).
  int sched_bm = 0, sched_bn = 0, tail_mode = 0;
  // M-tiles per super-group of the tile order (routed_tile_coord); 0 = the tile's own (RoutedGemmCfg::GROUP_M).
  int group_m = 0;
  // Split-K (direct path, tail_mode 0, not the SwiGLU kernels): with splits > 1 the contraction is
  // cut into `splits` ranges of whole 64-element slabs, each workgroup handles one (tile, range) and
  // stores its fp32 partial sums to P[split][routed row][N]; a reduce pass adds them and scatters
  // the rows.  For outputs too small to fill the chip with tiles over a long contraction.
  int splits = 1;
  float* P = nullptr;
  // Split tail (direct path, single weight per group): the launcher runs the whole rounds of 256 tiles
  // first and then the remaining tiles cut into tail_split_factor() K ranges each, so that the last,
  // partial round takes a fraction of a tile time.  P_tail holds kTailSlots fp32 tiles of the
  // kernel's macro tile; a reduce pass adds the ranges and scatters the rows.  NULL: the remainder
  // runs as smaller tiles over all of K (tail_mode 2).
  float* P_tail = nullptr;
};

// Grouped split-K GEMM used for the weight gradients:
//   P[grp][split][R, Cc] (fp32) = sum over this split's 64-column slabs of  A[R, k] * B[Cc, k]^T
// Group grp contracts over columns [k_begin(grp), k_begin(grp) + k_len(grp)) of the two row-major
// operands; the ranges come from counts[] on the device:
//   group 0 = [0, pad64(counts[0])),  group 1 = [pad64(counts[0]), + pad64(M - counts[0])).
// K-major kernels: A is instead the untransposed operand, [M + 64, R] rows in routed order (row stride
// lda, 16-byte aligned rows, R % 8 == 0); group grp contracts over its rows [counts[0] * grp, ...) in
// slabs of 64.  The rows of a group's last slab that lie past the group's end (the next group's rows, or
// the 64 rows of padding the buffer must hold past row M) are loaded and then cleared in LDS: their
// contents never count.
struct SplitKArgs {
  const uint16_t* A; int64_t lda;  // [R, Kpad]
  const uint16_t* B; int64_t ldb;  // [Cc, Kpad]
  float* P;                        // [2][splits][R][Cc]
  const int32_t* counts;
  int M;                           // routed rows in total (both groups)
  int R, Cc, splits;
  // splits == 1 only: store bf16 results straight to out[grp][r * out_sr + c * out_sc] instead of
  // fp32 partials (no reduce pass).  NULL: partials go to P.
  uint16_t* out[2] = {nullptr, nullptr};
  int64_t out_sr = 0, out_sc = 0;
};

// Weight-gradient GEMM of the MaskedLinear backward on the untransposed operands (gemm_dw_gather.hpp):
//   dW_g[r, c] = sum over the rows m of group g of G[m, r] * X[m, c],   rows found through perm.
// R % 8 == 0, Cc % 8 == 0, R, Cc >= 8, 16-byte aligned rows, and M * ld * 2 + 2 * cols < 2^32 for both operands.
struct GatherDwArgs {
  const uint16_t* G; int64_t ldg;   // [M, R] rows in token order (the upstream gradient)
  const uint16_t* X; int64_t ldx;   // [M, Cc] rows in token order (the layer's input)
  const int32_t* perm;              // routed position -> token row
  const int32_t* counts;
  SplitKArgs s;                     // R, Cc, splits, M, P / out as for the grouped split-K GEMM (A, B, lda, ldb unused)
};

}  // namespace ffnk
