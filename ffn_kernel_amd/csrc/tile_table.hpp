// gfx950 tile table: which kernel family and macro tile each (op, M, K, N) uses.
//
// The reference looks its tile up with find_spec(table, M // 1024) in A100-tuned JSON files
// holding one entry each (ffn_kernel/utils.py:3-5, ffn_kernel/bf16_linear_fwd.json,
// bf16_ffn_fwd.json, bf16_linear_bwd.json).  On MI355X the choice is driven by how many
// workgroups a shape yields against 256 CUs, so the table is keyed on the real extents.
#pragma once
#include "launch.hpp"
#include "common.hpp"

namespace ffnk {

constexpr int kCus = 256;

// Smallest M for which the LDS-tiled path is used by the FFN forward; below it the
// weight-streaming kernels win because the op is bound by reading the weights once.
constexpr int kStreamMaxM = 64;

struct TileChoice {
  int tile;    // TileId
  int splits;  // split-K factor (weight-gradient GEMM only)
};

// Routed GEMM over M rows and n_out output columns.
inline int pick_routed_tile(int64_t M, int64_t n_out, bool dual) {
  auto tiles = [&](int tile) {
    const TileGeom t = tile_geom(tile, dual);
    return cdiv64(M, t.block_m) * cdiv64(n_out, t.block_n_out);
  };
  if (tiles(TILE_256x256_W8) >= 2 * kCus) return TILE_256x256_W8;  // at least two full waves of 256x256 tiles
  if (tiles(TILE_128x128_W4) >= kCus) return TILE_128x128_W4;
  return TILE_SMALL_W4;
}

// Weight-gradient GEMM: two [R, Cc] outputs, contraction over about M / 2 rows each.
inline TileChoice pick_splitk_tile(int64_t M, int64_t R, int64_t Cc) {
  TileChoice c;
  // Large outputs: the 256x256 tile fills the chip on its own, no split needed (and the GEMM then
  // stores bf16 directly, without partials or a reduce pass).
  if (2 * cdiv64(R, 256) * cdiv64(Cc, 256) >= 2 * kCus) {
    c.tile = TILE_256x256_W8;
    c.splits = 1;
    return c;
  }
  c.tile = TILE_128x128_W4;
  const int64_t tiles = 2 * cdiv64(R, 128) * cdiv64(Cc, 128);
  int64_t s = cdiv64(2 * kCus, tiles);            // aim at two workgroups per CU
  const int64_t slabs = cdiv64(cdiv64(M, 2), 64);  // 64-row slabs per group at an even split
  if (s > slabs) s = slabs;
  if (s > 16) s = 16;
  if (s < 1) s = 1;
  c.splits = (int)s;
  return c;
}

// Decode shapes: the streaming kernels need whole 128-element K chunks in both projections.
inline bool stream_shape_ok(int64_t M, int64_t d, int64_t h) {
  return M >= 1 && M <= kStreamMaxM && d >= 128 && h >= 128 && d % 128 == 0 && h % 128 == 0 && d % 16 == 0;
}

// Split-K factor of the streamed down-projection.  A workgroup covers `rows_per_block` weight rows
// x one K range that its `waves` wavefronts share.  Aim at about 16 wavefronts per CU and per
// modality, keep at least four 128-element chunks per wavefront, prefer a split that gives every
// wavefront the same number of chunks.  1 means no cross-workgroup split: the kernel then stores
// the output itself and no reduce pass runs.
inline int stream_down_splits(int64_t d, int64_t h, int rows_per_block, int waves) {
  const int64_t row_blocks = cdiv64(d, rows_per_block);
  const int64_t chunks = h / 128;
  int64_t s = cdiv64((int64_t)16 * kCus, row_blocks * waves);
  if (s > chunks / (4 * waves)) s = chunks / (4 * waves);
  if (s > 16) s = 16;
  if (s < 1) s = 1;
  for (int64_t c = s; c >= 1 && c * 2 > s; --c)
    if (chunks % (c * waves) == 0) return (int)c;
  return (int)s;
}

}  // namespace ffnk
