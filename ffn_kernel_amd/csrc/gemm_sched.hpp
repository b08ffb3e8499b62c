// Tile order of the routed GEMMs, shared by the GEMM kernel and the reduce pass of its split tail.
#pragma once
#include "common.hpp"

namespace ffnk {

constexpr int kCusPerChip = 256;
constexpr int kTailSlots = 256;      // (tile, K range) pairs of a split tail never exceed one per CU
constexpr int kTailMaxSplits = 16;

struct TileCoord {
  int grp;      // 0 = visual, 1 = text
  int row0;     // first routed position of the tile
  int row_end;  // end of the tile's group
  int n0;       // first output column
};

// Tiles are bm rows x bn output columns; M-tiles never straddle the two groups.
__host__ __device__ inline int routed_tile_count(int n_vis, int M, int N, int bm, int bn) {
  return (cdiv(n_vis, bm) + cdiv(M - n_vis, bm)) * cdiv(N, bn);
}

// Position L of the order -> tile.  The order walks super-groups of group_m M-tiles column by
// column, so that tiles sharing A rows / B columns are neighbours.
__host__ __device__ inline TileCoord routed_tile_coord(int L, int n_vis, int M, int N, int bm, int bn, int group_m) {
  const int tiles_v = cdiv(n_vis, bm);
  const int tiles_m = tiles_v + cdiv(M - n_vis, bm);
  const int tiles_n = cdiv(N, bn);
  // Up to two groups' worth of M-tiles form a single super-group: a short last group of one or two
  // M-tiles would stream its weights again with nobody to share them with.
  if (tiles_m <= 2 * group_m) group_m = tiles_m;
  const int width = group_m * tiles_n;
  const int first_m = (L / width) * group_m;
  const int gsz = group_m < tiles_m - first_m ? group_m : tiles_m - first_m;
  const int tile_m = first_m + (L % width) % gsz;
  const int tile_n = (L % width) / gsz;
  TileCoord t;
  t.grp = tile_m < tiles_v ? 0 : 1;
  t.row0 = t.grp == 0 ? tile_m * bm : n_vis + (tile_m - tiles_v) * bm;
  t.row_end = t.grp == 0 ? n_vis : M;
  t.n0 = tile_n * bn;
  return t;
}

// Split tail: the tiles past the last whole round of kCusPerChip are each cut into this many K
// ranges, so that the (tile, range) pairs fill about one round; ranges keep at least 8 slabs.
__host__ __device__ inline int tail_split_factor(int n_tail, int slabs) {
  if (n_tail <= 0) return 1;
  int s = kTailSlots / n_tail;
  if (s > kTailMaxSplits) s = kTailMaxSplits;
  if (s > slabs / 8) s = slabs / 8;
  if (s < 1) s = 1;
  return cdiv(slabs, cdiv(slabs, s));  // no empty range
}

}  // namespace ffnk
