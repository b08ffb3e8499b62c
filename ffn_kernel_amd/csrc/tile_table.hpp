// gfx950 tile table: which kernel family and macro tile each (op, M, K, N) uses.
//
// The reference looks its tile up with find_spec(table, M // 1024) in A100-tuned JSON files
// holding one entry each (ffn_kernel/utils.py:3-5, ffn_kernel/bf16_linear_fwd.json,
// bf16_ffn_fwd.json, bf16_linear_bwd.json).  On MI355X the choice is driven by how many
// workgroups a shape yields against 256 CUs, so the table is keyed on the real extents.
#pragma once
#include "launch.hpp"
#include "common.hpp"
#include "gemm_sched.hpp"

namespace ffnk {

constexpr int kCus = 256;

// Smallest M for which the LDS-tiled path is used by the FFN forward; below it the
// weight-streaming kernels win because the op is bound by reading the weights once.
constexpr int kStreamMaxM = 64;

struct TileChoice {
  int tile;    // TileId
  int splits;  // split-K factor (weight-gradient GEMM only)
  bool tuned;  // the pair is a measured plan (as timed by the tuner), not the rules' guess
};

// Measured plans.  `python -m ffn_kernel_amd.tune --emit` times every candidate (tile x split-K factor)
// per operation, shape and M bucket on the GPU and writes tile_table_gen.hpp: one entry wherever the best
// candidate beat the rules and the cost model below by a margin.  The pick_* functions consult these
// entries first (exact contraction / output extents, M inside the bucket) and fall back to the rules.
// This is what the reference's find_spec/*.py searches and bf16_*.json tables are to its kernels
// (find_spec/find.py:18-64, ffn_kernel/utils.py:3-5).
enum TunedOp : int {
  TUNED_PLAIN = 0,   // MaskedLinear forward (gathered rows in, scattered rows out; whole-call timing): k = contraction, n = output columns
  TUNED_DUAL = 1,    // SwiGLU GEMM: k = contraction (d), n = output columns (h)
  TUNED_SPLITK = 2,  // weight-gradient GEMM: k = R (rows of the in-place operand), n = Cc
  TUNED_DOWN = 3,    // MaskedFFN down projection (routed-order rows in, scattered out; stage timing): k = contraction (h), n = output columns (d)
  TUNED_NONE = -1,   // a GEMM the tuner does not measure (the backward's dx GEMMs): rules only
};
struct TunedPlan {
  int op;            // TunedOp, -1 ends the table
  int m_lo, m_hi;    // rows M of the call, inclusive
  int k, n;
  int tile, splits;
  int group_m;       // M-tiles per super-group of the tile order (GemmArgs::group_m); 0 = the tile's own
};
}  // namespace ffnk
#include "tile_table_gen.hpp"
namespace ffnk {

inline const TunedPlan* tuned_plan(int op, int64_t M, int64_t k, int64_t n) {
  for (const TunedPlan* p = kTunedPlans; p->op >= 0; ++p)
    if (p->op == op && p->k == k && p->n == n && M >= p->m_lo && M <= p->m_hi) return p;
  return nullptr;
}

// Super-group size of a measured plan for this operation and shape, 0 where there is none (the tile's own then).
inline int tuned_group_m(int op, int64_t M, int64_t k, int64_t n) {
  const TunedPlan* t = tuned_plan(op, M, k, n);
  return t ? t->group_m : 0;
}

// Routed GEMM over M rows and n_out output columns (K: the contraction, 0 = not known to the caller).
// `op`: whose measured plans apply (TUNED_NONE: none; the tuner times each operation with its own gather /
// scatter pattern and its own launches around the GEMM, so one operation's plan says nothing about another's).
inline int pick_routed_tile(int64_t M, int64_t n_out, bool dual, int64_t K = 0, bool use_table = true,
                            int op = TUNED_PLAIN) {
  if (use_table && K > 0 && (dual || op != TUNED_NONE)) {
    if (const TunedPlan* t = tuned_plan(dual ? TUNED_DUAL : op, M, K, n_out))
      if (dual || t->splits == 1) return t->tile;
  }
  auto tiles = [&](int tile) {
    const TileGeom t = tile_geom(tile, dual);
    return cdiv64(M, t.block_m) * cdiv64(n_out, t.block_n_out);
  };
  // At least two full rounds of 256x256 tiles.  The SwiGLU kernel runs them with four wavefronts of
  // 128x128 (a third fewer LDS reads per flop; measured 4 % faster at M = 32768, d = 4096, h = 14336); so do the
  // single-weight kernels over a long contraction (1-2.5 % faster at K = 4096 and 14336, N = 4096, M >= 16384),
  // which otherwise keep eight wavefronts of 128x64 (less exposed when K is short).
  if (tiles(TILE_256x256_W8) >= 2 * kCus) return dual || K >= 4096 ? TILE_256x256_W4 : TILE_256x256_W8;
  if (tiles(TILE_128x128_W4) >= kCus) return TILE_128x128_W4;
  return TILE_SMALL_W4;
}

// Tile and split-K factor of a routed GEMM with a single weight per group and a workspace for
// partial sums (the FFN down projection).  When the output yields fewer tiles than the chip has
// workgroup slots and the contraction is long, each workgroup would stream a long weight panel on
// its own while most CUs idle; cutting K into `splits` ranges of whole 64-element slabs fills the
// chip, at the price of fp32 partials (4 * splits * M * n_out bytes written, then read by the
// reduce pass).  The choice minimises a cost model fitted to a sweep over M = 128 ... 4096 at
// n_out = 4096, K = 14336 (it reproduces the measured best of every M there; the table's previous
// choice was 1.1x to 1.7x slower):
//   time = rounds * (5 us + slabs_per_range * t_slab) + splits * M * n_out * 8 bytes / 4 TB/s
//   rounds = ceil(tiles * splits / slots),  slots = 256 CUs * workgroups per CU by LDS use,
//   t_slab = 1.2 us for the 256x256 tile, 0.8 us for the 128x128 and 128x64 tiles.
// The unsplit 256x256 tile is priced with its split tail (see routed_plan_cost).
// Limited to M <= 4096 (above it the tiles fill the chip, and the reduce pass launches one row per
// blockIdx.y); larger M keeps pick_routed_tile and no split.
struct RoutedPlan {
  int tile;
  int splits;
};

inline double routed_plan_cost(int64_t M, int64_t n_out, int64_t K, int tile, int splits) {
  const TileGeom t = tile_geom(tile, false);
  const int64_t tiles = (cdiv64(M, t.block_m) + 1) * cdiv64(n_out, t.block_n_out);
  const int64_t slots = (int64_t)kCus * (tile == TILE_SMALL_W4 ? 3 : tile == TILE_128x128_W4 ? 2 : 1);
  const double t_slab = (tile == TILE_256x256_W8 || tile == TILE_256x256_W4) ? 1.2 : tile == TILE_128x128_R4 ? 0.4 : 0.8;
  const int64_t slabs = cdiv64(cdiv64(K, 64), splits);
  const double reduce = splits > 1 ? (double)splits * (double)M * (double)n_out * 8.0 / 4.0e6 : 0.0;
  if (tile == TILE_256x256_W8 && splits == 1 && K % 64 == 0 && tiles > slots) {
    // Unsplit 256x256 tiles past one round: the launcher runs the whole rounds, then the remaining tiles
    // cut into K ranges (split tail) - a fraction of a round, a second launch and a small reduce pass.
    const int64_t tail = tiles % slots;
    double c = (double)(tiles / slots) * (5.0 + (double)slabs * t_slab);
    if (tail > 0) c += 15.0 + (double)cdiv64(slabs, tail_split_factor((int)tail, (int)slabs)) * t_slab;
    return c;
  }
  return (double)cdiv64(tiles * splits, slots) * (5.0 + (double)slabs * t_slab) + reduce;
}

// Best split for a given tile: ranges of at least 8 slabs, no empty range.
inline int pick_routed_splits(int64_t M, int64_t n_out, int64_t K, int tile) {
  if (M > 4096 || K % 64 != 0 || tile == TILE_256x256_W4) return 1;
  const int64_t nk = K / 64;
  int best = 1;
  double best_cost = routed_plan_cost(M, n_out, K, tile, 1);
  for (int s = 2; s <= 16 && nk / s >= 8; ++s) {
    if (cdiv64(nk, cdiv64(nk, s)) != s) continue;  // would leave an empty range
    const double c = routed_plan_cost(M, n_out, K, tile, s);
    if (c < best_cost) {
      best_cost = c;
      best = s;
    }
  }
  return best;
}

inline RoutedPlan pick_routed_plan(int64_t M, int64_t n_out, int64_t K, bool use_table = true, int op = TUNED_DOWN) {
  RoutedPlan p;
  if (use_table && op != TUNED_NONE)
    if (const TunedPlan* t = tuned_plan(op, M, K, n_out)) {
      p.tile = t->tile;
      p.splits = (K % 64 == 0 && M < 65536 && n_out % 4 == 0) ? t->splits : 1;
      return p;
    }
  p.tile = pick_routed_tile(M, n_out, false, K, use_table, op);
  p.splits = 1;
  if (M > 4096 || K % 64 != 0) return p;
  double best_cost = 0.0;
  const int cand[3] = {TILE_256x256_W8, TILE_128x128_W4, TILE_SMALL_W4};
  for (int i = 0; i < 3; ++i) {
    const int s = pick_routed_splits(M, n_out, K, cand[i]);
    const double c = routed_plan_cost(M, n_out, K, cand[i], s);
    if (i == 0 || c < best_cost) {
      best_cost = c;
      p.tile = cand[i];
      p.splits = s;
    }
  }
  return p;
}

// Weight-gradient GEMM: two [R, Cc] outputs, contraction over about M / 2 rows each.
inline TileChoice pick_splitk_tile(int64_t M, int64_t R, int64_t Cc, bool use_table = true) {
  TileChoice c;
  c.tuned = false;
  if (use_table)
    if (const TunedPlan* t = tuned_plan(TUNED_SPLITK, M, R, Cc)) {
      c.tile = t->tile;
      c.splits = t->splits;
      c.tuned = true;
      return c;
    }
  // Large outputs: the 256x256 tile fills the chip on its own, no split needed (and the GEMM then
  // stores bf16 directly, without partials or a reduce pass).
  if (2 * cdiv64(R, 256) * cdiv64(Cc, 256) >= 2 * kCus) {
    c.tile = TILE_256x256_W8;
    c.splits = 1;
    return c;
  }
  c.tile = TILE_128x128_W4;
  const int64_t tiles = 2 * cdiv64(R, 128) * cdiv64(Cc, 128);
  int64_t s = cdiv64(2 * kCus, tiles);            // aim at two workgroups per CU ...
  const int64_t slabs = cdiv64(cdiv64(M, 2), 64);  // 64-row slabs per group at an even split
  // ... with at least 16 slabs to each range: below that the partials and the reduce pass cost more than the idle CUs
  // (K = N = 1024, M = 256 ... 1024: one range is 20-30 % faster than the two to four that fill the chip)
  if (s > slabs / 16) s = slabs / 16;
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
