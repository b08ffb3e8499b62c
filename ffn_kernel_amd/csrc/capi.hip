// C ABI of libffnk (declared in include/ffnk.h): argument checks, workspace carving, path
// selection and kernel sequencing.  Nothing here allocates, frees or synchronises.
#include "../../include/ffnk.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>

#include "common.hpp"
#include "launch.hpp"
#include "tile_table.hpp"
#include "gemm_sched.hpp"

using namespace ffnk;

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
  return (int)e;
}

#define FFNK_HIP(expr, what)                       \
  do {                                             \
    hipError_t e__ = (expr);                       \
    if (e__ != hipSuccess) return hip_fail(e__, what); \
  } while (0)

// Row limit.  The row partition runs in one launch of at most 256 blocks (route.hip), each of which
// counts the whole mask once: 256 * M bytes of L2 / HBM reads, 4 GB and about a millisecond at 2^24 rows -
// linear in M, and small against any GEMM over that many rows.  The tile counts and workspace offsets
// derived from M stay inside 32-bit grids up to here for every N the column limit admits.
constexpr int64_t kMaxRows = (int64_t)1 << 24;
constexpr int64_t kMaxCols = (int64_t)1 << 24;

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
bool aligned2(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 1) == 0; }

int check_extents(int64_t M, int64_t K, int64_t N) {
  if (M < 0 || K < 0 || N < 0) return fail(FFNK_E_SHAPE, "negative extent M=%lld K=%lld N=%lld", (long long)M, (long long)K, (long long)N);
  if (M > kMaxRows) return fail(FFNK_E_SHAPE, "M=%lld exceeds %lld rows", (long long)M, (long long)kMaxRows);
  if (K > kMaxCols || N > kMaxCols) return fail(FFNK_E_SHAPE, "K=%lld or N=%lld exceeds %lld", (long long)K, (long long)N, (long long)kMaxCols);
  return FFNK_OK;
}

// Workspace regions.
struct RouteWs {
  int32_t* perm;
  int32_t* counts;
  size_t bytes;
};
size_t route_ws_bytes(int64_t M) { return ws_align((size_t)M * 4) + ws_align(8); }
RouteWs carve_route(uint8_t* ws, int64_t M) {
  RouteWs r;
  r.perm = reinterpret_cast<int32_t*>(ws);
  r.counts = reinterpret_cast<int32_t*>(ws + ws_align((size_t)M * 4));
  r.bytes = route_ws_bytes(M);
  return r;
}

// Tuner overrides, see ffnk_debug_force_tile / ffnk_debug_force_splits.
std::atomic<int> g_force_tile{-1};    // 0..3: that tile; -1: table, then rules; -2: rules only
std::atomic<int> g_force_splits{-1};  // >= 1: that split-K factor where a GEMM can be split
std::atomic<int> g_force_group_m{0};      // >= 1: M-tiles per super-group in the tile order of every routed GEMM
std::atomic<int> g_force_bwd_gather{-1};  // MaskedLinear backward: 1 = weight gradients from g and x in place, 0 = from transposes, -1 = plan

int forced_tile() {
  const int t = g_force_tile.load(std::memory_order_relaxed);
  return (t >= 0 && t < TILE_COUNT) ? t : -1;
}
bool use_tuned() { return g_force_tile.load(std::memory_order_relaxed) != -2; }
// GemmArgs::group_m of a routed GEMM: the forced value, else the measured plan's, else 0 (the tile's own).
int plan_group_m(int op, int64_t M, int64_t k, int64_t n) {
  if (const int f = g_force_group_m.load(std::memory_order_relaxed); f > 0) return f;
  return use_tuned() && op != TUNED_NONE ? tuned_group_m(op, M, k, n) : 0;
}
int forced_splits() {
  const int s = g_force_splits.load(std::memory_order_relaxed);
  return (s >= 1 && s <= 16) ? s : -1;
}

int64_t padded_rows(int64_t M) { return round_up64(M, 64) + 64; }  // >= pad64(nv) + pad64(M - nv)

// The row partition a call works with: the caller's (ffnk_routing_t, made by ffnk_route for the same mask
// and M) or, without one, the workspace's own region, filled by a route launch at the head of the call.
struct Routing {
  const int32_t* perm;
  const int32_t* counts;
};
int resolve_routing(const ffnk_routing_t* rt, const RouteWs& r, const uint8_t* mask, int64_t M, hipStream_t stream,
                    Routing* out) {
  if (rt != nullptr) {
    if (!rt->perm || !rt->counts) return fail(FFNK_E_NULL, "routing: perm or counts is NULL");
    out->perm = rt->perm;
    out->counts = rt->counts;
    return FFNK_OK;
  }
  FFNK_HIP(launch_route(mask, (int)M, r.perm, r.counts, stream), "route kernel");
  out->perm = r.perm;
  out->counts = r.counts;
  return FFNK_OK;
}

// Pseudo tile id of a measured weight-gradient plan: g and x read where they lie (gemm_dw_gather.hpp) on the 128x128 tile.
constexpr int kTileGatherDw = 5;

struct BwdPlan {
  bool dw_k_contig;  // dW memory is [N, K] (k contiguous): R = N, Cc = K
  int64_t R, Cc;
  TileChoice tc;
  bool gather;       // weight gradients from g and x in place, where the call's operands allow it (gather_dw_ok)
  int64_t ldt;       // row stride of the transposed operands
  size_t off_wt, off_gt, off_xt, off_p, total;
};
BwdPlan plan_bwd(int64_t M, int64_t K, int64_t N, bool dw_k_contig) {
  BwdPlan p;
  p.dw_k_contig = dw_k_contig;
  p.R = dw_k_contig ? N : K;
  p.Cc = dw_k_contig ? K : N;
  p.tc = pick_splitk_tile(M, p.R, p.Cc, use_tuned());
  // A measured plan names the form (5: in place; 0 / 2 / 4: from transposes).  Where nothing was measured: the in-place
  // form saves a launch and the transposes' 4 * M * (K + N) bytes of traffic, and its two-stage loop runs the GEMM's
  // M * K * N products about 15 % slower than the tiles that read transposes; on this part the two balance near
  // K * N / (K + N) = 1600 (K = N: faster by 19 % at 1024, 15 % at 2048, slower by 9 % at 4096).
  // Up to 1024 rows the transposes are a launch that moves next to nothing, and the in-place form wins at every size
  // (by 4-8 % at K = N = 4096, 8-33 % at 8192).
  p.gather = p.tc.tuned ? p.tc.tile == kTileGatherDw : (K * N <= 1536 * (K + N) || M <= 1024);
  if (p.tc.tile == kTileGatherDw) p.tc.tile = TILE_128x128_W4;
  if (forced_tile() >= 0) {
    p.tc.tile = forced_tile();
    p.gather = false;
  }
  if (const int fg = g_force_bwd_gather.load(std::memory_order_relaxed); fg >= 0) p.gather = fg == 1;
  if (forced_splits() >= 1) p.tc.splits = forced_splits();
  p.ldt = padded_rows(M);
  size_t o = route_ws_bytes(M);
  p.off_wt = o; o += 2 * ws_align((size_t)K * N * 2);
  p.off_gt = o; o += ws_align((size_t)N * p.ldt * 2);
  p.off_xt = o; o += ws_align((size_t)K * p.ldt * 2);
  p.off_p = o;  o += ws_align((size_t)2 * p.tc.splits * K * N * 4);
  p.total = o;
  return p;
}

// T13 and DH end in 64 rows of padding: the weight-gradient GEMMs load them in whole 64-row slabs (and
// clear what lies past a group's end before using it).
constexpr int kBwdPadRows = 64;

// MaskedFFN backward workspace: route | T13 [M + 64, 2h] | DH [M + 64, h] | W2^T, U2^T [h, d] | [W1^T|W3^T],
// [U1^T|U3^T] [d, 2h] | g^T, x^T [d, ldt] | H^T, dt1^T, dt3^T [h, ldt] | fp32 split-K partials.
struct FfnBwdPlan {
  BwdPlan up, dn;  // weight-gradient GEMM shapes: up = dW1/dW3 (K = d, N = h), dn = dW2 (K = h, N = d)
  int64_t ldt;
  size_t w2t_bytes;  // room at off_w2t: the W2^T / U2^T copies, or the dx GEMM's partials / split tail after them
  size_t off_t13, off_dh, off_w2t, off_w13t, off_gt, off_xt, off_ht, off_d1t, off_d3t, off_p, total;
};
// Which of the optional regions a call touches (decided from strides and alignment, the same way by the
// planner and by the backward itself): copies of the down / up weights for layouts the K-major kernels do not
// read in place, and transposes of H, dt1, dt3 when their rows do not fit 32-bit slab offsets.
struct FfnBwdPaths {
  bool w2_copy = true, w13_copy = true, acts_in_place = false, dx_direct = false;
};
constexpr FfnBwdPaths kFfnBwdWorstCase{};
// Weight-gradient split of the in-place path (H, dt1, dt3 read where they lie).
TileChoice ffn_bwd_in_place_choice(int64_t M, int64_t d, int64_t h) {
  TileChoice tc = pick_splitk_tile(M, h, d, use_tuned());
  if (tc.tile == kTileGatherDw) tc.tile = TILE_128x128_W4;  // a MaskedLinear plan of the same extents: the form does not exist here
  if (forced_splits() >= 1) tc.splits = forced_splits();
  return tc;
}
// Tile and split of the dx GEMM (2h-long contraction) and the bytes of partials or split tail it wants.
RoutedPlan ffn_bwd_dx_plan(int64_t M, int64_t d, int64_t h, bool dx_direct, size_t room, size_t* need);
FfnBwdPlan plan_ffn_bwd(int64_t M, int64_t d, int64_t h, bool dup_k_contig, bool ddn_k_contig,
                        const FfnBwdPaths& paths = kFfnBwdWorstCase) {
  FfnBwdPlan p;
  p.up = plan_bwd(M, d, h, dup_k_contig);
  p.dn = plan_bwd(M, h, d, ddn_k_contig);
  p.ldt = padded_rows(M);
  int splits = p.up.tc.splits > p.dn.tc.splits ? p.up.tc.splits : p.dn.tc.splits;
  if (paths.acts_in_place) splits = ffn_bwd_in_place_choice(M, d, h).splits;
  const size_t w2_copies = 2 * ws_align((size_t)h * d * 2);
  // The dx GEMM's partials (or split tail) live where the copies would, as far as they fit there - the same bound
  // whether or not the copies are made, so that the dx GEMM's plan does not depend on the layout.
  size_t dx_need = 0;
  ffn_bwd_dx_plan(M, d, h, paths.dx_direct, w2_copies, &dx_need);
  p.w2t_bytes = paths.w2_copy ? w2_copies : ws_align(dx_need);
  size_t o = route_ws_bytes(M);
  p.off_t13 = o;  o += ws_align((size_t)(M + kBwdPadRows) * 2 * h * 2);
  p.off_dh = o;   o += ws_align((size_t)(M + kBwdPadRows) * h * 2);
  p.off_w2t = o;  o += p.w2t_bytes;
  p.off_w13t = o; o += paths.w13_copy ? 2 * ws_align((size_t)d * 2 * h * 2) : 0;
  p.off_gt = o;   o += ws_align((size_t)d * p.ldt * 2);
  p.off_xt = o;   o += ws_align((size_t)d * p.ldt * 2);
  p.off_ht = o;   o += paths.acts_in_place ? 0 : ws_align((size_t)h * p.ldt * 2);
  p.off_d1t = o;  o += paths.acts_in_place ? 0 : ws_align((size_t)h * p.ldt * 2);
  p.off_d3t = o;  o += paths.acts_in_place ? 0 : ws_align((size_t)h * p.ldt * 2);
  p.off_p = o;    o += (paths.acts_in_place && splits == 1) ? 0 : ws_align((size_t)2 * splits * d * h * 4);
  p.total = o;
  return p;
}

// The direct global->LDS path addresses operands with 32-bit byte offsets: from the start of A
// when its rows are gathered, from the tile's first row otherwise (at most 256 rows away).
bool direct_ok(int64_t K, int64_t gathered_rows, int64_t lda, int64_t ldb) {
  constexpr int64_t k4g = (int64_t)1 << 32;
  if (K <= 0 || K % 64 != 0) return false;
  if (gathered_rows > 0 && gathered_rows * lda * 2 >= k4g) return false;
  return 256 * lda * 2 < k4g && 256 * ldb * 2 < k4g;
}

// The K-major kernels read a weight where the backward finds it: [K, N] rows of the contraction, N
// contiguous, row stride ldb.  Slabs are addressed with 32-bit byte offsets from their first row.
bool kmajor_ok(int64_t K, int64_t N, int64_t ldb, const void* w0, const void* w1) {
  constexpr int64_t k4g = (int64_t)1 << 32;
  return K > 0 && K % 64 == 0 && N >= 8 && N % 8 == 0 && ldb % 8 == 0 && ldb >= N && aligned16(w0) && aligned16(w1) &&
         ldb * 128 + 2 * N < k4g;
}

// Scratch of ffnk_masked_ffn_fwd_static: one copy per GPU, held from the moment the library's code
// object is loaded there until the process ends.  The name is a host-side stand-in, not a device
// address: host code only ever uses the per-device address that static_scratch() looks up.
static __device__ __align__(256) unsigned char scratch[FFNK_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Address of `scratch` on the GPU that holds `on_device` (the call's output): each GPU has its own copy
// of the array at its own address, and the kernels run where their operands live, which need not be the
// calling thread's current device.  Looked up once per device, with that device current (two threads that
// race here both get the same answer).
int static_scratch(const void* on_device, void** out) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, on_device) != hipSuccess || attr.type != hipMemoryTypeDevice) {
    (void)hipGetLastError();  // the query's own error must not surface in a later call
    return fail(FFNK_E_NULL, "ffnk_masked_ffn_fwd_static: out is not device memory");
  }
  const int dev = attr.device;
  if (dev < 0 || dev >= kMaxDevices) return fail(FFNK_E_SHAPE, "device index %d outside [0, %d)", dev, kMaxDevices);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    int cur = -1;
    FFNK_HIP(hipGetDevice(&cur), "hipGetDevice");
    if (cur != dev) FFNK_HIP(hipSetDevice(dev), "hipSetDevice");
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (cur != dev) FFNK_HIP(hipSetDevice(cur), "hipSetDevice");
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (p == nullptr) return fail(FFNK_E_NULL, "static scratch has no address on device %d", dev);
    g_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return FFNK_OK;
}

int routed_tile(int64_t M, int64_t n_out, bool dual, int64_t K = 0, int op = TUNED_PLAIN) {
  const int f = forced_tile();
  return f >= 0 ? f : pick_routed_tile(M, n_out, dual, K, use_tuned(), op);
}

bool use_stream_path(int64_t M, int64_t d, int64_t h) { return stream_shape_ok(M, d, h); }

// M <= 8: both projections run as contiguous-row dot-product streams.
bool use_dot_path(int64_t M, int64_t d, int64_t h) {
  return use_stream_path(M, d, h) && stream_dot_ok((int)M, (int)d) && stream_dot_ok((int)M, (int)h);
}

// 9 <= M <= 64 (or smaller M whose extents the dot kernels do not take): LDS-transposed MFMA streams.
bool use_tile_path(int64_t M, int64_t d, int64_t h) {
  return use_stream_path(M, d, h) && !use_dot_path(M, d, h) && stream_tile_ok((int)M, (int)d, (int)h);
}

int down_splits(int64_t M, int64_t d, int64_t h) {
  if (use_dot_path(M, d, h)) return 1;
  if (use_tile_path(M, d, h)) {
    // a forced factor (tuner) where every K range keeps the kernel's minimum of eight 128-element chunks
    const int fs = forced_splits(), chunks = (int)(h / 128);
    if (fs >= 1 && chunks - (int)cdiv64(chunks, fs) * (fs - 1) >= 8) return fs;
    return stream_tile_down_splits((int)M, (int)d, (int)h);
  }
  return stream_down_splits(d, h, stream_rows_per_block((int)M, false), stream_waves_per_block((int)M, false));
}

// Split-K factor of the down projection on the LDS-tiled path (1: none).
// Tile and split-K factor of the down projection on the LDS-tiled path (a forced tile keeps its own
// best split).
// `op`: whose measured plans apply (TunedOp).
RoutedPlan down_plan(int64_t M, int64_t d, int64_t h, int op = TUNED_DOWN) {
  RoutedPlan p;
  if (const int f = forced_tile(); f >= 0) {
    p.tile = f;
    p.splits = pick_routed_splits(M, d, h, p.tile);
  } else {
    p = pick_routed_plan(M, d, h, use_tuned(), op);
  }
  // a forced split-K factor: whole 64-element slabs, no empty range, what the reduce pass can address
  if (const int fs = forced_splits(); fs >= 1 && h % 64 == 0 && M < 65536 && cdiv64(h / 64, cdiv64(h / 64, fs)) == fs &&
      p.tile != TILE_256x256_W4)
    p.splits = fs;
  return p;
}
// dx GEMM of the MaskedFFN backward: few output tiles over a 2h-long contraction, so K is split like the forward's
// down projection when the fp32 partials fit `room`; an unsplit big tile wants room for its split tail instead.
RoutedPlan ffn_bwd_dx_plan(int64_t M, int64_t d, int64_t h, bool dx_direct, size_t room, size_t* need) {
  // Rules and cost model only: the measured plans are timings of other kernels (the forward's down
  // projection reads K-contiguous weights through another loop).
  RoutedPlan dxp = down_plan(M, d, 2 * h, TUNED_NONE);
  if (!dx_direct || (size_t)dxp.splits * M * d * 4 > room) {
    dxp.splits = 1;
    dxp.tile = routed_tile(M, d, false, 0, TUNED_NONE);
  }
  size_t n = 0;
  if (dxp.splits > 1) n = (size_t)dxp.splits * M * d * 4;
  else if (dx_direct && is_big_tile(dxp.tile) && (size_t)kTailSlots * 256 * 256 * 4 <= room) n = (size_t)kTailSlots * 256 * 256 * 4;
  if (need) *need = n;
  return dxp;
}
// Paths of the MaskedFFN backward for one layout: which weights are read in place and which copied, and whether
// H, dt1, dt3 are read in place by the weight-gradient GEMMs.  The backward and the lean workspace query both ask
// here, so that the regions a call touches are the regions its plan holds.
FfnBwdPaths ffn_bwd_paths(int64_t M, int64_t d, int64_t h, int64_t g_stride_m, int64_t up_stride_n, int64_t down_stride_k,
                          int64_t down_stride_n, const uint16_t* W1, const uint16_t* W3, const uint16_t* U1,
                          const uint16_t* U3, const uint16_t* W2, const uint16_t* U2, bool* w2_direct_out = nullptr,
                          bool* w2_kmajor_out = nullptr, bool* w13_kmajor_out = nullptr) {
  const int64_t ld13 = 2 * h;
  const bool w2_direct = down_stride_n == 1 && down_stride_k % 8 == 0 && down_stride_k >= d && aligned16(W2) && aligned16(U2);
  // The forward's layout ([d, h] rows, h contiguous) is K-major for the dh GEMM: read in place.
  const bool w2_kmajor = !w2_direct && down_stride_k == 1 && kmajor_ok(d, h, down_stride_n, W2, U2) &&
                         direct_ok(d, M, g_stride_m, 8);
  // The up-projection weights ([h, d] rows, d contiguous) are K-major for the dx GEMM: the contraction
  // runs through the gate weight's rows and on into the up weight's.
  const bool w13_kmajor = h % 64 == 0 && kmajor_ok(2 * h, d, up_stride_n, W1, W3) && aligned16(U1) && aligned16(U3) &&
                          direct_ok(2 * h, 0, ld13, 8);
  FfnBwdPaths paths;
  paths.w2_copy = !(w2_direct || w2_kmajor);
  paths.w13_copy = !w13_kmajor;
  paths.acts_in_place = ld13 * 128 + 2 * h < ((int64_t)1 << 32);
  paths.dx_direct = w13_kmajor || direct_ok(2 * h, 0, ld13, ld13);
  if (w2_direct_out) *w2_direct_out = w2_direct;
  if (w2_kmajor_out) *w2_kmajor_out = w2_kmajor;
  if (w13_kmajor_out) *w13_kmajor_out = w13_kmajor;
  return paths;
}

// MaskedLinear forward at decode sizes: 0 = LDS-tiled GEMM, 1 = dot-product streams (M <= 8),
// 2 = LDS-transposed streams (M <= 64).  The op is bound by reading each weight once.
int linear_stream_kind(int64_t M, int64_t K, int64_t N) {
  if (M < 1 || M > kStreamMaxM || K > kMaxCols || N > kMaxCols) return 0;
  if (stream_dot_ok((int)M, (int)K)) return 1;
  if (stream_tile_down_ok((int)M, (int)N, (int)K)) return 2;
  return 0;
}
int linear_stream_splits(int64_t M, int64_t K, int64_t N) {
  return linear_stream_kind(M, K, N) == 2 ? stream_tile_down_splits((int)M, (int)N, (int)K) : 1;
}

// MaskedLinear forward: the table's tile unless cutting K pays (few output tiles, long contraction).
RoutedPlan linear_plan(int64_t M, int64_t K, int64_t N) {
  RoutedPlan p = down_plan(M, N, K, TUNED_PLAIN);
  if (N % 4 != 0) p.splits = 1;  // the reduce pass moves four columns per thread
  if (p.splits == 1) p.tile = routed_tile(M, N, false, K, TUNED_PLAIN);
  return p;
}
// fp32 partials of the tiled MaskedLinear forward: split-K for the whole GEMM, or the split tail of
// the 256x256 tile.
size_t linear_partial_bytes(int64_t M, int64_t K, int64_t N) {
  const RoutedPlan p = linear_plan(M, K, N);
  if (p.splits > 1) return ws_align((size_t)p.splits * M * N * 4);
  if (is_big_tile(p.tile) && K % 64 == 0) return ws_align((size_t)kTailSlots * 256 * 256 * 4);
  return 0;
}
int down_tile(int64_t M, int64_t d, int64_t h) { return down_plan(M, d, h).tile; }
int tiled_down_splits(int64_t M, int64_t d, int64_t h) {
  return use_stream_path(M, d, h) ? 1 : down_plan(M, d, h).splits;
}
// fp32 partials of the tiled down projection: all rows when K is split for the whole GEMM, or the
// kTailSlots tiles of the split tail when the 256x256 tile runs unsplit.
size_t tiled_down_partial_bytes(int64_t M, int64_t d, int64_t h) {
  const RoutedPlan p = down_plan(M, d, h);
  if (p.splits > 1) return ws_align((size_t)p.splits * M * d * 4);
  if (is_big_tile(p.tile) && h % 64 == 0) return ws_align((size_t)kTailSlots * 256 * 256 * 4);
  return 0;
}

// Split-K factor of the weight-gradient GEMM when it shares a launch with the dx GEMM (both on 128x128
// tiles, two workgroups per CU).  The weight-gradient workgroups are few and long, the dx workgroups many
// and short and fill the CUs the others leave: the launch lasts as long as the longer of the two, in
// 64-row slabs of 0.8 us (a 128x128 tile's slab behind two LDS stages waits on its loads: measured).  Unsplit (no
// partials, no reduce pass, one launch fewer) unless cutting the contraction shortens the estimate by more than 35 %
// (K = N = 1024: at M = 8192, estimate 0.75, two or three ranges measure between 7 % slower and 16 % faster than one
// depending on the mask; at M = 16384, estimate 0.63, 17-26 % faster); never more ranges than the plan sized the
// partials for.
int fused_bwd_splits(int64_t M, int64_t K, int64_t N, int plan_splits) {
  const double slots = 2.0 * kCus, t_slab = 0.8;
  const double dw_tiles = 2.0 * (double)cdiv64(N, 128) * (double)cdiv64(K, 128);
  const double dx_units = (double)(cdiv64(M, 128) + 1) * (double)cdiv64(K, 128) * (double)cdiv64(N, 64);
  auto estimate = [&](int s) {
    const double dw_wgs = dw_tiles * s;
    const double dw_slabs = (double)cdiv64(cdiv64(M, 2 * 64), s) * (double)cdiv64((int64_t)dw_wgs, (int64_t)slots);
    const double rest = slots - dw_wgs > slots / 8 ? slots - dw_wgs : slots / 8;
    const double t = (dw_slabs > dx_units / rest ? dw_slabs : dx_units / rest) * t_slab;
    return s == 1 ? t : t + 4.0 + (double)s * 2.0 * (double)K * (double)N * 8.0 / 4.0e6;  // launch + partials at 4 TB/s
  };
  const double unsplit = estimate(1);
  int best = 1;
  double best_t = unsplit;
  for (int s = 2; s <= plan_splits; ++s) {
    const double t = estimate(s);
    if (t < best_t) {
      best = s;
      best_t = t;
    }
  }
  return best_t < 0.65 * unsplit ? best : 1;
}

// Whether the MaskedLinear backward runs its two GEMMs in one launch, and the split-K factor its
// weight-gradient GEMM is really launched with.  A measured plan and a forced factor are used as they are
// (that is what the tuner timed); only a factor the rules guessed goes through the fused launch's own model.
// The fused launch is one decision: it runs when the weights are readable in place and both GEMMs are on a 128x128
// tile; the weight-gradient plan (rules, measured plan or forced tile) says which of the two - two LDS stages, or
// the ring of four - and the dx GEMM follows it.
bool is_128_tile(int tile) { return tile == TILE_128x128_W4 || tile == TILE_128x128_R4; }
// The in-place weight-gradient GEMM addresses token rows with 32-bit byte offsets and moves 8-column chunks.
// (16-byte aligned in memory, so row strides are multiples of 8 as well).
bool gather_dw_ok(int64_t M, int64_t K, int64_t N, const void* g, int64_t g_stride_m, const void* x, int64_t x_stride_m) {
  constexpr int64_t k4g = (int64_t)1 << 32;
  return M > 0 && K >= 8 && N >= 8 && K % 8 == 0 && N % 8 == 0 && g_stride_m % 8 == 0 && x_stride_m % 8 == 0 &&
         M * g_stride_m * 2 + 2 * N < k4g && M * x_stride_m * 2 + 2 * K < k4g &&
         ((reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(x)) & 15) == 0;
}
// One launch for both GEMMs: the dx GEMM on a 128x128 tile over weights read in place, and the weight gradients on the
// same tile (the in-place form has no other).
bool bwd_is_fused(int64_t M, int64_t K, const BwdPlan& p, bool w_kmajor, bool in_place) {
  return w_kmajor && is_128_tile(routed_tile(M, K, false, 0, TUNED_NONE)) && (in_place || is_128_tile(p.tc.tile));
}
int bwd_dw_launch_splits(int64_t M, int64_t K, int64_t N, const BwdPlan& p, bool fused) {
  if (!fused || p.tc.tuned || forced_splits() >= 1) return p.tc.splits;
  return fused_bwd_splits(M, K, N, p.tc.splits);
}

}  // namespace

extern "C" {

int ffnk_version(void) { return FFNK_VERSION; }

int ffnk_debug_force_tile(int tile) {
  return g_force_tile.exchange(((tile >= 0 && tile < TILE_COUNT) || tile == -2) ? tile : -1);
}

int ffnk_debug_force_group_m(int group_m) { return g_force_group_m.exchange(group_m >= 1 && group_m <= 64 ? group_m : 0); }

int ffnk_debug_force_bwd_gather(int on) { return g_force_bwd_gather.exchange((on == 0 || on == 1) ? on : -1); }

int ffnk_debug_force_splits(int splits) { return g_force_splits.exchange((splits >= 1 && splits <= 16) ? splits : -1); }

const char* ffnk_last_error(void) { return g_err; }

int ffnk_route(const uint8_t* mask, int64_t M, int32_t* perm, int32_t* counts, void* stream) {
  if (int e = check_extents(M, 0, 0)) return e;
  if (!counts || (M > 0 && (!mask || !perm))) return fail(FFNK_E_NULL, "ffnk_route: NULL pointer");
  FFNK_HIP(launch_route(mask, (int)M, perm, counts, (hipStream_t)stream), "route kernel");
  return FFNK_OK;
}

size_t ffnk_workspace_bytes(int op, int64_t M, int64_t K, int64_t N) {
  if (M < 0 || K < 0 || N < 0 || M > kMaxRows || K > kMaxCols || N > kMaxCols) return (size_t)-1;
  switch (op) {
    case FFNK_OP_LINEAR_FWD: {
      // perm + counts + the fp32 split-K partials where the GEMM (or the streamed projection) is split
      if (linear_stream_kind(M, K, N)) {
        const int splits = linear_stream_splits(M, K, N);
        return route_ws_bytes(M) + (splits > 1 ? ws_align((size_t)splits * M * N * 4) : 0);
      }
      return route_ws_bytes(M) + linear_partial_bytes(M, K, N);
    }
    case FFNK_OP_FFN_FWD:
      // perm + counts + the [M, h] bf16 intermediate in routed order (N = h) + the fp32 split-K
      // partials of the down projection where it is split.
      return route_ws_bytes(M) + ws_align((size_t)M * round_up64(N, 8) * 2) +
             (use_stream_path(M, K, N) ? ws_align((size_t)down_splits(M, K, N) * M * K * 4) : tiled_down_partial_bytes(M, K, N));
    case FFNK_OP_LINEAR_BWD: {
      const BwdPlan a = plan_bwd(M, K, N, true), b = plan_bwd(M, K, N, false);
      return a.total > b.total ? a.total : b.total;
    }
    case FFNK_OP_FFN_BWD: {
      size_t best = 0;
      for (int i = 0; i < 4; ++i) {
        const size_t t = plan_ffn_bwd(M, K, N, (i & 1) != 0, (i & 2) != 0).total;
        if (t > best) best = t;
      }
      return best;
    }
    default:
      return (size_t)-1;
  }
}

size_t ffnk_workspace_bytes_ffn_bwd(int64_t M, int64_t d, int64_t h, int64_t g_stride_m, int64_t up_stride_n,
                                    int64_t down_stride_k, int64_t down_stride_n, int64_t dup_stride_k,
                                    int64_t ddown_stride_k) {
  if (M < 0 || d <= 0 || h <= 0 || M > kMaxRows || d > kMaxCols || h > kMaxCols) return (size_t)-1;
  const FfnBwdPaths paths = ffn_bwd_paths(M, d, h, g_stride_m, up_stride_n, down_stride_k, down_stride_n, nullptr, nullptr,
                                          nullptr, nullptr, nullptr, nullptr);
  return plan_ffn_bwd(M, d, h, dup_stride_k == 1, ddown_stride_k == 1, paths).total;
}

int ffnk_tile_config(int op, int64_t M, int64_t K, int64_t N, ffnk_tile_config_t* out) {
  if (!out) return fail(FFNK_E_NULL, "ffnk_tile_config: out is NULL");
  if (int e = check_extents(M, K, N)) return e;
  memset(out, 0, sizeof(*out));
  int tile;
  bool dual = false;
  int64_t contraction;
  int splits = 1;
  bool in_place = false;
  switch (op) {
    case FFNK_OP_LINEAR_FWD: { const RoutedPlan lp = linear_plan(M, K, N); tile = lp.tile; splits = lp.splits; contraction = K; break; }
    case FFNK_OP_FFN_FWD:
    case FFNK_OP_FFN_UP: tile = routed_tile(M, N, true, K); dual = true; contraction = K; break;
    case FFNK_OP_FFN_DOWN: tile = down_plan(M, K, N).tile; contraction = N; break;  // out cols = d = K, contraction h = N
    case FFNK_OP_LINEAR_BWD:
    case FFNK_OP_BWD_DX: tile = routed_tile(M, K, false, 0, TUNED_NONE); contraction = N; break;
    case FFNK_OP_BWD_DW: {
      // As launched for the reference's layout (nn.Linear.weight.T views, contiguous g): weights read in place.
      const BwdPlan bp = plan_bwd(M, K, N, true);
      const bool w_kmajor = N > 0 && N % 64 == 0 && K >= 8 && K % 8 == 0 && direct_ok(N, M, N, 8);
      in_place = bp.gather && gather_dw_ok(M, K, N, nullptr, N, nullptr, K);
      tile = in_place ? TILE_128x128_W4 : bp.tc.tile; contraction = M;
      splits = bwd_dw_launch_splits(M, K, N, bp, bwd_is_fused(M, K, bp, w_kmajor, in_place));
      break;
    }
    default: return fail(FFNK_E_OP, "unknown op %d", op);
  }
  const bool direct = contraction > 0 && contraction % 64 == 0;
  if (!direct && tile == TILE_256x256_W4) tile = TILE_256x256_W8;  // the four-wave tile runs on the direct path only
  const TileGeom gm = tile_geom(tile, dual);
  const bool stream = (op == FFNK_OP_FFN_FWD || op == FFNK_OP_FFN_UP || op == FFNK_OP_FFN_DOWN) && use_stream_path(M, K, N);
  out->path = stream ? FFNK_PATH_STREAM : FFNK_PATH_MFMA_TILED;
  out->block_m = gm.block_m;
  out->block_n = gm.block_n_out;
  out->block_k = 64;
  out->waves_m = gm.waves_m;
  out->waves_n = gm.waves_n;
  // the plan's super-group size, else the tile's own: 8 for the SwiGLU GEMM and over K-major weights (the backward's
  // dx GEMM in the usual layout), 4 for the other single-weight GEMMs
  int plan_gm = 0;
  switch (op) {
    case FFNK_OP_LINEAR_FWD: plan_gm = plan_group_m(TUNED_PLAIN, M, K, N); break;
    case FFNK_OP_FFN_FWD:
    case FFNK_OP_FFN_UP: plan_gm = plan_group_m(TUNED_DUAL, M, K, N); break;
    case FFNK_OP_FFN_DOWN: plan_gm = plan_group_m(TUNED_DOWN, M, N, K); break;
    default: plan_gm = plan_group_m(TUNED_NONE, M, K, N); break;
  }
  const bool kmajor_dx = op == FFNK_OP_LINEAR_BWD || op == FFNK_OP_BWD_DX;
  out->group_m = plan_gm > 0 ? plan_gm : (dual || kmajor_dx) ? 8 : 4;
  out->split_k = splits;
  out->direct_lds = (direct || in_place) ? 1 : 0;
  out->in_place = in_place ? 1 : 0;
  // 4: ring of four stages (128x128); 3: token panel in three stages, weight panel in two (single-weight 256x256 tiles)
  out->lds_stages = !out->direct_lds ? 2 : tile == TILE_128x128_R4 ? 4 : (is_big_tile(tile) && !dual) ? 3 : 2;
  if (op == FFNK_OP_FFN_DOWN && !stream) out->split_k = tiled_down_splits(M, K, N);
  if (op == FFNK_OP_LINEAR_FWD && linear_stream_kind(M, K, N)) {
    out->path = FFNK_PATH_STREAM;
    out->waves_m = out->waves_n = 1;
    out->group_m = 1;
    if (linear_stream_kind(M, K, N) == 1) {
      out->block_m = (int)M;
      out->block_n = stream_dot_rows_per_block((int)N, false, (int)K);
      out->block_k = 512 * stream_dot_slices_per_wave((int)K);
      out->split_k = (int)(K / out->block_k);
      out->lds_stages = 0;
      out->direct_lds = 0;
    } else {
      out->block_m = 16 * (int)cdiv64(M, 16);
      out->block_n = stream_tile_rows_per_block((int)M, false);
      out->block_k = 128;
      out->lds_stages = stream_tile_depth((int)M, false);
      out->direct_lds = stream_tile_direct((int)M, false);
      out->split_k = linear_stream_splits(M, K, N);
    }
    return FFNK_OK;
  }
  if (stream) {
    // Streaming kernels: a workgroup is 16 * RT weight rows x one K range whose four wavefronts
    // take a quarter each; operands go global -> registers, no LDS staging.
    const bool up = op != FFNK_OP_FFN_DOWN;
    out->block_m = 16 * (int)cdiv64(M, 16);
    out->block_n = stream_rows_per_block((int)M, up);
    out->block_k = stream_chunk_k((int)M, up);
    out->waves_m = 1;
    out->waves_n = 1;
    out->lds_stages = 0;
    out->group_m = 1;
    out->split_k = stream_waves_per_block((int)M, up) * (up ? 1 : down_splits(M, K, N));
    out->direct_lds = 0;
    if (use_tile_path(M, K, N)) {
      // LDS-transposed streams: block_n weight rows (of each matrix) x 128-element chunks, three in flight
      out->block_n = stream_tile_rows_per_block((int)M, up);
      out->block_k = 128;
      out->lds_stages = stream_tile_depth((int)M, up);
      out->direct_lds = stream_tile_direct((int)M, up);
      out->split_k = up ? 1 : down_splits(M, K, N);
    }
    if (use_dot_path(M, K, N)) {
      // dot-product streams: a workgroup is block_n weight rows x all of K, one wavefront per
      // block_k-element slice of K
      const int64_t contr = up ? K : N;
      out->block_m = (int)M;
      out->block_n = stream_dot_rows_per_block((int)(up ? N : K), up, (int)contr);
      out->block_k = 512 * stream_dot_slices_per_wave((int)contr);
      out->split_k = (int)(contr / out->block_k);
    }
  }
  return FFNK_OK;
}

int ffnk_masked_linear_fwd(const uint16_t* x, int64_t x_stride_m, const uint16_t* Wv, const uint16_t* Wt,
                           int64_t w_stride_k, int64_t w_stride_n, const uint8_t* mask, uint16_t* y,
                           int64_t y_stride_m, int64_t M, int64_t K, int64_t N, void* ws, size_t ws_bytes,
                           void* stream_) {
  return ffnk_masked_linear_fwd_routed(x, x_stride_m, Wv, Wt, w_stride_k, w_stride_n, mask, y, y_stride_m, M, K, N, ws,
                                       ws_bytes, stream_, nullptr);
}

int ffnk_masked_linear_fwd_routed(const uint16_t* x, int64_t x_stride_m, const uint16_t* Wv, const uint16_t* Wt,
                                  int64_t w_stride_k, int64_t w_stride_n, const uint8_t* mask, uint16_t* y,
                                  int64_t y_stride_m, int64_t M, int64_t K, int64_t N, void* ws, size_t ws_bytes,
                                  void* stream_, const ffnk_routing_t* routing) {
  hipStream_t stream = (hipStream_t)stream_;
  if (int e = check_extents(M, K, N)) return e;
  if (M == 0 || N == 0) return FFNK_OK;
  if (!x && K > 0) return fail(FFNK_E_NULL, "x is NULL");
  if ((!Wv || !Wt) && K > 0) return fail(FFNK_E_NULL, "weight pointer is NULL");
  if (!mask || !y) return fail(FFNK_E_NULL, "mask or y is NULL");
  if (!aligned2(x) || !aligned2(Wv) || !aligned2(Wt) || !aligned2(y)) return fail(FFNK_E_ALIGN, "bf16 pointer not 2-byte aligned");
  if (y_stride_m < N) return fail(FFNK_E_STRIDE, "y_stride_m=%lld < N=%lld", (long long)y_stride_m, (long long)N);

  const bool fast = K > 0 && K % 8 == 0 && x_stride_m % 8 == 0 && x_stride_m >= K && aligned16(x) &&
                    w_stride_k == 1 && w_stride_n % 8 == 0 && w_stride_n >= K && aligned16(Wv) && aligned16(Wt);
  if (!fast) {
    GenericLinearArgs a;
    a.x = x; a.sxm = x_stride_m; a.sxk = 1;
    a.W[0] = Wv; a.W[1] = Wt; a.swk = w_stride_k; a.swn = w_stride_n;
    a.mask = mask; a.y = y; a.sym = y_stride_m; a.syn = 1;
    a.M = (int)M; a.K = (int)K; a.N = (int)N;
    FFNK_HIP(launch_generic_linear(a, stream), "generic linear kernel");
    return FFNK_OK;
  }
  const size_t need = ffnk_workspace_bytes(FFNK_OP_LINEAR_FWD, M, K, N);
  if (ws_bytes < need || !ws) return fail(FFNK_E_WORKSPACE, "workspace %zu < %zu bytes", ws_bytes, need);
  if (!aligned16(ws)) return fail(FFNK_E_ALIGN, "workspace not 16-byte aligned");
  const RouteWs r = carve_route(static_cast<uint8_t*>(ws), M);
  if (const int kind = linear_stream_kind(M, K, N)) {
    // Decode sizes: the weight-streaming kernels of the FFN's down projection, fed token rows in
    // token order; they route from the mask themselves.
    if (kind == 2 && M * x_stride_m >= ((int64_t)1 << 30))
      return fail(FFNK_E_STRIDE, "x_stride_m=%lld: the decode kernels address the token rows with 32-bit offsets",
                  (long long)x_stride_m);
    const int splits = linear_stream_splits(M, K, N);
    StreamArgs a;
    a.X = x; a.ldx = x_stride_m; a.gather_x = 1; a.mask = mask; a.M = (int)M;
    a.W0[0] = Wv; a.W0[1] = Wt; a.W1[0] = a.W1[1] = nullptr; a.ldw = w_stride_n;
    a.Nrows = (int)N; a.K = (int)K; a.splits = splits; a.H = nullptr; a.ldh = 0;
    a.P = splits > 1 ? reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + r.bytes) : nullptr;
    a.out = y; a.ldo = y_stride_m;
    FFNK_HIP(kind == 1 ? launch_stream_dot_down(a, stream) : launch_stream_tile_down(a, stream), "streaming linear");
    if (splits > 1)
      FFNK_HIP(launch_stream_reduce(a.P, splits, (int)M, (int)N, mask, y, y_stride_m, stream), "streaming reduce");
    return FFNK_OK;
  }
  Routing rt;
  if (int e = resolve_routing(routing, r, mask, M, stream, &rt)) return e;
  GemmArgs g;
  g.A = x; g.lda = x_stride_m;
  g.B0[0] = Wv; g.B0[1] = Wt; g.B1[0] = g.B1[1] = nullptr; g.ldb = w_stride_n;
  g.C = y; g.ldc = y_stride_m;
  g.perm = rt.perm; g.counts = rt.counts;
  g.M = (int)M; g.N = (int)N; g.K = (int)K; g.group_m = plan_group_m(TUNED_PLAIN, M, K, N);
  const bool direct = direct_ok(K, M, x_stride_m, w_stride_n);
  RoutedPlan plan = linear_plan(M, K, N);
  if (!direct) {
    plan.splits = 1;
    plan.tile = routed_tile(M, N, false, K);
  }
  if (plan.splits > 1) {
    g.splits = plan.splits;
    g.P = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + r.bytes);
  } else if (direct && is_big_tile(plan.tile)) {
    g.P_tail = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + r.bytes);
  }
  FFNK_HIP(launch_linear_gemm(plan.tile, direct, g, stream), "linear GEMM");
  if (plan.splits > 1)
    FFNK_HIP(launch_routed_reduce(g.P, plan.splits, (int)M, (int)N, rt.perm, y, y_stride_m, stream), "linear reduce");
  return FFNK_OK;
}

int ffnk_masked_ffn_fwd(const uint16_t* x, int64_t x_stride_m, const uint16_t* W1, const uint16_t* W3,
                        const uint16_t* U1, const uint16_t* U3, int64_t up_stride_k, int64_t up_stride_n,
                        const uint16_t* W2, const uint16_t* U2, int64_t down_stride_k, int64_t down_stride_n,
                        const uint8_t* mask, uint16_t* out, int64_t out_stride_m, int64_t M, int64_t d,
                        int64_t h, void* ws, size_t ws_bytes, void* stream_) {
  return ffnk_masked_ffn_fwd_ev(x, x_stride_m, W1, W3, U1, U3, up_stride_k, up_stride_n, W2, U2, down_stride_k,
                                down_stride_n, mask, out, out_stride_m, M, d, h, ws, ws_bytes, stream_, nullptr);
}

}  // extern "C"

namespace {

// Forward shared by the entry points.  pre != NULL: also store the two pre-activations (routed order,
// [M, 2h], gate | up) for a later ffnk_masked_ffn_bwd_saved; only the LDS-tiled path can do that.
int ffn_fwd_impl(const uint16_t* x, int64_t x_stride_m, const uint16_t* W1, const uint16_t* W3, const uint16_t* U1,
                 const uint16_t* U3, int64_t up_stride_k, int64_t up_stride_n, const uint16_t* W2, const uint16_t* U2,
                 int64_t down_stride_k, int64_t down_stride_n, const uint8_t* mask, uint16_t* out, int64_t out_stride_m,
                 uint16_t* pre, int64_t pre_stride_m, int64_t M, int64_t d, int64_t h, void* ws, size_t ws_bytes,
                 void* stream_, void* const* events, const ffnk_routing_t* routing = nullptr) {
  hipStream_t stream = (hipStream_t)stream_;
  auto mark = [&](int i) -> hipError_t {
    if (events && events[i]) return hipEventRecord((hipEvent_t)events[i], stream);
    return hipSuccess;
  };
  if (int e = check_extents(M, d, h)) return e;
  if (M == 0 || d == 0) return FFNK_OK;
  if (!x || !mask || !out) return fail(FFNK_E_NULL, "x, mask or out is NULL");
  if (h > 0 && (!W1 || !W3 || !U1 || !U3 || !W2 || !U2)) return fail(FFNK_E_NULL, "weight pointer is NULL");
  if (!aligned2(x) || !aligned2(out) || !aligned2(W1) || !aligned2(W3) || !aligned2(U1) || !aligned2(U3) ||
      !aligned2(W2) || !aligned2(U2))
    return fail(FFNK_E_ALIGN, "bf16 pointer not 2-byte aligned");
  if (out_stride_m < d) return fail(FFNK_E_STRIDE, "out_stride_m=%lld < d=%lld", (long long)out_stride_m, (long long)d);
  if (pre != nullptr) {
    if (!ffnk_masked_ffn_can_save(M, d, h))
      return fail(FFNK_E_STRIDE, "MaskedFFN forward: pre-activations can only be saved on the LDS-tiled path "
                                 "(ffnk_masked_ffn_can_save)");
    if (pre_stride_m < 2 * h || pre_stride_m % 8 != 0 || !aligned16(pre))
      return fail(FFNK_E_STRIDE, "pre_stride_m=%lld: need >= 2h, a multiple of 8, and 16-byte aligned rows",
                  (long long)pre_stride_m);
  }
  const size_t need = ffnk_workspace_bytes(FFNK_OP_FFN_FWD, M, d, h);
  if (ws_bytes < need || !ws) return fail(FFNK_E_WORKSPACE, "workspace %zu < %zu bytes", ws_bytes, need);
  if (!aligned16(ws)) return fail(FFNK_E_ALIGN, "workspace not 16-byte aligned");

  uint8_t* wsb = static_cast<uint8_t*>(ws);
  const RouteWs r = carve_route(wsb, M);
  uint16_t* H = reinterpret_cast<uint16_t*>(wsb + r.bytes);
  const int64_t ldh = round_up64(h, 8);

  const bool fast = d % 8 == 0 && h > 0 && h % 8 == 0 && x_stride_m % 8 == 0 && x_stride_m >= d && aligned16(x) &&
                    up_stride_k == 1 && up_stride_n % 8 == 0 && up_stride_n >= d && down_stride_k == 1 &&
                    down_stride_n % 8 == 0 && down_stride_n >= h && aligned16(W1) && aligned16(W3) &&
                    aligned16(U1) && aligned16(U3) && aligned16(W2) && aligned16(U2);
  if (pre != nullptr && !fast)
    return fail(FFNK_E_STRIDE, "MaskedFFN forward: saving the pre-activations needs the fast layout (16-byte aligned, "
                               "K-contiguous operands)");
  if (!fast) {
    // Token-order intermediate, then the generic routed linear on it.
    GenericUpArgs u;
    u.x = x; u.sxm = x_stride_m;
    u.G[0] = W1; u.G[1] = U1; u.U[0] = W3; u.U[1] = U3; u.swk = up_stride_k; u.swn = up_stride_n;
    u.mask = mask; u.H = H; u.ldh = ldh;
    u.M = (int)M; u.K = (int)d; u.N = (int)h;
    FFNK_HIP(mark(0), "event record");
    FFNK_HIP(launch_generic_up(u, stream), "generic up kernel");
    FFNK_HIP(mark(1), "event record");
    GenericLinearArgs a;
    a.x = H; a.sxm = ldh; a.sxk = 1;
    a.W[0] = W2; a.W[1] = U2; a.swk = down_stride_k; a.swn = down_stride_n;
    a.mask = mask; a.y = out; a.sym = out_stride_m; a.syn = 1;
    a.M = (int)M; a.K = (int)h; a.N = (int)d;
    FFNK_HIP(launch_generic_linear(a, stream), "generic down kernel");
    FFNK_HIP(mark(2), "event record");
    return FFNK_OK;
  }

  if (use_stream_path(M, d, h)) {
    float* P = reinterpret_cast<float*>(wsb + r.bytes + ws_align((size_t)M * ldh * 2));
    const int splits = down_splits(M, d, h);
    FFNK_HIP(mark(0), "event record");
    StreamArgs u;
    u.X = x; u.ldx = x_stride_m; u.gather_x = 1; u.mask = mask; u.M = (int)M;
    u.W0[0] = W1; u.W0[1] = U1; u.W1[0] = W3; u.W1[1] = U3; u.ldw = up_stride_n;
    u.Nrows = (int)h; u.K = (int)d; u.splits = 1; u.H = H; u.ldh = ldh; u.P = nullptr; u.out = nullptr; u.ldo = 0;
    const bool dot = use_dot_path(M, d, h);
    const bool tiled = use_tile_path(M, d, h);
    if (tiled && M * x_stride_m >= ((int64_t)1 << 30))
      return fail(FFNK_E_STRIDE, "x_stride_m=%lld: the decode kernels address the token rows with 32-bit offsets",
                  (long long)x_stride_m);
    FFNK_HIP(dot ? launch_stream_dot_up(u, stream) : tiled ? launch_stream_tile_up(u, stream) : launch_stream_up(u, stream),
             "streaming up-projection");
    FFNK_HIP(mark(1), "event record");
    StreamArgs dn;
    dn.X = H; dn.ldx = ldh; dn.gather_x = 0; dn.mask = mask; dn.M = (int)M;
    dn.W0[0] = W2; dn.W0[1] = U2; dn.W1[0] = dn.W1[1] = nullptr; dn.ldw = down_stride_n;
    dn.Nrows = (int)d; dn.K = (int)h; dn.splits = splits; dn.H = nullptr; dn.ldh = 0;
    dn.P = splits > 1 ? P : nullptr; dn.out = out; dn.ldo = out_stride_m;
    FFNK_HIP(dot ? launch_stream_dot_down(dn, stream) : tiled ? launch_stream_tile_down(dn, stream) : launch_stream_down(dn, stream),
             "streaming down-projection");
    if (splits > 1)
      FFNK_HIP(launch_stream_reduce(P, splits, (int)M, (int)d, mask, out, out_stride_m, stream), "streaming reduce");
    FFNK_HIP(mark(2), "event record");
    return FFNK_OK;
  }

  Routing rt;
  if (int e = resolve_routing(routing, r, mask, M, stream, &rt)) return e;
  FFNK_HIP(mark(0), "event record");
  GemmArgs up;
  up.A = x; up.lda = x_stride_m;
  up.B0[0] = W1; up.B0[1] = U1; up.B1[0] = W3; up.B1[1] = U3; up.ldb = up_stride_n;
  up.C = H; up.ldc = ldh;
  up.perm = rt.perm; up.counts = rt.counts;
  up.M = (int)M; up.N = (int)h; up.K = (int)d; up.group_m = plan_group_m(TUNED_DUAL, M, d, h);
  up.C_pre = pre; up.ldc_pre = pre_stride_m;
  FFNK_HIP(launch_up_gemm(routed_tile(M, h, true, d), direct_ok(d, M, x_stride_m, up_stride_n), up, stream), "up-projection GEMM");
  FFNK_HIP(mark(1), "event record");
  GemmArgs dn;
  dn.A = H; dn.lda = ldh;
  dn.B0[0] = W2; dn.B0[1] = U2; dn.B1[0] = dn.B1[1] = nullptr; dn.ldb = down_stride_n;
  dn.C = out; dn.ldc = out_stride_m;
  dn.perm = rt.perm; dn.counts = rt.counts;
  dn.M = (int)M; dn.N = (int)d; dn.K = (int)h; dn.group_m = plan_group_m(TUNED_DOWN, M, h, d);
  const bool dn_direct = direct_ok(h, 0, ldh, down_stride_n);
  const int dn_splits = dn_direct ? tiled_down_splits(M, d, h) : 1;
  float* partials = reinterpret_cast<float*>(wsb + r.bytes + ws_align((size_t)M * ldh * 2));
  if (dn_splits > 1) {
    dn.splits = dn_splits;
    dn.P = partials;
  } else if (dn_direct && is_big_tile(down_tile(M, d, h))) {
    dn.P_tail = partials;  // the last, partial round of 256x256 tiles runs cut into K ranges
  }
  FFNK_HIP(launch_down_gemm(down_tile(M, d, h), dn_direct, dn, stream), "down-projection GEMM");
  if (dn_splits > 1)
    FFNK_HIP(launch_routed_reduce(dn.P, dn_splits, (int)M, (int)d, rt.perm, out, out_stride_m, stream), "down-projection reduce");
  FFNK_HIP(mark(2), "event record");
  return FFNK_OK;
}

}  // namespace

extern "C" {

int ffnk_masked_ffn_fwd_ev(const uint16_t* x, int64_t x_stride_m, const uint16_t* W1, const uint16_t* W3,
                           const uint16_t* U1, const uint16_t* U3, int64_t up_stride_k, int64_t up_stride_n,
                           const uint16_t* W2, const uint16_t* U2, int64_t down_stride_k, int64_t down_stride_n,
                           const uint8_t* mask, uint16_t* out, int64_t out_stride_m, int64_t M, int64_t d,
                           int64_t h, void* ws, size_t ws_bytes, void* stream_, void* const* events) {
  return ffn_fwd_impl(x, x_stride_m, W1, W3, U1, U3, up_stride_k, up_stride_n, W2, U2, down_stride_k, down_stride_n, mask,
                      out, out_stride_m, nullptr, 0, M, d, h, ws, ws_bytes, stream_, events);
}

int ffnk_masked_ffn_fwd_static(const uint16_t* x, int64_t x_stride_m, const uint16_t* W1, const uint16_t* W3,
                               const uint16_t* U1, const uint16_t* U3, int64_t up_stride_k, int64_t up_stride_n,
                               const uint16_t* W2, const uint16_t* U2, int64_t down_stride_k, int64_t down_stride_n,
                               const uint8_t* mask, uint16_t* out, int64_t out_stride_m, int64_t M, int64_t d,
                               int64_t h, void* stream_) {
  if (int e = check_extents(M, d, h)) return e;
  const size_t need = ffnk_workspace_bytes(FFNK_OP_FFN_FWD, M, d, h);
  if (need > (size_t)FFNK_STATIC_SCRATCH_BYTES)
    return fail(FFNK_E_WORKSPACE, "ffnk_masked_ffn_fwd_static: M=%lld d=%lld h=%lld needs %zu bytes of scratch, the static "
                                  "buffer holds %zu; use ffnk_masked_ffn_fwd with a workspace",
                (long long)M, (long long)d, (long long)h, need, (size_t)FFNK_STATIC_SCRATCH_BYTES);
  if (M == 0 || d == 0) return FFNK_OK;
  if (!out) return fail(FFNK_E_NULL, "x, mask or out is NULL");
  void* ws = nullptr;
  if (int e = static_scratch(out, &ws)) return e;
  // Nothing in the scratch has to start at zero: every region the forward reads (perm, counts, the
  // intermediate, the fp32 partials) is written by an earlier kernel of the same call.
  return ffn_fwd_impl(x, x_stride_m, W1, W3, U1, U3, up_stride_k, up_stride_n, W2, U2, down_stride_k, down_stride_n, mask,
                      out, out_stride_m, nullptr, 0, M, d, h, ws, (size_t)FFNK_STATIC_SCRATCH_BYTES, stream_, nullptr);
}

int ffnk_masked_ffn_fwd_routed(const uint16_t* x, int64_t x_stride_m, const uint16_t* W1, const uint16_t* W3,
                               const uint16_t* U1, const uint16_t* U3, int64_t up_stride_k, int64_t up_stride_n,
                               const uint16_t* W2, const uint16_t* U2, int64_t down_stride_k, int64_t down_stride_n,
                               const uint8_t* mask, uint16_t* out, int64_t out_stride_m, uint16_t* pre,
                               int64_t pre_stride_m, int64_t M, int64_t d, int64_t h, void* ws, size_t ws_bytes,
                               void* stream_, const ffnk_routing_t* routing) {
  return ffn_fwd_impl(x, x_stride_m, W1, W3, U1, U3, up_stride_k, up_stride_n, W2, U2, down_stride_k, down_stride_n, mask,
                      out, out_stride_m, pre, pre_stride_m, M, d, h, ws, ws_bytes, stream_, nullptr, routing);
}

int ffnk_masked_ffn_can_save(int64_t M, int64_t d, int64_t h) {
  return (M > 0 && d > 0 && h > 0 && d % 8 == 0 && h % 8 == 0 && !use_stream_path(M, d, h)) ? 1 : 0;
}

int ffnk_masked_ffn_fwd_save(const uint16_t* x, int64_t x_stride_m, const uint16_t* W1, const uint16_t* W3,
                             const uint16_t* U1, const uint16_t* U3, int64_t up_stride_k, int64_t up_stride_n,
                             const uint16_t* W2, const uint16_t* U2, int64_t down_stride_k, int64_t down_stride_n,
                             const uint8_t* mask, uint16_t* out, int64_t out_stride_m, uint16_t* pre,
                             int64_t pre_stride_m, int64_t M, int64_t d, int64_t h, void* ws, size_t ws_bytes,
                             void* stream_) {
  if (!pre) return fail(FFNK_E_NULL, "pre is NULL");
  return ffn_fwd_impl(x, x_stride_m, W1, W3, U1, U3, up_stride_k, up_stride_n, W2, U2, down_stride_k, down_stride_n, mask,
                      out, out_stride_m, pre, pre_stride_m, M, d, h, ws, ws_bytes, stream_, nullptr);
}

int ffnk_masked_linear_bwd(const uint16_t* g, int64_t g_stride_m, const uint16_t* x, int64_t x_stride_m,
                           const uint16_t* Wv, const uint16_t* Wt, int64_t w_stride_k, int64_t w_stride_n,
                           const uint8_t* mask, uint16_t* dx, int64_t dx_stride_m, uint16_t* dWv, uint16_t* dWt,
                           int64_t dw_stride_k, int64_t dw_stride_n, int64_t M, int64_t K, int64_t N, void* ws,
                           size_t ws_bytes, void* stream_) {
  return ffnk_masked_linear_bwd_routed(g, g_stride_m, x, x_stride_m, Wv, Wt, w_stride_k, w_stride_n, mask, dx, dx_stride_m,
                                       dWv, dWt, dw_stride_k, dw_stride_n, M, K, N, ws, ws_bytes, stream_, nullptr);
}

int ffnk_masked_linear_bwd_routed(const uint16_t* g, int64_t g_stride_m, const uint16_t* x, int64_t x_stride_m,
                                  const uint16_t* Wv, const uint16_t* Wt, int64_t w_stride_k, int64_t w_stride_n,
                                  const uint8_t* mask, uint16_t* dx, int64_t dx_stride_m, uint16_t* dWv, uint16_t* dWt,
                                  int64_t dw_stride_k, int64_t dw_stride_n, int64_t M, int64_t K, int64_t N, void* ws,
                                  size_t ws_bytes, void* stream_, const ffnk_routing_t* routing) {
  hipStream_t stream = (hipStream_t)stream_;
  if (int e = check_extents(M, K, N)) return e;
  if (K == 0) return FFNK_OK;  // dx and dW are empty
  if (M > 0 && (!mask || !dx || !x)) return fail(FFNK_E_NULL, "mask, x or dx is NULL");
  if (M > 0 && N > 0 && (!g || !Wv || !Wt)) return fail(FFNK_E_NULL, "g or weight pointer is NULL");
  if (N > 0 && (!dWv || !dWt)) return fail(FFNK_E_NULL, "dW pointer is NULL");
  if (!aligned2(g) || !aligned2(x) || !aligned2(Wv) || !aligned2(Wt) || !aligned2(dx) || !aligned2(dWv) || !aligned2(dWt))
    return fail(FFNK_E_ALIGN, "bf16 pointer not 2-byte aligned");
  if (dx_stride_m < K) return fail(FFNK_E_STRIDE, "dx_stride_m=%lld < K=%lld", (long long)dx_stride_m, (long long)K);

  const bool fast = M > 0 && N > 0 && K % 8 == 0 && N % 8 == 0 && g_stride_m % 8 == 0 && g_stride_m >= N &&
                    x_stride_m % 8 == 0 && x_stride_m >= K && aligned16(g) && aligned16(x) &&
                    direct_ok(64, 0, padded_rows(M), padded_rows(M));  // transposed operands have M-long rows
  if (!fast) {
    GenericBwdArgs a;
    a.g = g; a.sgm = g_stride_m; a.x = x; a.sxm = x_stride_m;
    a.W[0] = Wv; a.W[1] = Wt; a.swk = w_stride_k; a.swn = w_stride_n;
    a.mask = mask; a.dx = dx; a.sdxm = dx_stride_m;
    a.dW[0] = dWv; a.dW[1] = dWt; a.sdk = dw_stride_k; a.sdn = dw_stride_n;
    a.M = (int)M; a.K = (int)K; a.N = (int)N;
    FFNK_HIP(launch_generic_bwd(a, stream), "generic backward kernels");
    return FFNK_OK;
  }

  const BwdPlan p = plan_bwd(M, K, N, dw_stride_k == 1);
  if (ws_bytes < p.total || !ws) return fail(FFNK_E_WORKSPACE, "workspace %zu < %zu bytes", ws_bytes, p.total);
  if (!aligned16(ws)) return fail(FFNK_E_ALIGN, "workspace not 16-byte aligned");
  uint8_t* wsb = static_cast<uint8_t*>(ws);
  const RouteWs r = carve_route(wsb, M);
  Routing rt;
  if (int e = resolve_routing(routing, r, mask, M, stream, &rt)) return e;

  // ---- dx = gather(g) @ W_g^T, contraction over N: needs the weights as [K, N] rows, N contiguous ----
  const uint16_t* wt[2] = {Wv, Wt};
  int64_t ldw = w_stride_k;
  const bool w_direct = w_stride_n == 1 && w_stride_k % 8 == 0 && w_stride_k >= N && aligned16(Wv) && aligned16(Wt);
  // The forward's layout ([N, K] rows, K contiguous) is K-major for this GEMM: no copy either.
  const bool w_kmajor = !w_direct && w_stride_k == 1 && kmajor_ok(N, K, w_stride_n, Wv, Wt) && direct_ok(N, M, g_stride_m, 8);
  if (w_kmajor) {
    ldw = w_stride_n;
  } else if (!w_direct) {
    uint16_t* c0 = reinterpret_cast<uint16_t*>(wsb + p.off_wt);
    uint16_t* c1 = reinterpret_cast<uint16_t*>(wsb + p.off_wt + ws_align((size_t)K * N * 2));
    FFNK_HIP(launch_strided_copy2d(Wv, w_stride_k, w_stride_n, c0, N, (int)K, (int)N, stream), "weight transpose");
    FFNK_HIP(launch_strided_copy2d(Wt, w_stride_k, w_stride_n, c1, N, (int)K, (int)N, stream), "weight transpose");
    wt[0] = c0; wt[1] = c1; ldw = N;
  }
  GemmArgs a;
  a.A = g; a.lda = g_stride_m;
  a.B0[0] = wt[0]; a.B0[1] = wt[1]; a.B1[0] = a.B1[1] = nullptr; a.ldb = ldw;
  a.C = dx; a.ldc = dx_stride_m;
  a.perm = rt.perm; a.counts = rt.counts;
  a.M = (int)M; a.N = (int)K; a.K = (int)N; a.group_m = plan_group_m(TUNED_NONE, M, N, K);
  const int dx_tile = routed_tile(M, K, false, 0, TUNED_NONE);
  // Both GEMMs on the 128x128 tile and the weights readable in place: one launch runs the two side by
  // side (after the transposes it depends on), see below.
  const bool gather = p.gather && gather_dw_ok(M, K, N, g, g_stride_m, x, x_stride_m);
  const bool fused = bwd_is_fused(M, K, p, w_kmajor, gather);
  if (!fused) {
    if (w_kmajor) FFNK_HIP(launch_linear_gemm_kmajor(dx_tile, a, stream), "dx GEMM");
    else FFNK_HIP(launch_linear_gemm(dx_tile, direct_ok(N, M, g_stride_m, ldw), a, stream), "dx GEMM");
  }

  // ---- dW_g = x_g^T g_g, contraction over the rows of group g ----
  float* P = reinterpret_cast<float*>(wsb + p.off_p);
  SplitKArgs s;
  s.P = P; s.counts = rt.counts; s.M = (int)M;
  s.R = (int)p.R; s.Cc = (int)p.Cc; s.splits = p.tc.splits;
  const int64_t sr = p.dw_k_contig ? dw_stride_n : dw_stride_k;
  const int64_t sc = p.dw_k_contig ? dw_stride_k : dw_stride_n;
  s.splits = bwd_dw_launch_splits(M, K, N, p, fused);
  if (s.splits == 1) { s.out[0] = dWv; s.out[1] = dWt; s.out_sr = sr; s.out_sc = sc; }
  if (gather) {
    // g and x read where they lie: the row operand of the output is g when dW's memory is [N, K], x otherwise
    GatherDwArgs gw;
    gw.G = p.dw_k_contig ? g : x; gw.ldg = p.dw_k_contig ? g_stride_m : x_stride_m;
    gw.X = p.dw_k_contig ? x : g; gw.ldx = p.dw_k_contig ? x_stride_m : g_stride_m;
    gw.perm = rt.perm; gw.counts = rt.counts;
    s.A = s.B = nullptr; s.lda = s.ldb = 0;
    gw.s = s;
    if (fused) FFNK_HIP(launch_fused_bwd_gather(a, gw, stream), "fused dx / dW GEMM");
    else FFNK_HIP(launch_gathered_dw(gw, stream), "dW GEMM");
  } else {
    uint16_t* GT = reinterpret_cast<uint16_t*>(wsb + p.off_gt);  // [N, ldt]
    uint16_t* XT = reinterpret_cast<uint16_t*>(wsb + p.off_xt);  // [K, ldt]
    FFNK_HIP(launch_gather_transpose2(g, g_stride_m, (int)N, GT, x, x_stride_m, (int)K, XT, p.ldt, rt.perm, rt.counts,
                                      (int)M, stream), "g / x transpose");
    s.A = p.dw_k_contig ? GT : XT; s.lda = p.ldt;
    s.B = p.dw_k_contig ? XT : GT; s.ldb = p.ldt;
    if (fused) FFNK_HIP(launch_fused_bwd(a, s, p.tc.tile == TILE_128x128_R4, stream), "fused dx / dW GEMM");
    else FFNK_HIP(launch_splitk_gemm(p.tc.tile, s, stream), "dW split-K GEMM");
  }
  if (s.splits > 1)
    FFNK_HIP(launch_splitk_reduce(P, s.splits, (int)p.R, (int)p.Cc, dWv, dWt, sr, sc, stream), "dW reduce");
  return FFNK_OK;
}

}  // extern "C"

namespace {

// Backward shared by the entry points.  pre != NULL: the pre-activations a forward saved
// (ffnk_masked_ffn_fwd_save, same mask), read-only; NULL: recompute them with two routed GEMMs.
int ffn_bwd_impl(const uint16_t* g, int64_t g_stride_m, const uint16_t* x, int64_t x_stride_m, const uint16_t* W1,
                 const uint16_t* W3, const uint16_t* U1, const uint16_t* U3, int64_t up_stride_k, int64_t up_stride_n,
                 const uint16_t* W2, const uint16_t* U2, int64_t down_stride_k, int64_t down_stride_n,
                 const uint8_t* mask, const uint16_t* pre, int64_t pre_stride_m, uint16_t* dx, int64_t dx_stride_m,
                 uint16_t* dW1, uint16_t* dW3, uint16_t* dU1, uint16_t* dU3, int64_t dup_stride_k, int64_t dup_stride_n,
                 uint16_t* dW2, uint16_t* dU2, int64_t ddown_stride_k, int64_t ddown_stride_n, int64_t M, int64_t d,
                 int64_t h, void* ws, size_t ws_bytes, void* stream_, const ffnk_routing_t* routing = nullptr) {
  hipStream_t stream = (hipStream_t)stream_;
  if (pre != nullptr && (pre_stride_m < 2 * h || pre_stride_m % 8 != 0 || !aligned16(pre)))
    return fail(FFNK_E_STRIDE, "pre_stride_m=%lld: need >= 2h, a multiple of 8, and 16-byte aligned rows",
                (long long)pre_stride_m);
  if (int e = check_extents(M, d, h)) return e;
  if (d == 0 || h == 0) return fail(FFNK_E_SHAPE, "MaskedFFN backward needs d > 0 and h > 0");
  if (!W1 || !W3 || !U1 || !U3 || !W2 || !U2 || !dW1 || !dW3 || !dU1 || !dU3 || !dW2 || !dU2)
    return fail(FFNK_E_NULL, "weight or weight-gradient pointer is NULL");
  if (M > 0 && (!g || !x || !mask || !dx)) return fail(FFNK_E_NULL, "g, x, mask or dx is NULL");
  if (dx_stride_m < d) return fail(FFNK_E_STRIDE, "dx_stride_m=%lld < d=%lld", (long long)dx_stride_m, (long long)d);
  const bool ok = d % 8 == 0 && h % 8 == 0 && g_stride_m % 8 == 0 && g_stride_m >= d && x_stride_m % 8 == 0 &&
                  x_stride_m >= d && (M == 0 || (aligned16(g) && aligned16(x))) && up_stride_k == 1 &&
                  up_stride_n % 8 == 0 && up_stride_n >= d && aligned16(W1) && aligned16(W3) && aligned16(U1) &&
                  aligned16(U3) && aligned2(W2) && aligned2(U2) && aligned2(dx) && aligned2(dW1) && aligned2(dW3) &&
                  aligned2(dU1) && aligned2(dU3) && aligned2(dW2) && aligned2(dU2) &&
                  direct_ok(64, 0, padded_rows(M), padded_rows(M));
  if (!ok)
    return fail(FFNK_E_STRIDE, "MaskedFFN backward: d, h and the row strides must be multiples of 8, rows 16-byte "
                               "aligned and the up-projection weights K-contiguous (up_stride_k == 1)");
  // Which optional regions this layout needs (ffnk_workspace_bytes_ffn_bwd asks the same function).
  const int64_t ld13 = 2 * h;
  bool w2_direct = false, w2_kmajor = false, w13_kmajor = false;
  const FfnBwdPaths paths = ffn_bwd_paths(M, d, h, g_stride_m, up_stride_n, down_stride_k, down_stride_n, W1, W3, U1, U3, W2,
                                          U2, &w2_direct, &w2_kmajor, &w13_kmajor);
  const FfnBwdPlan p = plan_ffn_bwd(M, d, h, dup_stride_k == 1, ddown_stride_k == 1, paths);
  if (ws_bytes < p.total || !ws)
    return fail(FFNK_E_WORKSPACE, "workspace %zu < %zu bytes (ffnk_workspace_bytes_ffn_bwd sizes it for aligned pointers; "
                                  "ffnk_workspace_bytes(FFNK_OP_FFN_BWD) for any layout)", ws_bytes, p.total);
  if (!aligned16(ws)) return fail(FFNK_E_ALIGN, "workspace not 16-byte aligned");
  uint8_t* wsb = static_cast<uint8_t*>(ws);
  const RouteWs r = carve_route(wsb, M);
  uint16_t* T13 = reinterpret_cast<uint16_t*>(wsb + p.off_t13);
  uint16_t* DH = reinterpret_cast<uint16_t*>(wsb + p.off_dh);
  Routing rt;
  if (int e = resolve_routing(routing, r, mask, M, stream, &rt)) return e;

  // ---- pre-activations, routed order: T13[:, 0:h] = x A1, T13[:, h:2h] = x A3 ----
  GemmArgs a;
  a.A = x; a.lda = x_stride_m;
  a.B1[0] = a.B1[1] = nullptr; a.ldb = up_stride_n;
  a.ldc = ld13; a.perm = rt.perm; a.counts = rt.counts;
  a.M = (int)M; a.N = (int)h; a.K = (int)d; a.group_m = plan_group_m(TUNED_NONE, M, d, h);
  const bool up_direct = direct_ok(d, M, x_stride_m, up_stride_n);
  if (pre == nullptr) {
    a.B0[0] = W1; a.B0[1] = U1; a.C = T13;
    FFNK_HIP(launch_gather_gemm(routed_tile(M, h, false), up_direct, a, stream), "t1 GEMM");
    a.B0[0] = W3; a.B0[1] = U3; a.C = T13 + h;
    FFNK_HIP(launch_gather_gemm(routed_tile(M, h, false), up_direct, a, stream), "t3 GEMM");
  }

  // ---- dh = gather(g) @ A2^T: contraction over d needs the down weights as [h, d] rows ----
  const uint16_t* w2t[2] = {W2, U2};
  int64_t ld2 = down_stride_k;
  if (w2_kmajor) {
    ld2 = down_stride_n;
  } else if (!w2_direct) {
    uint16_t* c0 = reinterpret_cast<uint16_t*>(wsb + p.off_w2t);
    uint16_t* c1 = reinterpret_cast<uint16_t*>(wsb + p.off_w2t + ws_align((size_t)h * d * 2));
    FFNK_HIP(launch_strided_copy2d(W2, down_stride_k, down_stride_n, c0, d, (int)h, (int)d, stream), "weight transpose");
    FFNK_HIP(launch_strided_copy2d(U2, down_stride_k, down_stride_n, c1, d, (int)h, (int)d, stream), "weight transpose");
    w2t[0] = c0; w2t[1] = c1; ld2 = d;
  }
  a.A = g; a.lda = g_stride_m; a.B0[0] = w2t[0]; a.B0[1] = w2t[1]; a.ldb = ld2;
  a.C = DH; a.ldc = h;
  if (w2_kmajor) FFNK_HIP(launch_gather_gemm_kmajor(routed_tile(M, h, false), a, stream), "dh GEMM");
  else FFNK_HIP(launch_gather_gemm(routed_tile(M, h, false), direct_ok(d, M, g_stride_m, ld2), a, stream), "dh GEMM");

  // ---- elementwise: T13 <- (dt1 | dt3), DH <- the SwiGLU intermediate ----
  FFNK_HIP(launch_swiglu_bwd(pre ? pre : T13, pre ? pre_stride_m : ld13, T13, ld13, DH, h, (int)M, (int)h, stream),
           "SwiGLU backward pass");

  // ---- dx = (dt1 | dt3) @ (A1^T | A3^T)^T: one GEMM over the concatenated contraction of length 2h ----
  // In place over the K-major up-projection weights, or over one [d, 2h] copy per modality.
  GemmArgs b;
  b.A = T13; b.lda = ld13;
  if (w13_kmajor) {
    b.B0[0] = W1; b.B0[1] = U1; b.B1[0] = W3; b.B1[1] = U3; b.ldb = up_stride_n;
    b.k_switch = (int)h;
  } else {
    uint16_t* w13[2] = {reinterpret_cast<uint16_t*>(wsb + p.off_w13t),
                        reinterpret_cast<uint16_t*>(wsb + p.off_w13t + ws_align((size_t)d * 2 * h * 2))};
    FFNK_HIP(launch_strided_copy2d(W1, up_stride_k, up_stride_n, w13[0], ld13, (int)d, (int)h, stream), "weight transpose");
    FFNK_HIP(launch_strided_copy2d(W3, up_stride_k, up_stride_n, w13[0] + h, ld13, (int)d, (int)h, stream), "weight transpose");
    FFNK_HIP(launch_strided_copy2d(U1, up_stride_k, up_stride_n, w13[1], ld13, (int)d, (int)h, stream), "weight transpose");
    FFNK_HIP(launch_strided_copy2d(U3, up_stride_k, up_stride_n, w13[1] + h, ld13, (int)d, (int)h, stream), "weight transpose");
    b.B0[0] = w13[0]; b.B0[1] = w13[1]; b.B1[0] = b.B1[1] = nullptr; b.ldb = ld13;
  }
  b.C = dx; b.ldc = dx_stride_m; b.perm = rt.perm; b.counts = rt.counts;
  b.M = (int)M; b.N = (int)d; b.K = (int)(2 * h); b.group_m = plan_group_m(TUNED_NONE, M, 2 * h, d);
  // Few output tiles over a 2h-long contraction: split K like the forward's down projection.  The
  // fp32 partials live where the W2^T copies were (dead since the dh GEMM), if they fit there.
  const bool dx_direct = paths.dx_direct;
  size_t dx_need = 0;
  const RoutedPlan dxp = ffn_bwd_dx_plan(M, d, h, dx_direct, 2 * ws_align((size_t)h * d * 2), &dx_need);
  if (dx_need > p.w2t_bytes) return fail(FFNK_E_WORKSPACE, "internal: dx partials %zu > %zu planned", dx_need, p.w2t_bytes);
  if (dxp.splits > 1) {
    b.splits = dxp.splits;
    b.P = reinterpret_cast<float*>(wsb + p.off_w2t);
  } else if (dx_need > 0) {
    b.P_tail = reinterpret_cast<float*>(wsb + p.off_w2t);  // split tail of the last, partial round
  }
  if (w13_kmajor) FFNK_HIP(launch_down_gemm_kmajor(dxp.tile, b, stream), "dx GEMM");
  else FFNK_HIP(launch_down_gemm(dxp.tile, dx_direct, b, stream), "dx GEMM");
  if (dxp.splits > 1)
    FFNK_HIP(launch_routed_reduce(b.P, dxp.splits, (int)M, (int)d, rt.perm, dx, dx_stride_m, stream), "dx reduce");

  // ---- weight gradients: contraction over the rows of each group.  x and g are gathered into
  // 64-padded transposes; H, dt1 and dt3 (routed order already) are read in place by the K-major
  // kernels, or transposed as well when their row strides do not fit 32-bit slab offsets. ----
  uint16_t* GT = reinterpret_cast<uint16_t*>(wsb + p.off_gt);    // [d, ldt]
  uint16_t* XT = reinterpret_cast<uint16_t*>(wsb + p.off_xt);    // [d, ldt]
  float* P = reinterpret_cast<float*>(wsb + p.off_p);
  const bool in_place = paths.acts_in_place;
  if (in_place) {
    FFNK_HIP(launch_gather_transpose2(g, g_stride_m, (int)d, GT, x, x_stride_m, (int)d, XT, p.ldt, rt.perm, rt.counts, (int)M,
                                      stream, false, false), "g / x transpose");
    const TileChoice tc = ffn_bwd_in_place_choice(M, d, h);
    const int tile = forced_tile() >= 0 ? forced_tile() : tc.tile;
    // out[r * sr + c * sc]: r runs over h (the in-place operand's columns), c over d
    auto weight_grad_in_place = [&](const uint16_t* rows, int64_t ld_rows, const uint16_t* cT, uint16_t* o0, uint16_t* o1,
                                    int64_t sr, int64_t sc) -> int {
      SplitKArgs s;
      s.A = rows; s.lda = ld_rows;
      s.B = cT; s.ldb = p.ldt;
      s.P = P; s.counts = rt.counts; s.M = (int)M;
      s.R = (int)h; s.Cc = (int)d; s.splits = tc.splits;
      if (tc.splits == 1) { s.out[0] = o0; s.out[1] = o1; s.out_sr = sr; s.out_sc = sc; }
      FFNK_HIP(launch_splitk_gemm_kmajor(tile, s, stream), "dW split-K GEMM");
      if (tc.splits > 1)
        FFNK_HIP(launch_splitk_reduce(P, tc.splits, (int)h, (int)d, o0, o1, sr, sc, stream), "dW reduce");
      return FFNK_OK;
    };
    if (int e = weight_grad_in_place(DH, h, GT, dW2, dU2, ddown_stride_k, ddown_stride_n)) return e;
    if (int e = weight_grad_in_place(T13, ld13, XT, dW1, dU1, dup_stride_n, dup_stride_k)) return e;
    if (int e = weight_grad_in_place(T13 + h, ld13, XT, dW3, dU3, dup_stride_n, dup_stride_k)) return e;
    return FFNK_OK;
  }
  uint16_t* HT = reinterpret_cast<uint16_t*>(wsb + p.off_ht);    // [h, ldt]
  uint16_t* D1T = reinterpret_cast<uint16_t*>(wsb + p.off_d1t);  // [h, ldt]
  uint16_t* D3T = reinterpret_cast<uint16_t*>(wsb + p.off_d3t);  // [h, ldt]
  FFNK_HIP(launch_gather_transpose2(g, g_stride_m, (int)d, GT, DH, h, (int)h, HT, p.ldt, rt.perm, rt.counts, (int)M,
                                    stream, false, true), "g / intermediate transpose");
  FFNK_HIP(launch_gather_transpose2(x, x_stride_m, (int)d, XT, T13, ld13, (int)h, D1T, p.ldt, rt.perm, rt.counts,
                                    (int)M, stream, false, true), "x / dt1 transpose");
  FFNK_HIP(launch_gather_transpose2(T13 + h, ld13, (int)h, D3T, nullptr, 0, 0, nullptr, p.ldt, rt.perm, rt.counts,
                                    (int)M, stream, true, false), "dt3 transpose");
  auto weight_grad = [&](const BwdPlan& q, const uint16_t* gT, const uint16_t* xT, uint16_t* o0, uint16_t* o1,
                         int64_t sk, int64_t sn) -> int {
    SplitKArgs s;
    s.A = q.dw_k_contig ? gT : xT; s.lda = p.ldt;
    s.B = q.dw_k_contig ? xT : gT; s.ldb = p.ldt;
    s.P = P; s.counts = rt.counts; s.M = (int)M;
    s.R = (int)q.R; s.Cc = (int)q.Cc; s.splits = q.tc.splits;
    const int64_t sr = q.dw_k_contig ? sn : sk, sc = q.dw_k_contig ? sk : sn;
    if (q.tc.splits == 1) { s.out[0] = o0; s.out[1] = o1; s.out_sr = sr; s.out_sc = sc; }
    FFNK_HIP(launch_splitk_gemm(q.tc.tile, s, stream), "dW split-K GEMM");
    if (q.tc.splits > 1)
      FFNK_HIP(launch_splitk_reduce(P, q.tc.splits, (int)q.R, (int)q.Cc, o0, o1, sr, sc, stream), "dW reduce");
    return FFNK_OK;
  };
  if (int e = weight_grad(p.dn, GT, HT, dW2, dU2, ddown_stride_k, ddown_stride_n)) return e;
  if (int e = weight_grad(p.up, D1T, XT, dW1, dU1, dup_stride_k, dup_stride_n)) return e;
  if (int e = weight_grad(p.up, D3T, XT, dW3, dU3, dup_stride_k, dup_stride_n)) return e;
  return FFNK_OK;
}

}  // namespace

extern "C" {

int ffnk_masked_ffn_bwd(const uint16_t* g, int64_t g_stride_m, const uint16_t* x, int64_t x_stride_m,
                        const uint16_t* W1, const uint16_t* W3, const uint16_t* U1, const uint16_t* U3,
                        int64_t up_stride_k, int64_t up_stride_n, const uint16_t* W2, const uint16_t* U2,
                        int64_t down_stride_k, int64_t down_stride_n, const uint8_t* mask, uint16_t* dx,
                        int64_t dx_stride_m, uint16_t* dW1, uint16_t* dW3, uint16_t* dU1, uint16_t* dU3,
                        int64_t dup_stride_k, int64_t dup_stride_n, uint16_t* dW2, uint16_t* dU2,
                        int64_t ddown_stride_k, int64_t ddown_stride_n, int64_t M, int64_t d, int64_t h, void* ws,
                        size_t ws_bytes, void* stream_) {
  return ffn_bwd_impl(g, g_stride_m, x, x_stride_m, W1, W3, U1, U3, up_stride_k, up_stride_n, W2, U2, down_stride_k,
                      down_stride_n, mask, nullptr, 0, dx, dx_stride_m, dW1, dW3, dU1, dU3, dup_stride_k, dup_stride_n,
                      dW2, dU2, ddown_stride_k, ddown_stride_n, M, d, h, ws, ws_bytes, stream_);
}

int ffnk_masked_ffn_bwd_routed(const uint16_t* g, int64_t g_stride_m, const uint16_t* x, int64_t x_stride_m,
                               const uint16_t* W1, const uint16_t* W3, const uint16_t* U1, const uint16_t* U3,
                               int64_t up_stride_k, int64_t up_stride_n, const uint16_t* W2, const uint16_t* U2,
                               int64_t down_stride_k, int64_t down_stride_n, const uint8_t* mask, const uint16_t* pre,
                               int64_t pre_stride_m, uint16_t* dx, int64_t dx_stride_m, uint16_t* dW1, uint16_t* dW3,
                               uint16_t* dU1, uint16_t* dU3, int64_t dup_stride_k, int64_t dup_stride_n, uint16_t* dW2,
                               uint16_t* dU2, int64_t ddown_stride_k, int64_t ddown_stride_n, int64_t M, int64_t d,
                               int64_t h, void* ws, size_t ws_bytes, void* stream_, const ffnk_routing_t* routing) {
  return ffn_bwd_impl(g, g_stride_m, x, x_stride_m, W1, W3, U1, U3, up_stride_k, up_stride_n, W2, U2, down_stride_k,
                      down_stride_n, mask, pre, pre_stride_m, dx, dx_stride_m, dW1, dW3, dU1, dU3, dup_stride_k,
                      dup_stride_n, dW2, dU2, ddown_stride_k, ddown_stride_n, M, d, h, ws, ws_bytes, stream_, routing);
}

int ffnk_masked_ffn_bwd_saved(const uint16_t* g, int64_t g_stride_m, const uint16_t* x, int64_t x_stride_m,
                              const uint16_t* W1, const uint16_t* W3, const uint16_t* U1, const uint16_t* U3,
                              int64_t up_stride_k, int64_t up_stride_n, const uint16_t* W2, const uint16_t* U2,
                              int64_t down_stride_k, int64_t down_stride_n, const uint8_t* mask, const uint16_t* pre,
                              int64_t pre_stride_m, uint16_t* dx, int64_t dx_stride_m, uint16_t* dW1, uint16_t* dW3,
                              uint16_t* dU1, uint16_t* dU3, int64_t dup_stride_k, int64_t dup_stride_n, uint16_t* dW2,
                              uint16_t* dU2, int64_t ddown_stride_k, int64_t ddown_stride_n, int64_t M, int64_t d,
                              int64_t h, void* ws, size_t ws_bytes, void* stream_) {
  if (M > 0 && !pre) return fail(FFNK_E_NULL, "pre is NULL");
  return ffn_bwd_impl(g, g_stride_m, x, x_stride_m, W1, W3, U1, U3, up_stride_k, up_stride_n, W2, U2, down_stride_k,
                      down_stride_n, mask, pre, pre_stride_m, dx, dx_stride_m, dW1, dW3, dU1, dU3, dup_stride_k,
                      dup_stride_n, dW2, dU2, ddown_stride_k, ddown_stride_n, M, d, h, ws, ws_bytes, stream_);
}

}  // extern "C"
