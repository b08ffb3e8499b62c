/*
 * ffnk.h — C ABI of libffnk.so: mask-routed bf16 linear / SwiGLU-FFN kernels for
 * AMD MI355X (gfx950).
 *
 * This is the boundary the reference crosses when its Python launchers start a Triton
 * kernel (ffn_kernel/linear.py:418-452, 455-496; ffn_kernel/ffn.py:527-560).  Every
 * pointer below is a DEVICE pointer unless its comment says otherwise.  Every entry
 * point only enqueues work on `stream` (a hipStream_t passed as void*, NULL = the
 * null stream): no host synchronisation, no allocation, no free.  Scratch memory is
 * supplied by the caller through (`ws`, `ws_bytes`); its required size comes from
 * ffnk_workspace_bytes().
 *
 * Return value of every int-returning function: 0 on success; a negative FFNK_E_*
 * code for a rejected argument; a positive value is a hipError_t from the runtime.
 * ffnk_last_error() returns a thread-local text for the last non-zero return.
 *
 * Tensors are bf16 stored as uint16_t.  `mask` is one byte per token row
 * (torch.bool storage): non-zero = visual row, zero = text row.
 */
#ifndef FFNK_H
#define FFNK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FFNK_VERSION 102

#if defined(__GNUC__)
#define FFNK_API __attribute__((visibility("default")))
#else
#define FFNK_API
#endif

enum {
  FFNK_OK = 0,
  FFNK_E_NULL = -1,       /* a required pointer is NULL                         */
  FFNK_E_SHAPE = -2,      /* negative / overflowing / unsupported extent        */
  FFNK_E_STRIDE = -3,     /* stride combination no kernel here can address      */
  FFNK_E_ALIGN = -4,      /* pointer not 2-byte aligned                         */
  FFNK_E_WORKSPACE = -5,  /* ws_bytes smaller than ffnk_workspace_bytes()       */
  FFNK_E_OP = -6          /* unknown op id                                      */
};

/* op ids for ffnk_workspace_bytes / ffnk_tile_config */
enum {
  FFNK_OP_LINEAR_FWD = 0, /* MaskedLinear forward                (K = in, N = out)  */
  FFNK_OP_FFN_FWD = 1,    /* MaskedFFN forward                   (K = d,  N = h)    */
  FFNK_OP_LINEAR_BWD = 2, /* MaskedLinear backward               (K = in, N = out)  */
  FFNK_OP_FFN_UP = 3,     /* tile_config only: up-projection + SwiGLU stage         */
  FFNK_OP_FFN_DOWN = 4,   /* tile_config only: down-projection stage                */
  FFNK_OP_BWD_DX = 5,     /* tile_config only: dx GEMM of the backward              */
  FFNK_OP_BWD_DW = 6,     /* tile_config only: dW GEMM of the backward              */
  FFNK_OP_FFN_BWD = 7     /* workspace_bytes only: MaskedFFN backward (K = d, N = h) */
};

/* kernel families reported by ffnk_tile_config */
enum {
  FFNK_PATH_MFMA_TILED = 0,   /* LDS-staged MFMA macro-tile GEMM (large M)          */
  FFNK_PATH_STREAM = 1,       /* weight-streaming MFMA kernels (decode, small M)    */
  FFNK_PATH_GENERIC = 2       /* any-stride scalar kernel (unaligned / odd strides) */
};

/* One entry of the gfx950 tile table (replaces the reference's find_spec() lookup in
 * its A100-tuned JSON tables: ffn_kernel/utils.py:3-5, ffn_kernel/bf16_*_fwd.json). */
typedef struct ffnk_tile_config_t {
  int32_t path;        /* FFNK_PATH_*                                              */
  int32_t block_m;     /* token rows per workgroup tile                            */
  int32_t block_n;     /* output columns per workgroup tile                        */
  int32_t block_k;     /* contraction elements per LDS stage / per streamed chunk  */
  int32_t waves_m;     /* wavefront grid inside the workgroup                      */
  int32_t waves_n;
  int32_t lds_stages;  /* LDS buffers in flight                                    */
  int32_t group_m;     /* M-tiles per L2 super-group in the tile order             */
  int32_t split_k;     /* contraction splits reduced by a second kernel (1 = none) */
  int32_t direct_lds;  /* 1 = global->LDS loads bypass registers                   */
  int32_t in_place;    /* FFNK_OP_BWD_DW: 1 = the weight-gradient GEMM reads g and x
                          where they lie, 0 = routed transposes written first      */
} ffnk_tile_config_t;

FFNK_API int ffnk_version(void);

/* Text for the calling thread's last non-zero return ("" if none). Never NULL. */
FFNK_API const char* ffnk_last_error(void);

/*
 * Row partition.  Writes perm[0..M) = indices of visual rows in ascending order followed
 * by indices of text rows in ascending order (a stable partition of 0..M-1 by mask), and
 * counts[0] = number of visual rows, counts[1] = number of text rows.
 * No counterpart kernel in the reference (it routes per tile, ffn_kernel/linear.py:120-149);
 * it yields the same row -> weight assignment as the mask test there.
 */
FFNK_API int ffnk_route(const uint8_t* mask, int64_t M, int32_t* perm, int32_t* counts, void* stream);

/*
 * A row partition made earlier by ffnk_route for the same mask and M, handed to the *_routed entry points
 * below so that the operations of a layer - and a forward and its backward - share one partition instead
 * of each running its own.  perm: int32[M], counts: int32[2], both DEVICE memory that holds ffnk_route's
 * output by the time the call's kernels run (same stream, or ordered by the caller) and stays unchanged
 * until they have finished.  The struct itself is host memory, read during the call.  The reference has
 * nothing to share here: its kernels re-test the mask inside every tile of every launch
 * (ffn_kernel/linear.py:120-149, ffn_kernel/ffn.py:61-105).
 */
typedef struct ffnk_routing_t {
  const int32_t* perm;
  const int32_t* counts;
} ffnk_routing_t;

/* Bytes of scratch the op needs for these extents (0 is a valid answer).
 * Returns (size_t)-1 for an unknown op or invalid extents. */
FFNK_API size_t ffnk_workspace_bytes(int op, int64_t M, int64_t K, int64_t N);

/* Scratch of ffnk_masked_ffn_bwd / ffnk_masked_ffn_bwd_saved for one layout of the weights (element strides as
 * passed to those calls), assuming 16-byte aligned pointers.  ffnk_workspace_bytes(FFNK_OP_FFN_BWD, ...) covers every
 * layout and reserves room for copies of the weights and transposes of the intermediates that the usual layout
 * (nn.Linear.weight.T views, d and h multiples of 64) never touches - 1.6 GB of 2.7 GB at M = 8192, d = 4096,
 * h = 14336; this query leaves that out.  A call whose pointers turn out not to be aligned needs the larger size
 * and says so (FFNK_E_WORKSPACE).  No counterpart in the reference, whose MaskedFFN.backward raises
 * (ffn_kernel/ops.py:34-38).  Returns (size_t)-1 for invalid extents. */
FFNK_API size_t ffnk_workspace_bytes_ffn_bwd(int64_t M, int64_t d, int64_t h, int64_t g_stride_m, int64_t up_stride_n,
                                             int64_t down_stride_k, int64_t down_stride_n, int64_t dup_stride_k,
                                             int64_t ddown_stride_k);

/* Which tile-table entry the library uses for these extents. */
FFNK_API int ffnk_tile_config(int op, int64_t M, int64_t K, int64_t N, ffnk_tile_config_t* out);

/*
 * Tuner-only hooks (python -m ffn_kernel_amd.tune, the counterpart of the reference's find_spec scripts
 * sweeps, and the tests that run every compiled tile).  ffnk_debug_force_tile: every LDS-tiled GEMM
 * launched by this process uses tile id `tile` (0 = 256x256 / 8 waves, 1 = 256x256 / 4 waves,
 * 2 = 128x128 / 4 waves, 3 = small, 4 = 128x128 / 4 waves behind a ring of four LDS stages); -1 returns to the tile table (measured plans first, then the
 * rules); -2 uses the rules only, ignoring the measured plans (what the tuner compares against).
 * ffnk_debug_force_splits: every GEMM that can cut its contraction (single-weight routed GEMMs with
 * a workspace, weight-gradient GEMMs) uses `splits` ranges (1..16) where the shape allows it; -1
 * returns to the table.  Both are process-global atomics read at every call (ffnk_workspace_bytes
 * answers for the current setting); production callers leave them alone.  Each returns the previous
 * value.
 */
FFNK_API int ffnk_debug_force_tile(int tile);
FFNK_API int ffnk_debug_force_splits(int splits);
/* MaskedLinear backward, tuner-only like the two above: 1 = the weight-gradient GEMM reads g and x where they lie
 * (rows found through perm) wherever the operands allow it, 0 = it reads routed, padded transposes written by an
 * elementwise pass first, -1 = the plan decides.  Returns the previous value. */
FFNK_API int ffnk_debug_force_bwd_gather(int on);
/* Tuner-only as well: every routed GEMM walks its tiles in super-groups of `group_m` M-tiles (1..64) instead of the
 * tile's own (8 for the SwiGLU GEMM and the K-major kernels, 4 for the other single-weight GEMMs); 0 returns to those.
 * The counterpart of the GROUP_SIZE_M dimension of the reference's searches (find_spec/bf16_linear_fwd.py:45-53).
 * Returns the previous value. */
FFNK_API int ffnk_debug_force_group_m(int group_m);

/*
 * MaskedLinear forward — replaces _bf16_linear_forward (ffn_kernel/linear.py:418-452):
 *   y[m, :] = x[m, :] @ (mask[m] ? Wv : Wt)      for m in [0, M)
 * x: [M, K], element strides (x_stride_m, 1).  Wv, Wt: logical [K, N] with element strides
 * (w_stride_k, w_stride_n) as in the reference call (b1.stride(0), b1.stride(1),
 * linear.py:442-443); nn.Linear.weight.T gives (1, K).  y: [M, N] strides (y_stride_m, 1).
 * Accumulation is fp32; the result is rounded to bf16 once.
 */
FFNK_API int ffnk_masked_linear_fwd(const uint16_t* x, int64_t x_stride_m,
                           const uint16_t* Wv, const uint16_t* Wt,
                           int64_t w_stride_k, int64_t w_stride_n,
                           const uint8_t* mask,
                           uint16_t* y, int64_t y_stride_m,
                           int64_t M, int64_t K, int64_t N,
                           void* ws, size_t ws_bytes, void* stream);

/* ffnk_masked_linear_fwd with the row partition handed in (routing == NULL: exactly ffnk_masked_linear_fwd).
 * `mask` is still required: the weight-streaming kernels for M <= 64 and the any-stride kernels read it
 * themselves and ignore `routing`.  What it replaces: the per-tile mask test of ffn_kernel/linear.py:120-149. */
FFNK_API int ffnk_masked_linear_fwd_routed(const uint16_t* x, int64_t x_stride_m,
                                  const uint16_t* Wv, const uint16_t* Wt,
                                  int64_t w_stride_k, int64_t w_stride_n,
                                  const uint8_t* mask,
                                  uint16_t* y, int64_t y_stride_m,
                                  int64_t M, int64_t K, int64_t N,
                                  void* ws, size_t ws_bytes, void* stream, const ffnk_routing_t* routing);

/*
 * MaskedFFN forward — replaces _bf16_ffn_forward followed by _bf16_linear_forward
 * (ffn_kernel/ops.py:30-32, ffn_kernel/ffn.py:527-560):
 *   visual row:  out = (silu(x W1) * (x W3)) W2        text row: same with U1, U3, U2
 * W1, W3, U1, U3: logical [d, h] with strides (up_stride_k, up_stride_n) shared by all four
 * (ffn.py:551); W2, U2: logical [h, d] with strides (down_stride_k, down_stride_n).
 * The [M, h] intermediate is rounded to bf16 once (as the reference stores it, ffn.py:113).
 * Picks the macro-tile path or the weight-streaming path from M.
 */
FFNK_API int ffnk_masked_ffn_fwd(const uint16_t* x, int64_t x_stride_m,
                        const uint16_t* W1, const uint16_t* W3,
                        const uint16_t* U1, const uint16_t* U3,
                        int64_t up_stride_k, int64_t up_stride_n,
                        const uint16_t* W2, const uint16_t* U2,
                        int64_t down_stride_k, int64_t down_stride_n,
                        const uint8_t* mask,
                        uint16_t* out, int64_t out_stride_m,
                        int64_t M, int64_t d, int64_t h,
                        void* ws, size_t ws_bytes, void* stream);

/*
 * Same as ffnk_masked_ffn_fwd, with stage timing for profilers and benchmarks: `events` is
 * NULL or a HOST array of three hipEvent_t handles (each may be NULL) that are recorded on
 * `stream` after the row partition, after the up-projection + SwiGLU stage and after the
 * down-projection stage.  The caller creates, reads and destroys the events.
 * No counterpart in the reference (it times whole module calls with an external wall-clock
 * profiler, test_ffn.py:21-29).
 */
FFNK_API int ffnk_masked_ffn_fwd_ev(const uint16_t* x, int64_t x_stride_m,
                           const uint16_t* W1, const uint16_t* W3,
                           const uint16_t* U1, const uint16_t* U3,
                           int64_t up_stride_k, int64_t up_stride_n,
                           const uint16_t* W2, const uint16_t* U2,
                           int64_t down_stride_k, int64_t down_stride_n,
                           const uint8_t* mask,
                           uint16_t* out, int64_t out_stride_m,
                           int64_t M, int64_t d, int64_t h,
                           void* ws, size_t ws_bytes, void* stream, void* const* events);

/*
 * ffnk_masked_ffn_fwd without a workspace argument and without any allocation: for callers that
 * cannot allocate device memory around the call (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Scratch is a static
 * device array of FFNK_STATIC_SCRATCH_BYTES inside the library (each GPU the library runs on holds
 * its own copy until the process ends); shapes whose ffnk_workspace_bytes(FFNK_OP_FFN_FWD, M, d, h)
 * exceeds that return FFNK_E_WORKSPACE (at d = 4096, h = 14336 every M up to 256 fits).  Same
 * kernels and results as ffnk_masked_ffn_fwd.  All calls on one GPU share that GPU's array:
 * calls that overlap on one GPU (different streams or threads) race; calls on one stream are
 * ordered and safe.  The first call on each GPU looks the array's address up (no allocation); make
 * that call outside stream capture.
 */
#define FFNK_STATIC_SCRATCH_BYTES (32u << 20)
FFNK_API int ffnk_masked_ffn_fwd_static(const uint16_t* x, int64_t x_stride_m,
                               const uint16_t* W1, const uint16_t* W3,
                               const uint16_t* U1, const uint16_t* U3,
                               int64_t up_stride_k, int64_t up_stride_n,
                               const uint16_t* W2, const uint16_t* U2,
                               int64_t down_stride_k, int64_t down_stride_n,
                               const uint8_t* mask,
                               uint16_t* out, int64_t out_stride_m,
                               int64_t M, int64_t d, int64_t h, void* stream);

/*
 * MaskedLinear backward — replaces _bf16_linear_backward (ffn_kernel/linear.py:455-496):
 *   dx[m, :]  = g[m, :] @ (mask[m] ? Wv : Wt)^T
 *   dWv       = x[visual rows]^T @ g[visual rows]       (exact zeros if there are none)
 *   dWt       = x[text rows]^T   @ g[text rows]
 * g: [M, N] strides (g_stride_m, 1); x: [M, K]; Wv/Wt as in the forward; dx: [M, K];
 * dWv, dWt: logical [K, N] with strides (dw_stride_k, dw_stride_n) (the reference
 * allocates them with empty_like(b1), linear.py:475).  Deterministic: no atomics.
 */
FFNK_API int ffnk_masked_linear_bwd(const uint16_t* g, int64_t g_stride_m,
                           const uint16_t* x, int64_t x_stride_m,
                           const uint16_t* Wv, const uint16_t* Wt,
                           int64_t w_stride_k, int64_t w_stride_n,
                           const uint8_t* mask,
                           uint16_t* dx, int64_t dx_stride_m,
                           uint16_t* dWv, uint16_t* dWt,
                           int64_t dw_stride_k, int64_t dw_stride_n,
                           int64_t M, int64_t K, int64_t N,
                           void* ws, size_t ws_bytes, void* stream);

/* ffnk_masked_linear_bwd with the row partition handed in (routing == NULL: exactly ffnk_masked_linear_bwd);
 * a backward can reuse the partition its forward ran with.  Replaces the mask tests of
 * ffn_kernel/linear.py:288-291, 299-313, 398-403. */
FFNK_API int ffnk_masked_linear_bwd_routed(const uint16_t* g, int64_t g_stride_m,
                                  const uint16_t* x, int64_t x_stride_m,
                                  const uint16_t* Wv, const uint16_t* Wt,
                                  int64_t w_stride_k, int64_t w_stride_n,
                                  const uint8_t* mask,
                                  uint16_t* dx, int64_t dx_stride_m,
                                  uint16_t* dWv, uint16_t* dWt,
                                  int64_t dw_stride_k, int64_t dw_stride_n,
                                  int64_t M, int64_t K, int64_t N,
                                  void* ws, size_t ws_bytes, void* stream, const ffnk_routing_t* routing);

/*
 * MaskedFFN backward.  The reference declares it but raises NotImplementedError
 * (ffn_kernel/ops.py:34-38); its README (README.md:159-172) sketches the decomposition used
 * here: an elementwise SwiGLU-gradient pass between routed GEMMs.  For row m with
 * (A1, A2, A3) = mask[m] ? (W1, W2, W3) : (U1, U2, U3), t1 = x[m] @ A1, t3 = x[m] @ A3:
 *   dh  = g[m] @ A2^T
 *   dt1 = dh * t3 * silu'(t1),  dt3 = dh * silu(t1),  silu'(t) = s + t s (1 - s), s = sigmoid(t)
 *   dx[m] = dt1 @ A1^T + dt3 @ A3^T
 *   dA1 = sum over the group's rows of x[m]^T dt1,  dA3 likewise with dt3,
 *   dA2 = sum of (silu(t1) * t3)^T g[m]            (exact zeros for an empty group)
 * g: [M, d]; x: [M, d]; weights and strides as in ffnk_masked_ffn_fwd, with the up-projection
 * weights K-contiguous (up_stride_k == 1: the nn.Linear.weight.T views the reference passes);
 * dW1/dW3/dU1/dU3: logical [d, h] with strides (dup_stride_k, dup_stride_n); dW2/dU2: logical
 * [h, d] with strides (ddown_stride_k, ddown_stride_n).  t1, t3, dh, dt1, dt3 and the
 * intermediate are held in bf16 between the GEMMs (the forward does the same for the
 * intermediate); accumulation is fp32; deterministic, no atomics.  With d and h multiples of 64 and
 * the weight views the reference passes (or a down weight whose d axis is contiguous) every GEMM reads
 * the weights in place; other extents and strides are first copied into the workspace.
 * Workspace: ffnk_workspace_bytes(FFNK_OP_FFN_BWD, M, d, h).  Layouts outside the above
 * (d or h not a multiple of 8, unaligned rows, up_stride_k != 1) return FFNK_E_STRIDE.
 */
FFNK_API int ffnk_masked_ffn_bwd(const uint16_t* g, int64_t g_stride_m,
                        const uint16_t* x, int64_t x_stride_m,
                        const uint16_t* W1, const uint16_t* W3,
                        const uint16_t* U1, const uint16_t* U3,
                        int64_t up_stride_k, int64_t up_stride_n,
                        const uint16_t* W2, const uint16_t* U2,
                        int64_t down_stride_k, int64_t down_stride_n,
                        const uint8_t* mask,
                        uint16_t* dx, int64_t dx_stride_m,
                        uint16_t* dW1, uint16_t* dW3, uint16_t* dU1, uint16_t* dU3,
                        int64_t dup_stride_k, int64_t dup_stride_n,
                        uint16_t* dW2, uint16_t* dU2,
                        int64_t ddown_stride_k, int64_t ddown_stride_n,
                        int64_t M, int64_t d, int64_t h,
                        void* ws, size_t ws_bytes, void* stream);

/*
 * Training forward / backward pair that keeps the pre-activations instead of recomputing them.
 * No counterpart in the live reference (its forward keeps nothing; the dead work-in-progress forward
 * of ffn_kernel/ffn.py:116-221 stores t1 and t3 for the same purpose).
 *
 * ffnk_masked_ffn_fwd_save is ffnk_masked_ffn_fwd and additionally writes pre: [M, 2h] bf16, row
 * stride pre_stride_m (>= 2h, multiple of 8, rows 16-byte aligned), rows in ROUTED order (visual
 * rows first, each group ascending), columns [0, h) = t1 = x A1, [h, 2h) = t3 = x A3, rounded to
 * bf16 from the fp32 accumulators - what the recomputing backward would produce.  Only the LDS-tiled
 * path can do it: ffnk_masked_ffn_can_save(M, d, h) says whether this shape qualifies (M > 64, d and h
 * multiples of 8); the fast layout of ffnk_masked_ffn_fwd is required on top.  FFNK_E_STRIDE otherwise.
 *
 * ffnk_masked_ffn_bwd_saved is ffnk_masked_ffn_bwd with those pre-activations (same mask), read-only:
 * it skips the two recompute GEMMs (a quarter of the backward's GEMM work).
 */
FFNK_API int ffnk_masked_ffn_can_save(int64_t M, int64_t d, int64_t h);

FFNK_API int ffnk_masked_ffn_fwd_save(const uint16_t* x, int64_t x_stride_m,
                             const uint16_t* W1, const uint16_t* W3,
                             const uint16_t* U1, const uint16_t* U3,
                             int64_t up_stride_k, int64_t up_stride_n,
                             const uint16_t* W2, const uint16_t* U2,
                             int64_t down_stride_k, int64_t down_stride_n,
                             const uint8_t* mask,
                             uint16_t* out, int64_t out_stride_m,
                             uint16_t* pre, int64_t pre_stride_m,
                             int64_t M, int64_t d, int64_t h,
                             void* ws, size_t ws_bytes, void* stream);

FFNK_API int ffnk_masked_ffn_bwd_saved(const uint16_t* g, int64_t g_stride_m,
                              const uint16_t* x, int64_t x_stride_m,
                              const uint16_t* W1, const uint16_t* W3,
                              const uint16_t* U1, const uint16_t* U3,
                              int64_t up_stride_k, int64_t up_stride_n,
                              const uint16_t* W2, const uint16_t* U2,
                              int64_t down_stride_k, int64_t down_stride_n,
                              const uint8_t* mask,
                              const uint16_t* pre, int64_t pre_stride_m,
                              uint16_t* dx, int64_t dx_stride_m,
                              uint16_t* dW1, uint16_t* dW3, uint16_t* dU1, uint16_t* dU3,
                              int64_t dup_stride_k, int64_t dup_stride_n,
                              uint16_t* dW2, uint16_t* dU2,
                              int64_t ddown_stride_k, int64_t ddown_stride_n,
                              int64_t M, int64_t d, int64_t h,
                              void* ws, size_t ws_bytes, void* stream);

/*
 * The MaskedFFN forward and backward with the row partition handed in (see ffnk_routing_t; routing == NULL:
 * a route launch at the head of the call, as in the plain entry points).  `pre` is optional in both:
 * forward: NULL = ffnk_masked_ffn_fwd, else ffnk_masked_ffn_fwd_save; backward: NULL = ffnk_masked_ffn_bwd
 * (recompute), else ffnk_masked_ffn_bwd_saved.  Replaces the per-tile mask tests of ffn_kernel/ffn.py:61-105
 * and ffn_kernel/linear.py:120-149.
 */
FFNK_API int ffnk_masked_ffn_fwd_routed(const uint16_t* x, int64_t x_stride_m,
                               const uint16_t* W1, const uint16_t* W3,
                               const uint16_t* U1, const uint16_t* U3,
                               int64_t up_stride_k, int64_t up_stride_n,
                               const uint16_t* W2, const uint16_t* U2,
                               int64_t down_stride_k, int64_t down_stride_n,
                               const uint8_t* mask,
                               uint16_t* out, int64_t out_stride_m,
                               uint16_t* pre, int64_t pre_stride_m,
                               int64_t M, int64_t d, int64_t h,
                               void* ws, size_t ws_bytes, void* stream, const ffnk_routing_t* routing);

FFNK_API int ffnk_masked_ffn_bwd_routed(const uint16_t* g, int64_t g_stride_m,
                               const uint16_t* x, int64_t x_stride_m,
                               const uint16_t* W1, const uint16_t* W3,
                               const uint16_t* U1, const uint16_t* U3,
                               int64_t up_stride_k, int64_t up_stride_n,
                               const uint16_t* W2, const uint16_t* U2,
                               int64_t down_stride_k, int64_t down_stride_n,
                               const uint8_t* mask,
                               const uint16_t* pre, int64_t pre_stride_m,
                               uint16_t* dx, int64_t dx_stride_m,
                               uint16_t* dW1, uint16_t* dW3, uint16_t* dU1, uint16_t* dU3,
                               int64_t dup_stride_k, int64_t dup_stride_n,
                               uint16_t* dW2, uint16_t* dU2,
                               int64_t ddown_stride_k, int64_t ddown_stride_n,
                               int64_t M, int64_t d, int64_t h,
                               void* ws, size_t ws_bytes, void* stream, const ffnk_routing_t* routing);

#ifdef __cplusplus
}
#endif
#endif /* FFNK_H */
