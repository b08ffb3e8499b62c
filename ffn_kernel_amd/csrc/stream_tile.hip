// Weight-streaming MFMA kernels for decode-shaped MaskedFFN calls with 9 <= M <= 64 token rows.
//
// The op is bound by reading each present modality's weights once, and the MFMA operand layout
// (lane = row, 16 bytes of K) would make every global load touch 16 rows x 64 bytes.  So the loads
// are decoupled from that layout:
//   * a wavefront owns two 16-row weight tiles (gate + up rows of the same outputs, or two row
//     tiles of the down projection) and streams them in 128-element K chunks with loads that cover
//     4 rows x 256 contiguous bytes each, kept three or four chunks (24-32 KB) ahead in registers;
//   * each chunk is transposed through a wave-private, XOR-swizzled LDS tile (ds_write_b128 in load
//     layout, ds_read_b128 in MFMA fragment layout, both bank-conflict free; one wavefront's LDS
//     operations execute in order, so the tile needs neither double buffering nor waits);
//   * the token rows of the chunk (x, or the SwiGLU intermediate) are staged once per workgroup in an
//     LDS slab that its wavefronts share.  For up to two m-tiles the slab is double-buffered and goes
//     through registers, fetched at the same distance as the weights so that the in-order load
//     counter never forces a weight load to complete early.  For three and four m-tiles the staging
//     registers would not fit beside the weight ring, so the slab is a ring of buffers filled by
//     direct global -> LDS loads (swizzled on the global side) and read with ds_read_b128 written
//     as inline assembly: a compiler-visible LDS read of an array that direct loads write makes the
//     compiler drain every load in flight first;
//   * one raw s_barrier per chunk hands the slab over; it does not drain the loads in flight;
//   * the K loop is split into a branch-free steady part and a guarded tail: a load behind a uniform
//     branch makes the compiler's load-counter waits conservative for the whole loop.
// The up projection covers all of K in one workgroup (SwiGLU epilogue, routed-order H); the down
// projection splits K across workgroups into fp32 partials that stream_reduce_kernel sums.
// Same role as the reference's small-M launches of its GEMM tiles (ffn_kernel/ffn.py:527-560,
// ffn_kernel/linear.py:418-452).
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"

namespace ffnk {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kTK = 128;    // K elements per chunk (16 pieces of 16 bytes per row)
// Shape per number of 16-row m-tiles the call can have (ceil(M / 16)): wavefronts per workgroup
// (sharing one token-row slab; fewer wavefronts = less barrier coupling and more workgroups, but
// every thread then stages more of the slab) and chunks in flight per wavefront (register budget).
// dma: the token-row slab is filled by direct global -> LDS loads (no staging registers, which is
// what lets the 3- and 4-m-tile shapes run two-wavefront workgroups) instead of through registers.
struct TileShapeEntry { int waves, depth, dma; };
// One table per projection.  Four wavefronts per up-projection workgroup for three and four m-tiles (half the
// slab traffic per weight byte, 80 KB of LDS, one round of workgroups instead of 1.75 with both modalities at
// M = 64) measured 1-2 % slower than two at M = 48 and 64 and the same at M = 32; the tables stay equal.
constexpr TileShapeEntry kTileShapesUp[4] = {{2, 4, 0}, {2, 3, 0}, {2, 3, 1}, {2, 3, 1}};
constexpr TileShapeEntry kTileShapesDown[4] = {{2, 4, 0}, {2, 3, 0}, {2, 3, 1}, {2, 3, 1}};
constexpr const TileShapeEntry& tile_shape(int ntm_max, bool dual) { return dual ? kTileShapesUp[ntm_max - 1] : kTileShapesDown[ntm_max - 1]; }
constexpr int kTMaxM = 64;

struct TileJob {
  int grp, split, p0, mg, n0, c0, nc;  // n0: first weight row of the workgroup; c0 / nc: chunk range
};

// xs: [2][NTM * 16 token rows][16 pieces] 16-byte slots; wst: this wavefront's [2 tiles][16 rows][16 pieces].
template <int NTM, bool DUAL, int kTWaves, int kTD, bool XDMA>
__device__ __forceinline__ void tile_rows(const StreamArgs& a, const TileJob& t, const int* s_perm, u32x4_t* xs,
                                          u32x4_t* wst) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, lq = lane >> 4;
  const int64_t kbase = (int64_t)t.c0 * kTK;

  // weight tiles of this wavefront
  int rbase[2];
  const uint16_t* wp[2];
  if (DUAL) {
    rbase[0] = rbase[1] = t.n0 + wave * 16;
    wp[0] = a.W0[t.grp];
    wp[1] = a.W1[t.grp];
  } else {
    rbase[0] = t.n0 + wave * 32;
    rbase[1] = rbase[0] + 16;
    wp[0] = wp[1] = a.W0[t.grp];
  }
#pragma unroll
  for (int w = 0; w < 2; ++w) wp[w] += (int64_t)(rbase[w] + lq) * a.ldw + kbase + lrow * 8;  // load u adds 4 u rows
  const int64_t w_step = 4 * a.ldw;

  // Token-row slab, register path: two buffers of [NTM * 16 rows][16 pieces].  Each thread stages
  // piece (tid & 15) of slab rows p * XR + (tid >> 4); slot = row * 16 + (piece ^ row & 15).
  constexpr int XR = kTWaves * 4;                  // slab rows one pass of the workgroup covers
  constexpr int XP = XDMA ? 1 : NTM * 16 / XR;     // passes (register path only)
  const uint16_t* xp[XP];
  if (!XDMA) {
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int j = p * XR + (tid >> 4);
      const int pos = t.p0 + min(j, t.mg - 1);  // surplus slab rows repeat the last row; dropped in the epilogue
      const int64_t src = a.gather_x ? (int64_t)s_perm[pos] : (int64_t)pos;
      xp[p] = a.X + src * a.ldx + kbase + (tid & 15) * 8;
    }
  }
  // Token-row slab, direct path: kTD buffers filled by global -> LDS loads.  One load instruction of a
  // wavefront fills four consecutive slab rows: lane l writes slot l of that 1 KB, i.e. row
  // 4 g + (l >> 4), position l & 15, which must hold piece (position ^ row & 15) of the row - the
  // swizzle is applied on the global side.
  constexpr int XG = XDMA ? NTM * 4 / kTWaves : 1;  // 4-row groups per wavefront per chunk
  static_assert(!XDMA || XG * kTWaves == NTM * 4, "slab rows must divide among the wavefronts");
  uint32_t xoff[XG];
  if (XDMA) {
#pragma unroll
    for (int i = 0; i < XG; ++i) {
      const int j = 4 * (wave + kTWaves * i) + lq;
      const int pos = t.p0 + min(j, t.mg - 1);
      const int64_t src = a.gather_x ? (int64_t)s_perm[pos] : (int64_t)pos;
      xoff[i] = (uint32_t)((src * a.ldx + kbase + ((lrow ^ (j & 15)) * 8)) * 2);  // bytes; host checks M * ldx < 2^30
    }
  }

  // Workgroups walk their chunk range from different starting chunks (wrapping around): weight rows
  // are a power-of-two number of bytes apart, so workgroups sitting at the same K offset would all
  // pull from the same few HBM channels.
  const int nc = t.nc;
  const int rot = (int)((blockIdx.x * 11u) % (unsigned)nc);
  auto phys = [&](int c) { const int pc = c + rot; return (pc >= nc ? pc - nc : pc) * kTK; };
  u32x4_t wr[kTD][2][4];
  auto loadw = [&](int s, int c) {
    const int64_t ko = phys(c);
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int u = 0; u < 4; ++u)
        wr[s][w][u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(wp[w] + u * w_step + ko));
  };
  u32x4_t xr[XDMA ? 1 : kTD][XP];
  auto loadx = [&](int s, int c) {
    const int64_t ko = phys(c);
#pragma unroll
    for (int p = 0; p < XP; ++p) xr[s][p] = *reinterpret_cast<const u32x4_t*>(xp[p] + ko);
  };
  auto stage_x = [&](int s, int c) {
    u32x4_t* dst = xs + (c & 1) * (NTM * 256);
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int j = p * XR + (tid >> 4);
      dst[j * 16 + ((tid & 15) ^ (j & 15))] = xr[s][p];
    }
  };
  auto lds_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wavefront's LDS writes have landed; loads stay in flight
    __builtin_amdgcn_s_barrier();
  };
  // ---- direct path ----
#if defined(__HIP_DEVICE_COMPILE__)
  const __amdgpu_buffer_rsrc_t xrs = __builtin_amdgcn_make_buffer_rsrc((void*)a.X, 0, 0xffffffff, 0x00020000);
#endif
  auto dma_x = [&](int slot, int c) {
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" ::: "memory");  // the explicit waits below count loads: keep this one where it is written
    u32x4_t* slab = xs + slot * (NTM * 256);
    const int ko = phys(c) * 2;
#pragma unroll
    for (int i = 0; i < XG; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xrs, (__attribute__((address_space(3))) void*)(slab + (wave + kTWaves * i) * 64),
                                               16, xoff[i], ko, 0, 0);
    asm volatile("" ::: "memory");
#endif
  };
  // Loads a wavefront has issued after the slab loads of chunk c + 1 by the end of chunk c's iteration:
  // weights of c+2 .. c+kTD ... (kTD - 1) x 8, slab loads of c+2 .. c+kTD-1 ... (kTD - 2) x XG.
  constexpr int kAfterX = (kTD - 1) * 8 + (kTD - 2) * XG;
  static_assert(kAfterX < 64, "vmcnt is a 6-bit counter");
  constexpr int kWaitSteady = (kAfterX & 15) | (7 << 4) | ((kAfterX >> 4) << 14);  // vmcnt(kAfterX) lgkmcnt(0)
  constexpr int kWaitAll = 7 << 4;                                                 // vmcnt(0) lgkmcnt(0)
  // Make the next chunk's slab visible to the workgroup: own slab loads landed, then barrier.
  auto slab_barrier = [&](bool steady) {
    asm volatile("" ::: "memory");
    if (steady) __builtin_amdgcn_s_waitcnt(kWaitSteady);
    else __builtin_amdgcn_s_waitcnt(kWaitAll);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  // The slab is read with ds_read_b128 written as inline assembly: a compiler-visible LDS read of an
  // array that direct loads write makes the compiler drain every load in flight first.  The waits for
  // these reads are therefore explicit too (slab_wait).
  const uint32_t xs_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)xs;
  uint32_t xaddr[4];  // this lane's slab address per k-step: row lrow, piece (4 s + lq) ^ lrow
#pragma unroll
  for (int s = 0; s < 4; ++s) xaddr[s] = xs_addr + (uint32_t)(lrow * 16 + ((s * 4 + lq) ^ lrow)) * 16;

  f32x4_t acc[2][NTM];
#pragma unroll
  for (int w = 0; w < 2; ++w)
#pragma unroll
    for (int m = 0; m < NTM; ++m) acc[w][m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  // Token rows this lane stores in the epilogue: s_perm lives in the staging tiles' memory, which the first chunk
  // overwrites (every wavefront passes the prologue's barrier between these reads and that write).
  int out_row[NTM];
#pragma unroll
  for (int m = 0; m < NTM; ++m) out_row[m] = (!DUAL && m * 16 + lrow < t.mg) ? s_perm[t.p0 + m * 16 + lrow] : 0;

  // One chunk.  STEADY: every chunk whose loads this iteration would issue exists, so the loads are
  // unconditional and the compiler's load-counter waits are exact; otherwise the loads are guarded,
  // which makes the compiler wait for more than it needs - only the last 2 kTD chunks of a workgroup
  // run that way.  Register path: loads go out as w(c + kTD), x(c + 1 + kTD).  Direct path: x(c + kTD - 1)
  // into the slab chunk c - 1 used, then w(c + kTD).  Either way the token rows of a chunk are fetched
  // right after its weights, so waiting for them never forces younger weight loads to land.
  auto chunk = [&](int u3, int c, auto steady_tag) {
    constexpr bool STEADY = decltype(steady_tag)::value;
    if (XDMA) {
      if (STEADY || c + kTD - 1 < nc) dma_x((u3 + kTD - 1) % kTD, c + kTD - 1);
    }
    // weights of chunk c: registers -> swizzled staging tile
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int row = 4 * u + lq;
        wst[w * 256 + row * 16 + (lrow ^ row)] = wr[u3][w][u];
      }
    if (STEADY || c + kTD < nc) loadw(u3, c + kTD);
    if (!XDMA) {
      // token rows of chunk c + 1 -> the other slab buffer (its last readers passed the previous barrier)
      if (STEADY || c + 1 < nc) {
        stage_x((u3 + 1) % kTD, c + 1);
        if (STEADY || c + 1 + kTD < nc) loadx((u3 + 1) % kTD, c + 1 + kTD);
      }
    }
    const u32x4_t* xb = xs + (c & 1) * (NTM * 256);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int piece = (s * 4 + lq) ^ lrow;
      const bf16x8_t wf0 = __builtin_bit_cast(bf16x8_t, wst[lrow * 16 + piece]);
      const bf16x8_t wf1 = __builtin_bit_cast(bf16x8_t, wst[256 + lrow * 16 + piece]);
      u32x4_t xv[NTM];
      if (XDMA) {
#pragma unroll
        for (int m = 0; m < NTM; ++m)
          asm volatile("ds_read_b128 %0, %1 offset:%2"
                       : "=v"(xv[m])
                       : "v"(xaddr[s]), "n"((u3 * NTM * 256 + m * 256) * 16)
                       : "memory");
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int m = 0; m < NTM; ++m) asm volatile("" : "+v"(xv[m]));  // uses below stay after the wait
      } else {
#pragma unroll
        for (int m = 0; m < NTM; ++m) xv[m] = xb[(m * 16 + lrow) * 16 + piece];
      }
#pragma unroll
      for (int m = 0; m < NTM; ++m) {
        const bf16x8_t xf = __builtin_bit_cast(bf16x8_t, xv[m]);
        acc[0][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf0, xf, acc[0][m], 0, 0, 0);
        acc[1][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf1, xf, acc[1][m], 0, 0, 0);
      }
    }
    // the next chunk's slab must be complete, and this chunk's reads done, before anyone moves on
    // (executed the same number of times by every wavefront: nc is uniform)
    if (XDMA) slab_barrier(STEADY);
    else lds_barrier();
  };

  // prologue (nc >= 2 kTD, checked on the host)
  if (XDMA) {
    // w(0) x(0) w(1) x(1) ... w(kTD - 1)
#pragma unroll
    for (int s = 0; s < kTD; ++s) {
      loadw(s, s);
      if (s < kTD - 1) dma_x(s, s);
    }
    slab_barrier(true);
  } else {
    // weights of chunks 0 .. kTD-1, token rows of chunks 0 .. kTD; chunk 0's go straight to the slab
    loadx(0, 0);
#pragma unroll
    for (int s = 0; s < kTD; ++s) {
      loadw(s, s);
      if (s >= 1) loadx(s, s);
    }
    stage_x(0, 0);
    loadx(0, kTD);
    lds_barrier();
  }

  int c0 = 0;
  for (; c0 + 2 * kTD < nc; c0 += kTD) {
#pragma unroll
    for (int u3 = 0; u3 < kTD; ++u3) chunk(u3, c0 + u3, std::true_type{});
  }
  for (; c0 < nc; c0 += kTD) {
#pragma unroll
    for (int u3 = 0; u3 < kTD; ++u3) {
      if (c0 + u3 < nc) chunk(u3, c0 + u3, std::false_type{});  // uniform over the workgroup
    }
  }

  // acc[w][m][v]: weight row rbase[w] + 4 * lq + v, token row m * 16 + lrow of the group.
#pragma unroll
  for (int m = 0; m < NTM; ++m) {
    const int row = m * 16 + lrow;
    if (row >= t.mg) continue;
    if (DUAL) {
      const f32x4_t g = acc[0][m], u = acc[1][m];
      uint2 v2;
      v2.x = pack2bf(swiglu(g[0], u[0]), swiglu(g[1], u[1]));
      v2.y = pack2bf(swiglu(g[2], u[2]), swiglu(g[3], u[3]));
      *reinterpret_cast<uint2*>(a.H + (int64_t)(t.p0 + row) * a.ldh + rbase[0] + 4 * lq) = v2;
    } else {
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const f32x4_t o = acc[w][m];
        const int n_out = rbase[w] + 4 * lq;
        if (a.P != nullptr) {
          *reinterpret_cast<float4*>(a.P + ((int64_t)t.split * a.M + (t.p0 + row)) * a.Nrows + n_out) =
              make_float4(o[0], o[1], o[2], o[3]);
        } else {
          uint16_t* dst = a.out + (int64_t)out_row[m] * a.ldo + n_out;
          if ((reinterpret_cast<uintptr_t>(dst) & 7) == 0) {
            uint2 v2;
            v2.x = pack2bf(o[0], o[1]);
            v2.y = pack2bf(o[2], o[3]);
            *reinterpret_cast<uint2*>(dst) = v2;
          } else {
            dst[0] = f2bf(o[0]); dst[1] = f2bf(o[1]); dst[2] = f2bf(o[2]); dst[3] = f2bf(o[3]);
          }
        }
      }
    }
  }
}

__device__ __forceinline__ int route64(const uint8_t* mask, int M, int* s_perm, int* s_nvis) {
  if (threadIdx.x < kWave) {
    const int l = threadIdx.x;
    const bool valid = l < M;
    const bool vis = valid && mask[l] != 0;
    const unsigned long long vm = __ballot(vis);
    const unsigned long long am = __ballot(valid);
    const unsigned long long lt = (l == 0) ? 0ull : (~0ull >> (64 - l));
    const int nv = __popcll(vm);
    if (valid) s_perm[vis ? __popcll(vm & lt) : nv + __popcll(~vm & am & lt)] = l;
    if (l == 0) *s_nvis = nv;
  }
  __syncthreads();
  return *s_nvis;
}

// grid.x = 2 groups x splits x row blocks (visual workgroups first); 256 threads.
template <int NTM_MAX, bool DUAL, int kTWaves, int kTD, bool XDMA>
__global__ __launch_bounds__(kTWaves * kWave, 2) void stream_tile_kernel(const StreamArgs a) {
  __shared__ u32x4_t xs[(XDMA ? kTD : 2) * NTM_MAX * 256];
  __shared__ u32x4_t wst_all[kTWaves * 512];
  // The routing table shares the staging tiles' memory (it is read before the first chunk is staged): with four
  // wavefronts and a ring of three four-m-tile slabs the arrays above are exactly 80 KB, two workgroups per CU.
  int* s_perm = reinterpret_cast<int*>(wst_all);
  int* s_nvis_p = s_perm + kTMaxM;
  const int n_vis = route64(a.mask, a.M, s_perm, s_nvis_p);
  constexpr int ROWS = DUAL ? 16 * kTWaves : 32 * kTWaves;
  const int row_blocks = a.Nrows / ROWS;
  const int per_grp = row_blocks * a.splits;
  TileJob t;
  t.grp = blockIdx.x / per_grp;
  const int rem = blockIdx.x % per_grp;
  t.split = rem / row_blocks;
  t.p0 = t.grp == 0 ? 0 : n_vis;
  t.mg = t.grp == 0 ? n_vis : a.M - n_vis;
  if (t.mg == 0) return;  // modality absent: its weights are never read (uniform over the workgroup)
  t.n0 = (rem % row_blocks) * ROWS;
  const int n_chunks = a.K / kTK;
  const int cps = cdiv(n_chunks, a.splits);
  t.c0 = min(t.split * cps, n_chunks);
  t.nc = min(t.c0 + cps, n_chunks) - t.c0;
  u32x4_t* wst = wst_all + (threadIdx.x >> 6) * 512;
  const int ntm = cdiv(t.mg, 16);
  if (NTM_MAX >= 4 && ntm >= 4) tile_rows<(NTM_MAX >= 4 ? 4 : 1), DUAL, kTWaves, kTD, XDMA>(a, t, s_perm, xs, wst);
  else if (NTM_MAX >= 3 && ntm == 3) tile_rows<(NTM_MAX >= 3 ? 3 : 1), DUAL, kTWaves, kTD, XDMA>(a, t, s_perm, xs, wst);
  else if (NTM_MAX >= 2 && ntm == 2) tile_rows<(NTM_MAX >= 2 ? 2 : 1), DUAL, kTWaves, kTD, XDMA>(a, t, s_perm, xs, wst);
  else tile_rows<1, DUAL, kTWaves, kTD, XDMA>(a, t, s_perm, xs, wst);
}

static const TileShapeEntry& shape_for(int M, bool dual) { return tile_shape(cdiv(M < 1 ? 1 : M > kTMaxM ? kTMaxM : M, 16), dual); }

int stream_tile_rows_per_block(int M, bool dual) { return (dual ? 16 : 32) * shape_for(M, dual).waves; }
int stream_tile_direct(int M, bool dual) { return shape_for(M, dual).dma; }
int stream_tile_depth(int M, bool dual) { return shape_for(M, dual).depth; }

constexpr int kTMinChunks = 8;  // >= 2 x the deepest ring: lets the kernels run an unconditional prologue

bool stream_tile_ok(int M, int d, int h) {
  return M >= 1 && M <= kTMaxM && d % kTK == 0 && h % kTK == 0 && d / kTK >= kTMinChunks && h / kTK >= kTMinChunks &&
         h % stream_tile_rows_per_block(M, true) == 0 && d % stream_tile_rows_per_block(M, false) == 0;
}

// A single-weight projection (down projection, linear layer) of Nrows outputs over K on these kernels.
bool stream_tile_down_ok(int M, int Nrows, int K) {
  return M >= 1 && M <= kTMaxM && K % kTK == 0 && K / kTK >= kTMinChunks && Nrows > 0 &&
         Nrows % stream_tile_rows_per_block(M, false) == 0;
}

// K split of the down projection: about one workgroup per CU and modality, at least eight chunks
// per workgroup, every split non-empty.
int stream_tile_down_splits(int M, int d, int h) {
  const int row_blocks = d / stream_tile_rows_per_block(M, false);
  const int n_chunks = h / kTK;
  int s = cdiv(256, row_blocks);
  if (s > n_chunks / kTMinChunks) s = n_chunks / kTMinChunks;
  if (s < 1) s = 1;
  // every split must keep at least kTMinChunks chunks (the last one gets the remainder)
  while (s > 1 && n_chunks - cdiv(n_chunks, s) * (s - 1) < kTMinChunks) --s;
  return s;
}

template <int NTM_MAX, bool DUAL>
static void launch_tile_n(const StreamArgs& a, hipStream_t stream) {
  constexpr int W = tile_shape(NTM_MAX, DUAL).waves, D = tile_shape(NTM_MAX, DUAL).depth;
  constexpr bool X = tile_shape(NTM_MAX, DUAL).dma != 0;
  const int blocks = 2 * (a.Nrows / ((DUAL ? 16 : 32) * W)) * a.splits;
  hipLaunchKernelGGL((stream_tile_kernel<NTM_MAX, DUAL, W, D, X>), dim3(blocks), dim3(W * kWave), 0, stream, a);
}

template <bool DUAL>
static hipError_t launch_tile(const StreamArgs& a, hipStream_t stream) {
  if (a.M < 1 || a.M > kTMaxM || a.K % kTK != 0 || a.splits < 1 || a.Nrows % stream_tile_rows_per_block(a.M, DUAL) != 0 ||
      a.ldw % 8 != 0 || a.ldx % 8 != 0)
    return hipErrorInvalidValue;
  const int n_chunks = a.K / kTK;
  if (n_chunks - cdiv(n_chunks, a.splits) * (a.splits - 1) < kTMinChunks) return hipErrorInvalidValue;  // a short split
  if ((int64_t)a.M * a.ldx >= (1ll << 30)) return hipErrorInvalidValue;  // 32-bit byte offsets into the token rows
  if (DUAL && (a.splits != 1 || a.H == nullptr)) return hipErrorInvalidValue;
  if (!DUAL && a.P == nullptr && (a.splits != 1 || a.out == nullptr)) return hipErrorInvalidValue;
  switch (cdiv(a.M, 16)) {
    case 1: launch_tile_n<1, DUAL>(a, stream); break;
    case 2: launch_tile_n<2, DUAL>(a, stream); break;
    case 3: launch_tile_n<3, DUAL>(a, stream); break;
    default: launch_tile_n<4, DUAL>(a, stream); break;
  }
  return hipGetLastError();
}

hipError_t launch_stream_tile_up(const StreamArgs& a, hipStream_t stream) { return launch_tile<true>(a, stream); }
hipError_t launch_stream_tile_down(const StreamArgs& a, hipStream_t stream) { return launch_tile<false>(a, stream); }

}  // namespace ffnk
