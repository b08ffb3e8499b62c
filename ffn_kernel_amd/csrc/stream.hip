// Weight-streaming kernels for decode-shaped MaskedFFN calls (M <= 64 token rows).
//
// With so few rows the op is bound by reading each present modality's three weight matrices
// once from HBM, so the design goal is bytes in flight, not MFMA occupancy:
//   * every wavefront owns 16 weight rows and streams them K-contiguously straight into MFMA
//     "A" fragments (v_mfma_f32_16x16x32_bf16: lane = row l % 16, 16 bytes at k + 8 * (l / 16)),
//     one 128-element K chunk (4 loads of 1 KB per matrix) ahead of the chunk being multiplied;
//   * the few token rows (x, or the SwiGLU intermediate) are L1/L2-resident and are loaded as
//     "B" fragments the same way, so wavefronts never wait for one another (no LDS, no barriers);
//   * the row -> modality routing is recomputed per workgroup from the mask (a 64-lane ballot), so
//     a call is three launches: up-projection + SwiGLU, split-K down-projection, reduce + scatter.
// The reference runs these shapes through its 128x64 GEMM tiles (ffn_kernel/ffn.py:527-560,
// ffn_kernel/linear.py:418-452), which leaves most of the GPU idle at M <= 64.
#include "common.hpp"
#include "launch.hpp"

namespace ffnk {

constexpr int kSK = 128;                    // K elements per streamed chunk
constexpr int kSMaxM = 64;

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// Routing of up to 64 rows, computed by wave 0 of the workgroup: s_perm[p] = token row at routed
// position p (visual rows first, ascending); returns the number of visual rows.
__device__ __forceinline__ int route_small(const uint8_t* mask, int M, int* s_perm, int* s_nvis) {
  if (threadIdx.x < kWave) {
    const int l = threadIdx.x;
    const bool valid = l < M;
    const bool vis = valid && mask[l] != 0;
    const unsigned long long vm = __ballot(vis);
    const unsigned long long am = __ballot(valid);
    const unsigned long long lt = (l == 0) ? 0ull : (~0ull >> (64 - l));
    const int nv = __popcll(vm);
    if (valid) {
      const int pos = vis ? __popcll(vm & lt) : nv + __popcll(~vm & am & lt);
      s_perm[pos] = l;
    }
    if (l == 0) *s_nvis = nv;
  }
  __syncthreads();
  return *s_nvis;
}

struct StreamTile {
  int grp, split, p0, mg, n0, c0, nc;
};

// K loop and epilogue of one wavefront for a group with NTM 16-row m-tiles.  The wavefront owns 16
// weight rows (of each matrix) and is independent of every other wavefront: weight fragments and
// token-row fragments are both loaded straight from global memory into MFMA operand registers
// (the token rows are few and L1/L2-resident), one 128-element K chunk ahead of the MFMAs.
// acc = W_frag (16 rows x 32 k) * X_frag (32 k x 16 token rows) per 16x16 tile.
template <int NTM, bool DUAL, int RT, int KS, int NWV>
__device__ __forceinline__ void stream_rows(const StreamArgs& a, const StreamTile& t, const int* s_perm,
                                            float* s_red) {
  constexpr int CK = KS * 32;  // K elements per chunk (t.c0 / t.nc count chunks of this size)
  const int lane = threadIdx.x & 63;
  const int lrow = lane & 15, lq = lane >> 4;
  constexpr int NW = RT * (DUAL ? 2 : 1);  // weight fragments per k-step: [row tile][gate, up]
  const uint16_t* wp[NW];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int n_ld = min(t.n0 + r * 16 + lrow, a.Nrows - 1);  // rows past the end are loaded but never stored
    wp[r * (DUAL ? 2 : 1)] = a.W0[t.grp] + (int64_t)n_ld * a.ldw + (int64_t)t.c0 * CK + lq * 8;
    if (DUAL) wp[r * 2 + 1] = a.W1[t.grp] + (int64_t)n_ld * a.ldw + (int64_t)t.c0 * CK + lq * 8;
  }
  const uint16_t* xp[NTM];
#pragma unroll
  for (int m = 0; m < NTM; ++m) {
    const int p = t.p0 + min(m * 16 + lrow, t.mg - 1);  // surplus rows repeat the last one; dropped below
    const int64_t src = a.gather_x ? (int64_t)s_perm[p] : (int64_t)p;
    xp[m] = a.X + src * a.ldx + (int64_t)t.c0 * CK + lq * 8;
  }

  f32x4_t acc[NW][NTM];
#pragma unroll
  for (int w = 0; w < NW; ++w)
#pragma unroll
    for (int m = 0; m < NTM; ++m) acc[w][m] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  u32x4_t wa[NW][KS], wb[NW][KS];    // two chunk buffers of weight fragments
  u32x4_t xa[NTM][KS], xb[NTM][KS];  // and of token-row fragments

  auto load = [&](u32x4_t (&dw)[NW][KS], u32x4_t (&dx)[NTM][KS], int c) {
    const int64_t ko = (int64_t)c * CK;
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int w = 0; w < NW; ++w)
        dw[w][s] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(wp[w] + ko + s * 32));
#pragma unroll
    for (int m = 0; m < NTM; ++m)
#pragma unroll
      for (int s = 0; s < KS; ++s) dx[m][s] = *reinterpret_cast<const u32x4_t*>(xp[m] + ko + s * 32);
  };
  auto compute = [&](const u32x4_t (&dw)[NW][KS], const u32x4_t (&dx)[NTM][KS]) {
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
      for (int m = 0; m < NTM; ++m) {
        const bf16x8_t xf = __builtin_bit_cast(bf16x8_t, dx[m][s]);
#pragma unroll
        for (int w = 0; w < NW; ++w)
          acc[w][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, dw[w][s]), xf, acc[w][m], 0, 0, 0);
      }
  };

  if (t.nc > 0) {
    load(wa, xa, 0);
    for (int c = 0; c < t.nc; c += 2) {
      if (c + 1 < t.nc) load(wb, xb, c + 1);
      compute(wa, xa);
      if (c + 1 < t.nc) {
        if (c + 2 < t.nc) load(wa, xa, c + 2);
        compute(wb, xb);
      }
    }
  }

  // The wavefronts of the workgroup hold partial sums over their shares of the K range:
  // add them up through LDS (fixed order: deterministic), wave 0 finishes.
  const int wave = threadIdx.x >> 6;
  if (wave > 0) {
#pragma unroll
    for (int w = 0; w < NW; ++w)
#pragma unroll
      for (int m = 0; m < NTM; ++m)
        *reinterpret_cast<f32x4_t*>(s_red + ((((wave - 1) * NW + w) * NTM + m) * 64 + lane) * 4) = acc[w][m];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int v = 0; v < NWV - 1; ++v)
#pragma unroll
    for (int w = 0; w < NW; ++w)
#pragma unroll
      for (int m = 0; m < NTM; ++m)
        acc[w][m] += *reinterpret_cast<const f32x4_t*>(s_red + (((v * NW + w) * NTM + m) * 64 + lane) * 4);

  // acc[.][m][v]: weight row n0 + 16 * (row tile) + 4 * lq + v, token row m * 16 + lrow of the group.
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int n_out = t.n0 + r * 16 + 4 * lq;
    if (n_out >= a.Nrows) continue;
#pragma unroll
    for (int m = 0; m < NTM; ++m) {
      const int row = m * 16 + lrow;
      if (row < t.mg) {
        if (DUAL) {
          const f32x4_t g = acc[r * 2][m], u = acc[r * 2 + (DUAL ? 1 : 0)][m];
          uint2 v2;
          v2.x = pack2bf(swiglu(g[0], u[0]), swiglu(g[1], u[1]));
          v2.y = pack2bf(swiglu(g[2], u[2]), swiglu(g[3], u[3]));
          *reinterpret_cast<uint2*>(a.H + (int64_t)(t.p0 + row) * a.ldh + n_out) = v2;
        } else if (a.P != nullptr) {
          const f32x4_t o = acc[r][m];
          *reinterpret_cast<float4*>(a.P + ((int64_t)t.split * a.M + (t.p0 + row)) * a.Nrows + n_out) =
              make_float4(o[0], o[1], o[2], o[3]);
        } else {
          // single split: this workgroup holds the complete sums, store the output row directly
          const f32x4_t o = acc[r][m];
          uint2 v2;
          v2.x = pack2bf(o[0], o[1]);
          v2.y = pack2bf(o[2], o[3]);
          uint16_t* dst = a.out + (int64_t)s_perm[t.p0 + row] * a.ldo + n_out;
          if ((reinterpret_cast<uintptr_t>(dst) & 7) == 0) *reinterpret_cast<uint2*>(dst) = v2;
          else { dst[0] = f2bf(o[0]); dst[1] = f2bf(o[1]); dst[2] = f2bf(o[2]); dst[3] = f2bf(o[3]); }
        }
      }
    }
  }
}

// NTM_MAX = ceil(M / 16), known on the host: bounds the register budget so that small-M calls
// run at higher occupancy.  A workgroup = 16 weight rows (of each matrix) x one K range; its four
// wavefronts take a quarter of the range each.
template <int NTM_MAX, bool DUAL, int RT, int KS, int NWV, int OCC>
__global__ __launch_bounds__(NWV * kWave, OCC) void stream_kernel(const StreamArgs a) {
  __shared__ int s_perm[kSMaxM];
  __shared__ int s_nvis;
  __shared__ __attribute__((aligned(16))) float s_red[(NWV - 1) * RT * (DUAL ? 2 : 1) * NTM_MAX * 64 * 4];
  const int n_vis = route_small(a.mask, a.M, s_perm, &s_nvis);

  // blockIdx -> (group, split, row block)
  const int row_blocks = cdiv(a.Nrows, 16 * RT);
  StreamTile t;
  // Group-major order: all workgroups of the visual group, then all of the text group.  (Interleaving
  // the groups was measured 1.5x slower when one modality is absent: its empty workgroups still take
  // their turn in the round-robin placement over CUs, so the real ones pile up on half of the CUs.)
  const int per_grp = row_blocks * a.splits;
  t.grp = blockIdx.x / per_grp;
  const int rem = blockIdx.x % per_grp;
  t.split = rem / row_blocks;
  t.p0 = t.grp == 0 ? 0 : n_vis;            // first routed position of the group
  t.mg = t.grp == 0 ? n_vis : a.M - n_vis;  // rows in the group
  if (t.mg == 0) return;                    // modality absent: its weights are never read
  t.n0 = (rem % row_blocks) * 16 * RT;
  // K range of the workgroup (this split), then this wavefront's quarter of it, in chunks
  // (splits are laid out in 128-element units so that the host's choice does not depend on KS)
  constexpr int PER128 = kSK / (KS * 32);
  const int n128 = a.K / kSK;
  const int cps = cdiv(n128, a.splits);
  const int b0 = min(t.split * cps, n128) * PER128, b1 = min((t.split + 1) * cps, n128) * PER128;
  const int per_wave = cdiv(b1 - b0, NWV);
  const int wave = threadIdx.x >> 6;
  t.c0 = min(b0 + wave * per_wave, b1);
  t.nc = min(t.c0 + per_wave, b1) - t.c0;

  const int ntm = cdiv(t.mg, 16);  // uniform over the workgroup
  if (NTM_MAX >= 4 && ntm >= 4) stream_rows<(NTM_MAX >= 4 ? 4 : 1), DUAL, RT, KS, NWV>(a, t, s_perm, s_red);
  else if (NTM_MAX >= 3 && ntm == 3) stream_rows<(NTM_MAX >= 3 ? 3 : 1), DUAL, RT, KS, NWV>(a, t, s_perm, s_red);
  else if (NTM_MAX >= 2 && ntm == 2) stream_rows<(NTM_MAX >= 2 ? 2 : 1), DUAL, RT, KS, NWV>(a, t, s_perm, s_red);
  else stream_rows<1, DUAL, RT, KS, NWV>(a, t, s_perm, s_red);
}

// out[perm[p], n] = bf16(sum_s P[s][p][n]); one workgroup per (routed row, 1024 columns).
__global__ __launch_bounds__(256) void stream_reduce_kernel(const float* __restrict__ P, int splits, int M, int N,
                                                            const uint8_t* __restrict__ mask,
                                                            uint16_t* __restrict__ out, int64_t ldo) {
  __shared__ int s_perm[kSMaxM];
  __shared__ int s_nvis;
  route_small(mask, M, s_perm, &s_nvis);
  const int p = blockIdx.y;
  const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (n >= N) return;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int k = 0; k < splits; ++k) {
    const float4 v = *reinterpret_cast<const float4*>(P + ((int64_t)k * M + p) * N + n);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  uint16_t* o = out + (int64_t)s_perm[p] * ldo + n;
  if ((reinterpret_cast<uintptr_t>(o) & 7) == 0) {
    uint2 v2;
    v2.x = pack2bf(s.x, s.y);
    v2.y = pack2bf(s.z, s.w);
    *reinterpret_cast<uint2*>(o) = v2;
  } else {
    o[0] = f2bf(s.x); o[1] = f2bf(s.y); o[2] = f2bf(s.z); o[3] = f2bf(s.w);
  }
}

// Shape of the streaming kernel per (m-tiles, projection): RT row tiles of 16 weight rows per
// wavefront (a token-row fragment is then used RT times), KS 32-element k-steps per chunk, NWV
// wavefronts per workgroup sharing the K range, OCC waves per SIMD the register budget allows.
template <int RT_, int KS_, int NWV_, int OCC_>
struct StreamShapeV {
  static constexpr int RT = RT_, KS = KS_, NWV = NWV_, OCC = OCC_;
};
template <int NTM_MAX, bool DUAL>
struct StreamShape : StreamShapeV<2, (DUAL ? 2 : 4), 4, 2> {};
template <>
struct StreamShape<1, true> : StreamShapeV<1, 4, 4, 4> {};
template <>
struct StreamShape<1, false> : StreamShapeV<1, 4, 16, 4> {};

int stream_rows_per_block(int M, bool dual) {
  switch (cdiv(M, 16)) {
    case 1: return 16 * (dual ? StreamShape<1, true>::RT : StreamShape<1, false>::RT);
    case 2: return 16 * (dual ? StreamShape<2, true>::RT : StreamShape<2, false>::RT);
    case 3: return 16 * (dual ? StreamShape<3, true>::RT : StreamShape<3, false>::RT);
    default: return 16 * (dual ? StreamShape<4, true>::RT : StreamShape<4, false>::RT);
  }
}

int stream_waves_per_block(int M, bool dual) {
  switch (cdiv(M, 16)) {
    case 1: return dual ? StreamShape<1, true>::NWV : StreamShape<1, false>::NWV;
    case 2: return dual ? StreamShape<2, true>::NWV : StreamShape<2, false>::NWV;
    case 3: return dual ? StreamShape<3, true>::NWV : StreamShape<3, false>::NWV;
    default: return dual ? StreamShape<4, true>::NWV : StreamShape<4, false>::NWV;
  }
}

int stream_chunk_k(int M, bool dual) {
  switch (cdiv(M, 16)) {
    case 1: return 32 * (dual ? StreamShape<1, true>::KS : StreamShape<1, false>::KS);
    case 2: return 32 * (dual ? StreamShape<2, true>::KS : StreamShape<2, false>::KS);
    case 3: return 32 * (dual ? StreamShape<3, true>::KS : StreamShape<3, false>::KS);
    default: return 32 * (dual ? StreamShape<4, true>::KS : StreamShape<4, false>::KS);
  }
}

template <int NTM_MAX, bool DUAL>
static void launch_stream_n(const StreamArgs& a, hipStream_t stream) {
  using S = StreamShape<NTM_MAX, DUAL>;
  const int blocks = 2 * cdiv(a.Nrows, 16 * S::RT) * a.splits;
  hipLaunchKernelGGL((stream_kernel<NTM_MAX, DUAL, S::RT, S::KS, S::NWV, S::OCC>), dim3(blocks), dim3(S::NWV * kWave), 0, stream, a);
}

template <bool DUAL>
static hipError_t launch_stream(const StreamArgs& a, hipStream_t stream) {
  if (a.M < 1 || a.M > kSMaxM || a.K % kSK != 0 || a.splits < 1) return hipErrorInvalidValue;
  if (!DUAL && a.P == nullptr && (a.splits != 1 || a.out == nullptr)) return hipErrorInvalidValue;
  switch (cdiv(a.M, 16)) {
    case 1: launch_stream_n<1, DUAL>(a, stream); break;
    case 2: launch_stream_n<2, DUAL>(a, stream); break;
    case 3: launch_stream_n<3, DUAL>(a, stream); break;
    default: launch_stream_n<4, DUAL>(a, stream); break;
  }
  return hipGetLastError();
}

hipError_t launch_stream_up(const StreamArgs& a, hipStream_t stream) { return launch_stream<true>(a, stream); }

hipError_t launch_stream_down(const StreamArgs& a, hipStream_t stream) { return launch_stream<false>(a, stream); }

hipError_t launch_stream_reduce(const float* P, int splits, int M, int N, const uint8_t* mask, uint16_t* out,
                                int64_t ldo, hipStream_t stream) {
  dim3 grid(cdiv(N, 1024), M);
  hipLaunchKernelGGL(stream_reduce_kernel, grid, dim3(256), 0, stream, P, splits, M, N, mask, out, ldo);
  return hipGetLastError();
}

}  // namespace ffnk
