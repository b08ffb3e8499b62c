// Weight-streaming kernels for the smallest MaskedFFN calls (M <= 8 token rows).
//
// With a handful of token rows the arithmetic is negligible, so nothing forces the MFMA operand
// layout on the loads (which makes every load instruction touch 16 rows x 64 bytes).  Here each
// wavefront owns a 512 * C element slice of K, keeps the token rows' values of that slice in
// registers, and streams weight rows through it as fully contiguous 1 KB loads (one row slice per
// instruction), DEPTH row slices in flight.  Products are v_dot2_f32_bf16 chains in fp32; four row
// slices at a time are summed over the 64 lanes with lane swaps + row rotations, the wavefronts of
// a workgroup (one per K slice) are summed through LDS in a fixed order, and the workgroup applies
// SwiGLU / stores the output rows itself: a call is two launches and no reduce pass.
// Same role as the reference's small-M launches of its GEMM tiles (ffn_kernel/ffn.py:527-560,
// ffn_kernel/linear.py:418-452).
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"

namespace ffnk {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

constexpr int kDotMaxM = 8;
constexpr int kDotSlice = 512;  // K elements one load instruction of a wavefront covers (64 lanes x 16 bytes)

__device__ __forceinline__ float dot8(const u32x4_t w, const u32x4_t x, float acc) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    // bit_cast of a vector element lvalue reads element 0 with this compiler: go through scalars
    const uint32_t we = w[e], xe = x[e];
    acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, we), __builtin_bit_cast(bf16x2_t, xe), acc, false);
  }
  return acc;
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
  return v + __builtin_bit_cast(float, r);
}

// In-place lane swaps of gfx950.  Written as inline assembly because the two-result compiler
// builtins (__builtin_amdgcn_permlane16_swap / permlane32_swap) return the first result twice with
// this toolchain.  The s_nop pads cover the VALU <-> permlane-swap wait states the compiler cannot
// see through the asm.
// rows (16 lanes each) a = [a0 a1 a2 a3], b = [b0 b1 b2 b3]  ->  a = [a0 b0 a2 b2], b = [a1 b1 a3 b3]
__device__ __forceinline__ void swap_rows16(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
// halves (32 lanes each) a = [a_lo a_hi], b = [b_lo b_hi]  ->  a = [a_lo b_lo], b = [a_hi b_hi]
__device__ __forceinline__ void swap_halves32(float& a, float& b) {
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}

// Every lane of 16-lane row q (lanes 16q .. 16q+15) returns the sum of v_q over all 64 lanes.
__device__ __forceinline__ float reduce4(float v0, float v1, float v2, float v3) {
  swap_rows16(v0, v1);
  const float a = v0 + v1;  // rows hold partial sums of: v0, v1, v0, v1
  swap_rows16(v2, v3);
  const float b = v2 + v3;  // rows: v2, v3, v2, v3
  float lo = a, hi = b;
  swap_halves32(lo, hi);
  float r = lo + hi;        // rows: v0, v1, v2, v3, each summed over the four rows
  r = dpp_add<0x128>(r);  // row_ror:8
  r = dpp_add<0x124>(r);  // row_ror:4
  r = dpp_add<0x122>(r);  // row_ror:2
  r = dpp_add<0x121>(r);  // row_ror:1
  return r;
}

struct DotTile {
  int grp, p0, mg, n_begin, n_rows;  // n_rows: rows of the workgroup, a multiple of 8 / (DUAL ? 2 : 1)
};

// One wavefront: K slice `wave` of every weight row of the workgroup, T token rows.
template <int T, bool DUAL, int C, int DEPTH>
__device__ __forceinline__ void dot_rows(const StreamArgs& a, const DotTile& t, const int* s_perm, float* s_red) {
  static_assert(DEPTH % 4 == 0, "row slices are reduced four at a time");
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t k0 = (int64_t)wave * (C * kDotSlice) + lane * 8;
  constexpr int MATS = DUAL ? 2 : 1;
  const int n_rv = t.n_rows * MATS;  // row slices ("row vectors") this wavefront streams; multiple of 8

  u32x4_t xr[T][C];
#pragma unroll
  for (int i = 0; i < T; ++i) {
    const int p = t.p0 + min(i, t.mg - 1);  // surplus token slots repeat the last row; never stored
    const int64_t src = a.gather_x ? (int64_t)s_perm[p] : (int64_t)p;
#pragma unroll
    for (int c = 0; c < C; ++c)
      xr[i][c] = *reinterpret_cast<const u32x4_t*>(a.X + src * a.ldx + k0 + c * kDotSlice);
  }

  const uint16_t* w0 = a.W0[t.grp] + k0;
  const uint16_t* w1 = DUAL ? a.W1[t.grp] + k0 : nullptr;
  auto rv_ptr = [&](int i) -> const uint16_t* {
    const int row = min(t.n_begin + (DUAL ? (i >> 1) : i), a.Nrows - 1);  // rows past the end: loaded, never stored
    return ((DUAL && (i & 1)) ? w1 : w0) + (int64_t)row * a.ldw;
  };
  u32x4_t ring[DEPTH][C];
  auto fetch = [&](int s, int i) {
    const uint16_t* p = rv_ptr(i);
#pragma unroll
    for (int c = 0; c < C; ++c)
      ring[s][c] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p + c * kDotSlice));
  };
#pragma unroll
  for (int s = 0; s < DEPTH; ++s) fetch(s, min(s, n_rv - 1));

  float* red = s_red + (int64_t)wave * n_rv * T;
  // Consume the DEPTH row slices in the ring starting at row vector i0; REFILL: fetch i0 + DEPTH + s
  // into the slot just consumed.
  auto consume = [&](int i0, auto refill) {
    constexpr bool REFILL = decltype(refill)::value;
#pragma unroll
    for (int b = 0; b < DEPTH / 4; ++b) {
      constexpr int TH = T > 4 ? 4 : T;  // tokens per pass: bounds the live partial sums
      float res[T];
#pragma unroll
      for (int h = 0; h < T; h += TH) {
        float part[4][TH];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int i = 0; i < TH; ++i) {
            float s = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c) s = dot8(ring[4 * b + j][c], xr[h + i][c], s);
            part[j][i] = s;
          }
#pragma unroll
        for (int i = 0; i < TH; ++i) res[h + i] = reduce4(part[0][i], part[1][i], part[2][i], part[3][i]);
      }
      if (REFILL) {
#pragma unroll
        for (int j = 0; j < 4; ++j) fetch(4 * b + j, i0 + DEPTH + 4 * b + j);
      }
      if ((lane & 15) == 0) {
        float* dst = red + (int64_t)(i0 + 4 * b + (lane >> 4)) * T;
#pragma unroll
        for (int i = 0; i < T; ++i) dst[i] = res[i];
      }
    }
  };
  int i0 = 0;
  for (; i0 + DEPTH < n_rv; i0 += DEPTH) consume(i0, std::true_type{});
  consume(i0, std::false_type{});
}

// Sum the wavefronts' partials and store: SwiGLU -> H (routed order) or out (token order).
template <int T, bool DUAL>
__device__ __forceinline__ void dot_finish(const StreamArgs& a, const DotTile& t, const int* s_perm, const float* s_red,
                                           int nwv) {
  constexpr int MATS = DUAL ? 2 : 1;
  const int n_rv = t.n_rows * MATS;
  for (int idx = threadIdx.x; idx < t.n_rows * T; idx += blockDim.x) {
    const int i = idx / t.n_rows, r = idx % t.n_rows;
    const int n = t.n_begin + r;
    if (i >= t.mg || n >= a.Nrows) continue;
    float s0 = 0.f, s1 = 0.f;
    for (int w = 0; w < nwv; ++w) {
      const float* red = s_red + (int64_t)w * n_rv * T;
      s0 += red[(r * MATS) * T + i];
      if (DUAL) s1 += red[(r * MATS + 1) * T + i];
    }
    if (DUAL) a.H[(int64_t)(t.p0 + i) * a.ldh + n] = f2bf(swiglu(s0, s1));
    else a.out[(int64_t)s_perm[t.p0 + i] * a.ldo + n] = f2bf(s0);
  }
}

__device__ __forceinline__ int route8(const uint8_t* mask, int M, int* s_perm, int* s_nvis) {
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

// grid.x = 2 * row_blocks (visual workgroups first), blockDim.x = 64 * (K / (512 * C)); rpb weight
// rows per workgroup.  Dynamic LDS: [waves][rpb * MATS][T_MAX] floats.
template <int T_MAX, bool DUAL, int C, int DEPTH, int NWV_MAX>
__global__ __launch_bounds__(NWV_MAX * kWave) void stream_dot_kernel(const StreamArgs a, const int rpb) {
  extern __shared__ __attribute__((aligned(16))) float s_red[];
  __shared__ int s_perm[kDotMaxM];
  __shared__ int s_nvis;
  const int n_vis = route8(a.mask, a.M, s_perm, &s_nvis);
  const int row_blocks = gridDim.x >> 1;
  DotTile t;
  t.grp = blockIdx.x / row_blocks;
  t.p0 = t.grp == 0 ? 0 : n_vis;
  t.mg = t.grp == 0 ? n_vis : a.M - n_vis;
  if (t.mg == 0) return;  // modality absent: its weights are never read
  t.n_begin = (blockIdx.x % row_blocks) * rpb;
  t.n_rows = rpb;
  const int nwv = blockDim.x >> 6;
  if (T_MAX >= 8 && t.mg > 4) {
    dot_rows<(T_MAX >= 8 ? 8 : 1), DUAL, C, DEPTH>(a, t, s_perm, s_red);
    __syncthreads();
    dot_finish<(T_MAX >= 8 ? 8 : 1), DUAL>(a, t, s_perm, s_red, nwv);
  } else if (T_MAX >= 4 && t.mg > 2) {
    dot_rows<(T_MAX >= 4 ? 4 : 1), DUAL, C, DEPTH>(a, t, s_perm, s_red);
    __syncthreads();
    dot_finish<(T_MAX >= 4 ? 4 : 1), DUAL>(a, t, s_perm, s_red, nwv);
  } else if (T_MAX >= 2 && t.mg > 1) {
    dot_rows<(T_MAX >= 2 ? 2 : 1), DUAL, C, DEPTH>(a, t, s_perm, s_red);
    __syncthreads();
    dot_finish<(T_MAX >= 2 ? 2 : 1), DUAL>(a, t, s_perm, s_red, nwv);
  } else {
    dot_rows<1, DUAL, C, DEPTH>(a, t, s_perm, s_red);
    __syncthreads();
    dot_finish<1, DUAL>(a, t, s_perm, s_red, nwv);
  }
}

// The dot kernels take K as waves x C x 512 elements with at most 16 wavefronts per workgroup.
bool stream_dot_ok(int M, int K) {
  if (M < 1 || M > kDotMaxM || K % kDotSlice != 0) return false;
  const int slices = K / kDotSlice;
  return slices <= 16 || (slices % 2 == 0 && slices <= 32);
}

// 512-element slices per wavefront: two when that still leaves at least four wavefronts.
int stream_dot_slices_per_wave(int K) {
  const int slices = K / kDotSlice;
  return (slices % 2 == 0 && slices >= 8) ? 2 : 1;
}

// Weight rows per workgroup: about `per_cu` workgroups per CU and modality, in whole reduce batches.
int stream_dot_rows_per_block(int Nrows, bool dual, int K) {
  const int c = stream_dot_slices_per_wave(K);
  const int waves = K / (kDotSlice * c);
  const int per_cu = waves <= 4 ? 2 : 1;
  const int unit = dual ? 4 : 8;
  int rpb = cdiv(cdiv(Nrows, 256 * per_cu), unit) * unit;
  // LDS: waves * rpb * mats * 8 floats <= 48 KB
  const int cap = (48 * 1024 / (waves * (dual ? 2 : 1) * 8 * 4)) / unit * unit;
  if (rpb > cap) rpb = cap;
  return rpb < unit ? unit : rpb;
}

template <int T_MAX, bool DUAL, int C>
static void launch_dot_c(const StreamArgs& a, hipStream_t stream) {
  const int waves = a.K / (kDotSlice * C);
  const int rpb = stream_dot_rows_per_block(a.Nrows, DUAL, a.K);
  const int row_blocks = cdiv(a.Nrows, rpb);
  const size_t lds = (size_t)waves * rpb * (DUAL ? 2 : 1) * T_MAX * sizeof(float);
  if (waves <= 4)
    hipLaunchKernelGGL((stream_dot_kernel<T_MAX, DUAL, C, 8, 4>), dim3(2 * row_blocks), dim3(waves * kWave), lds, stream, a, rpb);
  else if (waves <= 8)
    hipLaunchKernelGGL((stream_dot_kernel<T_MAX, DUAL, C, 8, 8>), dim3(2 * row_blocks), dim3(waves * kWave), lds, stream, a, rpb);
  else
    hipLaunchKernelGGL((stream_dot_kernel<T_MAX, DUAL, C, 4, 16>), dim3(2 * row_blocks), dim3(waves * kWave), lds, stream, a, rpb);
}

template <bool DUAL>
static hipError_t launch_dot(const StreamArgs& a, hipStream_t stream) {
  if (!stream_dot_ok(a.M, a.K) || a.splits != 1 || a.ldw % 8 != 0 || a.ldx % 8 != 0) return hipErrorInvalidValue;
  if (DUAL ? (a.H == nullptr) : (a.out == nullptr)) return hipErrorInvalidValue;
  const int c = stream_dot_slices_per_wave(a.K);
  const int tmax = a.M > 4 ? 8 : a.M > 2 ? 4 : a.M > 1 ? 2 : 1;
#define FFNK_DOT_CASE(TM)                                        \
  case TM:                                                       \
    if (c == 2) launch_dot_c<TM, DUAL, 2>(a, stream);            \
    else launch_dot_c<TM, DUAL, 1>(a, stream);                   \
    break;
  switch (tmax) {
    FFNK_DOT_CASE(1)
    FFNK_DOT_CASE(2)
    FFNK_DOT_CASE(4)
    FFNK_DOT_CASE(8)
  }
#undef FFNK_DOT_CASE
  return hipGetLastError();
}

hipError_t launch_stream_dot_up(const StreamArgs& a, hipStream_t stream) { return launch_dot<true>(a, stream); }
hipError_t launch_stream_dot_down(const StreamArgs& a, hipStream_t stream) { return launch_dot<false>(a, stream); }

}  // namespace ffnk
