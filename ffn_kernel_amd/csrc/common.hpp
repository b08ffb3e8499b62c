// Shared device/host helpers for the gfx950 kernels of libffnk.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

namespace ffnk {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int kWave = 64;

__host__ __device__ constexpr int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }
__host__ __device__ constexpr int cdiv(int a, int b) { return (a + b - 1) / b; }
__host__ __device__ constexpr int64_t round_up64(int64_t a, int64_t b) { return cdiv64(a, b) * b; }

// fp32 -> bf16, round to nearest even (NaN stays NaN).
__device__ __forceinline__ uint16_t f2bf(float f) {
  __bf16 b = static_cast<__bf16>(f);
  return __builtin_bit_cast(uint16_t, b);
}

__device__ __forceinline__ float bf2f(uint16_t v) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(v) << 16);
}

// Two fp32 -> packed pair of bf16 (lo in bits 0..15).
__device__ __forceinline__ uint32_t pack2bf(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));  // one v_cvt_pk_bf16_f32
}

// silu(g) * u in fp32: g * sigmoid(g) * u.
__device__ __forceinline__ float swiglu(float g, float u) {
  // v_exp_f32 and v_rcp_f32 are each good to 1 ulp, far inside the bf16 rounding of the result;
  // an IEEE division would cost about ten more instructions per element of the epilogue.
  const float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.44269504088896341f));
  return g * s * u;
}

// Workspace carving: every sub-buffer starts on a 256-byte boundary.
constexpr size_t kWsAlign = 256;
__host__ __device__ constexpr size_t ws_align(size_t n) { return (n + kWsAlign - 1) / kWsAlign * kWsAlign; }

}  // namespace ffnk
