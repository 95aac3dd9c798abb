// Vector types and small device helpers shared by the kernel sources.
#pragma once

#include <hip/hip_runtime.h>

#include "device_math.h"
#include "kernels.h"

namespace lc0mi {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx8 __attribute__((ext_vector_type(8)));

// 16-bit element types of activations and weights: IEEE half and bfloat16 (the same storage, kernels are
// instantiated for either). Vector forms and the 32x32x16 / 16x16x32 matrix instructions per type.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
template <typename T> struct Vec16;
template <> struct Vec16<half_t> { using v8 = half8; using v4 = half4; };
template <> struct Vec16<bf16_t> { using v8 = bf16x8; using v4 = bf16x4; };

namespace {

__device__ __forceinline__ floatx16 Mfma32(half8 a, half8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx16 Mfma32(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx4 Mfma16(half8 a, half8 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx4 Mfma16(bf16x8 a, bf16x8 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Calls f with a branch-free functor for the activation, so that unrolled
// epilogue loops do not carry a per-element switch.
template <typename F>
__device__ __forceinline__ void DispatchAct(int act, F&& f) {
  switch (act) {
    case 1: f([](float v) { return ActMish(v); }); break;
    case 2: f([](float v) { return v > 0.0f ? v : 0.0f; }); break;
    case 7: f([](float v) { return v * ActSigmoid(v); }); break;
    case 8: f([](float v) { return v > 0.0f ? v * v : 0.0f; }); break;
    case 3: f([](float v) { return v; }); break;
    default: f([act](float v) { return Activate(v, act); }); break;
  }
}

// bias[n..n+3] (zeros when there is no bias or past N).
__device__ __forceinline__ void LoadBias4(const float* bias, int n, int N, float out[4]) {
  if (bias != nullptr && n + 3 < N) {
    floatx4 b = *reinterpret_cast<const floatx4*>(bias + n);
    out[0] = b[0]; out[1] = b[1]; out[2] = b[2]; out[3] = b[3];
  } else {
#pragma unroll
    for (int r = 0; r < 4; r++) out[r] = (bias != nullptr && n + r < N) ? bias[n + r] : 0.0f;
  }
}

__device__ __forceinline__ float WaveSum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// The value of v in the lane that the data-parallel-primitive control CTRL selects (0xB1: lane ^ 1, 0x4E: lane ^ 2
// within a group of four, 0x141: mirrored within a group of eight).
template <int CTRL>
__device__ __forceinline__ float DppMove(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}

// Mean and 1 / sqrt(variance + eps) of row m from its partial (sum, sum of squares) pairs over n values.
__device__ __forceinline__ void RowMeanRstd(const float* stats, int parts, long long m, int n, float eps, float& mean,
                                            float& rstd) {
  const float2* s = reinterpret_cast<const float2*>(stats) + m * parts;
  float s1 = 0.0f, s2 = 0.0f;
  for (int i = 0; i < parts; i++) {
    const float2 v = s[i];
    s1 += v.x;
    s2 += v.y;
  }
  const float inv_n = 1.0f / (float)n;
  mean = s1 * inv_n;
  rstd = 1.0f / sqrtf(fmaxf(s2 * inv_n - mean * mean, 0.0f) + eps);
}

}  // namespace

}  // namespace lc0mi
