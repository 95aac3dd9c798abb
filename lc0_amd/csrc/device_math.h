// Device-side activation functions and the e4m3 pack shared by the kernel sources.
#pragma once

#include <hip/hip_runtime.h>

namespace lc0mi {

// lc0's ActivationFunction numbering (src/neural/tables/activation_function.h:24-35).
enum : int { kActMish = 1, kActRelu = 2, kActNone = 3, kActTanh = 4, kActSigmoid = 5, kActSelu = 6, kActSwish = 7,
             kActRelu2 = 8 };

// Activation functions (values as shared/activation.cc:51-100). The GEMM epilogues are bound by
// vector-ALU issue, so mish and swish use one hardware exponential and one hardware reciprocal
// (1 ulp each) instead of a correctly rounded division:
//   mish(v) = v * tanh(log(1 + e^v)) = v * n / (n + 2),  n = e^v * (e^v + 2).
// The exponent is clamped at 20, where n / (n + 2) already rounds to 1 in float.
static __device__ __forceinline__ float ActMish(float v) {
  const float e = __expf(__builtin_fminf(v, 20.0f));
  const float n = e * (e + 2.0f);
  return v * n * __builtin_amdgcn_rcpf(n + 2.0f);
}
static __device__ __forceinline__ float ActSigmoid(float v) { return __builtin_amdgcn_rcpf(1.0f + __expf(-v)); }
static __device__ __forceinline__ float Activate(float v, int act) {
  switch (act) {
    case 1: return ActMish(v);
    case 2: return v > 0.0f ? v : 0.0f;
    case 4: return tanhf(v);
    case 5: return ActSigmoid(v);
    case 6: {
      // Both sides computed for every lane and one select: with the exponential on one side only of a conditional
      // expression this became a branch per element (16384x1536x1024 product: 77 -> 73 us; 59 without activation).
      const bool pos = v > 0.0f;
      const float neg = 1.05070098f * 1.67326324f * (__expf(pos ? 0.0f : v) - 1.0f);
      return pos ? 1.05070098f * v : neg;
    }
    case 7: return v * ActSigmoid(v);
    case 8: return v > 0.0f ? v * v : 0.0f;
    default: return v;
  }
}

// 4 floats -> 4 e4m3 bytes (round to nearest even, saturating at +-448; the
// hardware conversion alone would turn |v| > 464 into NaN).
static __device__ __forceinline__ unsigned PackFp8x4(float a, float b, float c, float d) {
  a = __builtin_amdgcn_fmed3f(a, -448.0f, 448.0f);  // median of three = clamp, one instruction
  b = __builtin_amdgcn_fmed3f(b, -448.0f, 448.0f);
  c = __builtin_amdgcn_fmed3f(c, -448.0f, 448.0f);
  d = __builtin_amdgcn_fmed3f(d, -448.0f, 448.0f);
  int v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
  return (unsigned)v;
}

}  // namespace lc0mi
