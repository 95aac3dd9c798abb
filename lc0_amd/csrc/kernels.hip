// Hand-written gfx950 (CDNA4, wave64) kernels of the attention-body path other than the matrix products
// (gemm_kernels.hip) and the fused smolgen attention (smolgen_attention.hip).
//
// What each kernel replaces in the reference CPU backend (file:line):
//   expand_planes_*       BlasComputation::EncodePlanes + NCHW->NHWC + pos-enc concat
//                         blas/network_blas.cc:973-981, 630-652
//   layer_norm_kernel     LayerNorm2DWithSkipConnection   blas/encoder.h:29-66
//   attention_kernel      per-head QK^T, +smolgen, softmax, .V   blas/network_blas.cc:352-439
//   attn_policy_gather    promotion offsets + kAttnPolicyMap gather  blas/network_blas.cc:873-914
#include "kernel_common.h"

#include <algorithm>
#include <stdexcept>
#include <type_traits>
#include <utility>

namespace lc0mi {

// ---------------------------------------------------------------------------
// Input plane expansion.
// ---------------------------------------------------------------------------
namespace {
template <typename T, int V>   // V channels per thread and store: 8 when ld % 8 == 0, else 1
__global__ __launch_bounds__(256) void expand_planes_attn_kernel(const uint64_t* __restrict__ masks,
                                                                 const float* __restrict__ values,
                                                                 const T* __restrict__ extra, int n_extra,
                                                                 long long extra_batch_stride,
                                                                 T* __restrict__ out, int ld) {
  const int b = blockIdx.x;
  const T* ex = extra + (long long)b * extra_batch_stride;
  __shared__ uint64_t smask[112];
  __shared__ float sval[112];
  if (threadIdx.x < 112) {
    smask[threadIdx.x] = masks[(long long)b * 112 + threadIdx.x];
    sval[threadIdx.x] = values[(long long)b * 112 + threadIdx.x];
  }
  __syncthreads();
  T* o = out + (long long)b * 64 * ld;
  const int chunks = ld / V;
  // (a workgroup per 16 squares of a position: one per position left most CUs idle at up to a few hundred positions)
  const int sq_begin = blockIdx.y * 16;
  for (int i = threadIdx.x; i < 16 * chunks; i += 256) {
    const int sq = sq_begin + i / chunks, c0 = (i % chunks) * V;
    T v[V];
#pragma unroll
    for (int e = 0; e < V; e++) {
      const int c = c0 + e;
      T x = (T)0.0f;
      if (c < 112) {
        if ((smask[c] >> sq) & 1ull) x = (T)sval[c];
      } else if (c < 112 + n_extra) {
        x = ex[sq * n_extra + (c - 112)];
      }
      v[e] = x;
    }
    T* dst = o + (long long)sq * ld + c0;
    if constexpr (V == 1) {
      dst[0] = v[0];
    } else if constexpr (sizeof(T) == 2) {
      *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(v);
    } else {
      *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(v);
      *reinterpret_cast<uint4*>(dst + 4) = *reinterpret_cast<const uint4*>(v + 4);
    }
  }
}

// First 12 planes (the current position's pieces) square-major: out[b][sq * 12 + j].
template <typename T>
__global__ __launch_bounds__(256) void piece_planes_kernel(const uint64_t* __restrict__ masks,
                                                           const float* __restrict__ values,
                                                           T* __restrict__ out) {
  const int b = blockIdx.x;
  for (int i = threadIdx.x; i < 64 * 12; i += 256) {
    const int sq = i / 12, j = i - sq * 12;
    const bool bit = (masks[(long long)b * 112 + j] >> sq) & 1ull;
    out[(long long)b * 768 + i] = bit ? (T)values[(long long)b * 112 + j] : (T)0.0f;
  }
}

// x[b][sq][c] = x * mult[sq][c] + add[sq][c]
template <typename T>
__global__ __launch_bounds__(256) void input_gating_kernel(T* __restrict__ x, const float* __restrict__ mult,
                                                           const float* __restrict__ add, int per_sample,
                                                           long long total) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int j = (int)(i % per_sample);
  x[i] = (T)((float)x[i] * mult[j] + add[j]);
}

template <typename T>
__global__ __launch_bounds__(256) void expand_planes_nchw_kernel(const uint64_t* __restrict__ masks,
                                                                 const float* __restrict__ values,
                                                                 T* __restrict__ out, long long total) {
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  long long plane = i >> 6;
  int sq = (int)(i & 63);
  out[i] = ((masks[plane] >> sq) & 1ull) ? (T)values[plane] : (T)0.0f;
}
}  // namespace

template <typename T>
void LaunchExpandPlanesAttn(const uint64_t* masks, const float* values, const T* pos_enc, T* out, int ld,
                            int batch, hipStream_t stream) {
  if (batch <= 0) return;
  if (ld % 8 == 0) {
    hipLaunchKernelGGL((expand_planes_attn_kernel<T, 8>), dim3(batch, 4), dim3(256), 0, stream, masks, values, pos_enc, 64,
                       0LL, out, ld);
  } else {
    hipLaunchKernelGGL((expand_planes_attn_kernel<T, 1>), dim3(batch, 4), dim3(256), 0, stream, masks, values, pos_enc, 64,
                       0LL, out, ld);
  }
}

template <typename T>
void LaunchExpandPlanesDense(const uint64_t* masks, const float* values, const T* extra, int n_extra, T* out, int ld,
                             int batch, hipStream_t stream) {
  if (batch <= 0) return;
  if (ld % 8 == 0) {
    hipLaunchKernelGGL((expand_planes_attn_kernel<T, 8>), dim3(batch, 4), dim3(256), 0, stream, masks, values, extra,
                       n_extra, 64LL * n_extra, out, ld);
  } else {
    hipLaunchKernelGGL((expand_planes_attn_kernel<T, 1>), dim3(batch, 4), dim3(256), 0, stream, masks, values, extra,
                       n_extra, 64LL * n_extra, out, ld);
  }
}

template <typename T>
void LaunchPiecePlanes(const uint64_t* masks, const float* values, T* out, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  hipLaunchKernelGGL(piece_planes_kernel<T>, dim3(batch), dim3(256), 0, stream, masks, values, out);
}

template <typename T>
void LaunchInputGating(T* x, const float* mult, const float* add, int batch, int per_sample, hipStream_t stream) {
  const long long total = (long long)batch * per_sample;
  if (total <= 0) return;
  hipLaunchKernelGGL(input_gating_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, x, mult, add,
                     per_sample, total);
}
#define LC0MI_INSTANTIATE_PLANES(T)                                                                                  \
  template void LaunchExpandPlanesAttn<T>(const uint64_t*, const float*, const T*, T*, int, int, hipStream_t);       \
  template void LaunchExpandPlanesDense<T>(const uint64_t*, const float*, const T*, int, T*, int, int, hipStream_t); \
  template void LaunchPiecePlanes<T>(const uint64_t*, const float*, T*, int, hipStream_t);                           \
  template void LaunchInputGating<T>(T*, const float*, const float*, int, int, hipStream_t);
LC0MI_INSTANTIATE_PLANES(half_t)
LC0MI_INSTANTIATE_PLANES(bf16_t)
LC0MI_INSTANTIATE_PLANES(float)
#undef LC0MI_INSTANTIATE_PLANES

template <typename T>
void LaunchExpandPlanesNchw(const uint64_t* masks, const float* values, T* out, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  long long total = (long long)batch * 112 * 64;
  hipLaunchKernelGGL(expand_planes_nchw_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                     masks, values, out, total);
}
template void LaunchExpandPlanesNchw<half_t>(const uint64_t*, const float*, half_t*, int, hipStream_t);
template void LaunchExpandPlanesNchw<float>(const uint64_t*, const float*, float*, int, hipStream_t);

// ---------------------------------------------------------------------------
// Layer norm with optional skip: one wave per row, the row held in registers.
// ---------------------------------------------------------------------------
namespace {
template <int NV, typename ET>  // 16-byte vectors per lane, covers C <= 512 * NV; ET: half_t or bf16_t (bits in half_t storage)
__global__ __launch_bounds__(256) void layer_norm_kernel(const half_t* __restrict__ x, const half_t* skip,
                                                         half_t* y, uint8_t* yq, float q_mul,
                                                         const float* __restrict__ gamma,
                                                         const float* __restrict__ beta, int rows, int C,
                                                         float alpha, float eps, bool through) {
  using ev8 = typename Vec16<ET>::v8;
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int nvec = C / 8;
  const half_t* xr = x + (long long)row * C;
  const half_t* sr = skip ? skip + (long long)row * C : nullptr;
  float t[NV][8];
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int v = lane + i * 64;
    if (v < nvec) {
      // (through: x is not read again and is kept out of the caches on its way in)
      ev8 hx = through ? __builtin_nontemporal_load(reinterpret_cast<const ev8*>(xr + v * 8))
                       : *reinterpret_cast<const ev8*>(xr + v * 8);
      if (sr) {
        ev8 hs = *reinterpret_cast<const ev8*>(sr + v * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) t[i][e] = (float)hx[e] * alpha + (float)hs[e];
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++) t[i][e] = (float)hx[e] * alpha;
      }
#pragma unroll
      for (int e = 0; e < 8; e++) sum += t[i][e];
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) t[i][e] = 0.0f;
    }
  }
  const float mean = WaveSum(sum) / (float)C;
  float var = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    if (lane + i * 64 < nvec) {
#pragma unroll
      for (int e = 0; e < 8; e++) { float d = t[i][e] - mean; var += d * d; }
    }
  }
  var = WaveSum(var) / (float)C;
  const float den = 1.0f / sqrtf(var + eps);
  half_t* yr = y + (long long)row * C;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    int v = lane + i * 64;
    if (v < nvec) {
      ev8 o;
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; e++) {
        f[e] = beta[v * 8 + e] + gamma[v * 8 + e] * (t[i][e] - mean) * den;
        o[e] = (ET)f[e];
      }
      if (through) {   // written through at system scope: past L2, into the memory-side cache (the no-op: the wait
                       // states between a 16-byte store and a vector ALU write to its data registers)
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 2" ::"v"(yr + v * 8), "v"(o) : "memory");
      } else {
        *reinterpret_cast<ev8*>(yr + v * 8) = o;
      }
      if (yq) {  // e4m3 copy of the same row for the next fp8 GEMM
        uint2 q;
        q.x = PackFp8x4(f[0] * q_mul, f[1] * q_mul, f[2] * q_mul, f[3] * q_mul);
        q.y = PackFp8x4(f[4] * q_mul, f[5] * q_mul, f[6] * q_mul, f[7] * q_mul);
        *reinterpret_cast<uint2*>(yq + (long long)row * C + v * 8) = q;
      }
    }
  }
}

__global__ __launch_bounds__(256) void quantize_f8_kernel(const half_t* __restrict__ x, uint8_t* __restrict__ y,
                                                          long long nvec, float mul) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const half8 h = *reinterpret_cast<const half8*>(x + i * 8);
  uint2 q;
  q.x = PackFp8x4((float)h[0] * mul, (float)h[1] * mul, (float)h[2] * mul, (float)h[3] * mul);
  q.y = PackFp8x4((float)h[4] * mul, (float)h[5] * mul, (float)h[6] * mul, (float)h[7] * mul);
  *reinterpret_cast<uint2*>(y + i * 8) = q;
}
}  // namespace

namespace {
__global__ __launch_bounds__(256) void zero_kernel(float* p, long long n) {
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.0f;
}

// One workgroup per row; every thread keeps up to 4 vectors of 8 elements.
// EARLY (few rows, where the kernel's latency is the pass's): gamma and beta, which nobody has touched since the
// previous pass, are asked for first and arrive while the row is reduced; otherwise they are read where they are
// used, which leaves more of the CU to a GEMM on the other stream.
template <bool EARLY, typename ET>
__global__ __launch_bounds__(256) void layer_norm_rows_kernel(const float* __restrict__ xf, int n_partials,
                                                              long long partial_stride, const half_t* xh,
                                                              int pre_act, const half_t* skip, half_t* y,
                                                              const float* __restrict__ gamma,
                                                              const float* __restrict__ beta, int C, float alpha,
                                                              float eps, uint8_t* yq, float q_mul) {
  using ev8 = typename Vec16<ET>::v8;
  __shared__ float red[4];
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int nvec = C / 8;
  [[maybe_unused]] floatx4 gm[4][2], bt[4][2];
  if constexpr (EARLY) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int v = min(tid + i * 256, nvec - 1);
      gm[i][0] = *reinterpret_cast<const floatx4*>(gamma + v * 8);
      gm[i][1] = *reinterpret_cast<const floatx4*>(gamma + v * 8 + 4);
      bt[i][0] = *reinterpret_cast<const floatx4*>(beta + v * 8);
      bt[i][1] = *reinterpret_cast<const floatx4*>(beta + v * 8 + 4);
    }
  }
  float t[4][8];
  float sum = 0.0f;
  // One switch over the activation for the kernel, not one per element.
  DispatchAct(pre_act, [&](auto act_fn) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int v = tid + i * 256;
#pragma unroll
      for (int e = 0; e < 8; e++) t[i][e] = 0.0f;
      if (v < nvec) {
        const long long off = (long long)row * C + v * 8;
        if (xf != nullptr) {
          for (int part = 0; part < n_partials; part++) {
            floatx4 a = *reinterpret_cast<const floatx4*>(xf + part * partial_stride + off);
            floatx4 b = *reinterpret_cast<const floatx4*>(xf + part * partial_stride + off + 4);
#pragma unroll
            for (int e = 0; e < 4; e++) { t[i][e] += a[e]; t[i][4 + e] += b[e]; }
          }
        } else {
          ev8 h = *reinterpret_cast<const ev8*>(xh + off);
#pragma unroll
          for (int e = 0; e < 8; e++) t[i][e] = (float)h[e];
        }
#pragma unroll
        for (int e = 0; e < 8; e++) t[i][e] = act_fn(t[i][e]) * alpha;
        if (skip != nullptr) {
          ev8 hs = *reinterpret_cast<const ev8*>(skip + off);
#pragma unroll
          for (int e = 0; e < 8; e++) t[i][e] += (float)hs[e];
        }
#pragma unroll
        for (int e = 0; e < 8; e++) sum += t[i][e];
      }
    }
  });
  sum = WaveSum(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  const float mean = (red[0] + red[1] + red[2] + red[3]) / (float)C;
  __syncthreads();
  float var = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; i++)
    if (tid + i * 256 < nvec) {
#pragma unroll
      for (int e = 0; e < 8; e++) { float d = t[i][e] - mean; var += d * d; }
    }
  var = WaveSum(var);
  if (lane == 0) red[wave] = var;
  __syncthreads();
  const float den = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)C + eps);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int v = tid + i * 256;
    if (v < nvec) {
      if constexpr (!EARLY) {
        gm[i][0] = *reinterpret_cast<const floatx4*>(gamma + v * 8);
        gm[i][1] = *reinterpret_cast<const floatx4*>(gamma + v * 8 + 4);
        bt[i][0] = *reinterpret_cast<const floatx4*>(beta + v * 8);
        bt[i][1] = *reinterpret_cast<const floatx4*>(beta + v * 8 + 4);
      }
      ev8 o;
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; e++) {
        f[e] = bt[i][e / 4][e % 4] + gm[i][e / 4][e % 4] * (t[i][e] - mean) * den;
        o[e] = (ET)f[e];
      }
      *reinterpret_cast<ev8*>(y + (long long)row * C + v * 8) = o;
      if (yq != nullptr) {   // e4m3 copy of the same row (from the float values) for a following fp8 GEMM
        uint2 q;
        q.x = PackFp8x4(f[0] * q_mul, f[1] * q_mul, f[2] * q_mul, f[3] * q_mul);
        q.y = PackFp8x4(f[4] * q_mul, f[5] * q_mul, f[6] * q_mul, f[7] * q_mul);
        *reinterpret_cast<uint2*>(yq + (long long)row * C + v * 8) = q;
      }
    }
  }
}
}  // namespace

namespace {
__global__ __launch_bounds__(256) void copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, long long n) {
  long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src[i];
}
}  // namespace

void LaunchCopy(const void* src, void* dst, long long n_vec16, hipStream_t stream) {
  if (n_vec16 <= 0) return;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)((n_vec16 + 255) / 256)), dim3(256), 0, stream,
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), n_vec16);
}

void LaunchZero(float* p, long long n, hipStream_t stream) {
  if (n <= 0) return;
  hipLaunchKernelGGL(zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, p, n);
}

void LaunchLayerNormRows(const float* x_f32, int n_partials, long long partial_stride, const half_t* x_f16,
                         int pre_act, const half_t* skip, half_t* y, const float* gamma, const float* beta, int rows,
                         int C, float alpha, float eps, hipStream_t stream, bool bf16, uint8_t* y_f8, float f8_mul) {
  if (rows <= 0) return;
  auto launch = [&](auto early_tag, auto elem_tag) {
    using ET = decltype(elem_tag);
    hipLaunchKernelGGL((layer_norm_rows_kernel<decltype(early_tag)::value, ET>), dim3(rows), dim3(256), 0, stream, x_f32,
                       n_partials, partial_stride, x_f16, pre_act, skip, y, gamma, beta, C, alpha, eps, y_f8, f8_mul);
  };
  if (bf16) {
    if (rows <= 64) launch(std::true_type{}, bf16_t{});
    else launch(std::false_type{}, bf16_t{});
  } else {
    if (rows <= 64) launch(std::true_type{}, half_t{});
    else launch(std::false_type{}, half_t{});
  }
}

void LaunchLayerNorm(const half_t* x, const half_t* skip, half_t* y, const float* gamma, const float* beta,
                     int rows, int C, float alpha, float eps, hipStream_t stream, uint8_t* y_f8, float f8_mul, bool bf16,
                     bool through) {
  if (rows <= 0) return;
  dim3 grid((rows + 3) / 4), block(256);
  auto launch = [&](auto nv_tag, auto elem_tag) {
    hipLaunchKernelGGL((layer_norm_kernel<decltype(nv_tag)::value, decltype(elem_tag)>), grid, block, 0, stream, x, skip,
                       y, y_f8, f8_mul, gamma, beta, rows, C, alpha, eps, through);
  };
  auto by_width = [&](auto elem_tag) {
    if (C <= 512) launch(std::integral_constant<int, 1>{}, elem_tag);
    else if (C <= 1024) launch(std::integral_constant<int, 2>{}, elem_tag);
    else if (C <= 2048) launch(std::integral_constant<int, 4>{}, elem_tag);
    else launch(std::integral_constant<int, 16>{}, elem_tag);   // callers guarantee C <= 8192
  };
  if (bf16) by_width(bf16_t{});
  else by_width(half_t{});
}

namespace {
// out = max(out, max |x|), as float bits (non-negative floats order like unsigned integers).
__global__ __launch_bounds__(256) void absmax_kernel(const half_t* __restrict__ x, long long nvec, unsigned* out) {
  float m = 0.0f;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (long long)gridDim.x * 256) {
    const half8 h = *reinterpret_cast<const half8*>(x + i * 8);
#pragma unroll
    for (int e = 0; e < 8; e++) m = fmaxf(m, fabsf((float)h[e]));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  if ((threadIdx.x & 63) == 0) atomicMax(out, __float_as_uint(m));
}
}  // namespace

void LaunchAbsMax(const half_t* x, long long n, float* out, hipStream_t stream) {
  const long long nvec = n / 8;
  if (nvec <= 0) return;
  const unsigned blocks = (unsigned)std::min<long long>((nvec + 255) / 256, 2048);
  hipLaunchKernelGGL(absmax_kernel, dim3(blocks), dim3(256), 0, stream, x, nvec, reinterpret_cast<unsigned*>(out));
}

void LaunchQuantizeF8(const half_t* x, uint8_t* y, long long n, float mul, hipStream_t stream) {
  if (n <= 0) return;
  const long long nvec = n / 8;
  hipLaunchKernelGGL(quantize_f8_kernel, dim3((unsigned)((nvec + 255) / 256)), dim3(256), 0, stream, x, y, nvec, mul);
}

// ---------------------------------------------------------------------------
// Fused attention for 64 tokens and head depth 32: one wave per (sample, head).
//
// S^T = K.Q^T is computed so that a lane holds, for its query column, 32 of the
// 64 key logits in registers (the other 32 live in lane^32): the softmax over
// keys is an in-register reduction plus one cross-lane exchange. The
// probabilities are then already laid out as the "A" operand of P.V.
// Key order inside one 16-key MFMA step s for lane half g and slot e:
//   key = 16 s + 8 (e / 4) + 4 g + e % 4.
// ---------------------------------------------------------------------------
namespace {
// DEPTH = head depth (32, 64 or 128); OutT = half_t, or uint8_t for e4m3 output scaled by out_mul.
// Second launch bound = waves per SIMD the register allocation must allow: the kernel is a chain of
// dependent memory phases (q/k/v loads, bias loads, stores), so resident waves are what hides latency.
// ET: half_t or bf16_t (inputs, bias and a 16-bit output, all in half_t storage).
template <int DEPTH, typename OutT, typename ET>
__global__ __launch_bounds__(256, DEPTH == 32 ? 4 : DEPTH == 64 ? 3 : 1) void attention_kernel(const half_t* __restrict__ qkv,
                                                        const half_t* __restrict__ bias,
                                                        OutT* __restrict__ out, int total_heads, int heads,
                                                        float scale, float out_mul) {
  using ev8 = typename Vec16<ET>::v8;
  constexpr int kVStride = DEPTH + 8;  // halves per key row of V in LDS
  constexpr int DT = DEPTH / 32;       // 32-wide depth tiles of the output
  __shared__ __attribute__((aligned(16))) half_t Vs[4][64 * kVStride];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int gh_raw = blockIdx.x * 4 + wave;
  const bool live = gh_raw < total_heads;
  const int gh = live ? gh_raw : total_heads - 1;
  const int b = gh / heads, h = gh - b * heads;
  const int d_model = heads * DEPTH, ld = 3 * d_model;
  const half_t* Q = qkv + (long long)b * 64 * ld + h * DEPTH;
  const half_t* Kp = Q + d_model;
  const half_t* V = Q + 2 * d_model;
  const int r = lane & 31, g = lane >> 5;

  // Stage V (64 keys x DEPTH) into this wave's LDS region.
  half_t* vs = Vs[wave];
  constexpr int VCH = DEPTH / 8;  // 16-byte chunks per key row
#pragma unroll
  for (int i = 0; i < VCH; i++) {
    int v = lane + 64 * i;
    int row = v / VCH, cv = v - row * VCH;
    *reinterpret_cast<uint4*>(&vs[row * kVStride + cv * 8]) =
        *reinterpret_cast<const uint4*>(V + (long long)row * ld + cv * 8);
  }

  floatx16 st[2][2];
#pragma unroll
  for (int mt = 0; mt < 2; mt++)
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int e = 0; e < 16; e++) st[mt][nt][e] = 0.0f;
#pragma unroll
  for (int ks = 0; ks < DEPTH / 16; ks++) {
    ev8 kf[2], qf[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
      kf[t] = *reinterpret_cast<const ev8*>(Kp + (long long)(32 * t + r) * ld + 16 * ks + 8 * g);
      qf[t] = *reinterpret_cast<const ev8*>(Q + (long long)(32 * t + r) * ld + 16 * ks + 8 * g);
    }
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int nt = 0; nt < 2; nt++)
        st[mt][nt] = Mfma32(kf[mt], qf[nt], st[mt][nt]);
  }

  // Scale, add the smolgen logits, softmax over keys per query column.
  const half_t* bh = bias ? bias + (long long)gh * 4096 : nullptr;
#pragma unroll
  for (int nt = 0; nt < 2; nt++) {
    float mx = -3.0e38f;
#pragma unroll
    for (int mt = 0; mt < 2; mt++) {
#pragma unroll
      for (int bp = 0; bp < 2; bp++) {
        ev8 bv = {0, 0, 0, 0, 0, 0, 0, 0};
        if (bh) bv = *reinterpret_cast<const ev8*>(bh + ((nt * 2 + mt) * 2 + bp) * 512 + lane * 8);
#pragma unroll
        for (int e = 0; e < 8; e++) {
          float s = st[mt][nt][bp * 8 + e] * scale + (float)bv[e];
          st[mt][nt][bp * 8 + e] = s;
          mx = fmaxf(mx, s);
        }
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    float sum = 0.0f;
    const float kLog2e = 1.44269504f, neg_mx = -mx * kLog2e;
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        float ev = __builtin_amdgcn_exp2f(__builtin_fmaf(st[mt][nt][e], kLog2e, neg_mx));  // e^(s - mx)
        st[mt][nt][e] = ev;
        sum += ev;
      }
    sum += __shfl_xor(sum, 32, 64);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int e = 0; e < 16; e++) st[mt][nt][e] *= inv;
  }

  __syncthreads();  // V tile visible (each wave reads only its own region)

  floatx16 o[2][DT];
#pragma unroll
  for (int nt = 0; nt < 2; nt++)
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int e = 0; e < 16; e++) o[nt][dt][e] = 0.0f;
#pragma unroll
  for (int s = 0; s < 4; s++) {
    ev8 pf[2];
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int e = 0; e < 8; e++) pf[nt][e] = (ET)st[s / 2][nt][8 * (s % 2) + e];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      ev8 vf;
#pragma unroll
      for (int e = 0; e < 8; e++) vf[e] = __builtin_bit_cast(ET, vs[(16 * s + 8 * (e / 4) + 4 * g + (e % 4)) * kVStride + dt * 32 + r]);
#pragma unroll
      for (int nt = 0; nt < 2; nt++) o[nt][dt] = Mfma32(pf[nt], vf, o[nt][dt]);
    }
  }
  if (!live) return;
  // The accumulator layout would store 2 bytes per lane; go through this wave's LDS region (V is consumed)
  // so that the global stores are 16 bytes per lane and cover whole rows of the head.
  constexpr int kRowBytes = DEPTH * (int)sizeof(OutT);
  constexpr int kOStride = kRowBytes + 16;  // bytes per query row in LDS
  constexpr int kChunksPerRow = kRowBytes / 16;
  static_assert(64 * kOStride <= 64 * kVStride * (int)sizeof(half_t), "output staging fits the V region");
  unsigned char* os = reinterpret_cast<unsigned char*>(vs);
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int nt = 0; nt < 2; nt++)
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int q = 32 * nt + 8 * (e / 4) + 4 * g + (e % 4);
        OutT* dst = reinterpret_cast<OutT*>(os + q * kOStride) + dt * 32 + r;
        if constexpr (sizeof(OutT) == 1) {
          *dst = (uint8_t)(PackFp8x4(o[nt][dt][e] * out_mul, 0.0f, 0.0f, 0.0f) & 0xffu);
        } else {
          *dst = __builtin_bit_cast(OutT, (ET)o[nt][dt][e]);
        }
      }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the region is private to this wave
  __builtin_amdgcn_wave_barrier();
  unsigned char* O = reinterpret_cast<unsigned char*>(out + (long long)b * 64 * d_model + h * DEPTH);
  const long long o_row_bytes = (long long)d_model * (long long)sizeof(OutT);
#pragma unroll
  for (int i = 0; i < kChunksPerRow; i++) {
    const int idx = i * 64 + lane;
    const int q = idx / kChunksPerRow, c = idx - q * kChunksPerRow;
    *reinterpret_cast<uint4*>(O + q * o_row_bytes + c * 16) = *reinterpret_cast<const uint4*>(os + q * kOStride + c * 16);
  }
}
}  // namespace

__host__ __device__ int SmolgenBiasIndex(int q, int k) {
  int nt = q / 32, r = q % 32, mt = k / 32, kk = k % 32;
  int blk = kk / 8, g = (kk % 8) / 4, j = kk % 4;
  int lane = g * 32 + r;
  return ((nt * 2 + mt) * 2 + blk / 2) * 512 + lane * 8 + (blk % 2) * 4 + j;
}

namespace {
template <typename OutT>
void LaunchAttentionT(const half_t* qkv, const half_t* bias, OutT* out, float out_mul, int batch, int heads, int depth,
                      float scale, hipStream_t stream, bool bf16 = false) {
  const int total = batch * heads;
  if (total <= 0) return;
  const dim3 grid((total + 3) / 4), block(256);
  auto launch = [&](auto depth_tag, auto elem_tag) {
    hipLaunchKernelGGL((attention_kernel<decltype(depth_tag)::value, OutT, decltype(elem_tag)>), grid, block, 0, stream, qkv,
                       bias, out, total, heads, scale, out_mul);
  };
  auto by_depth = [&](auto elem_tag) {
    switch (depth) {
      case 32: launch(std::integral_constant<int, 32>{}, elem_tag); break;
      case 64: launch(std::integral_constant<int, 64>{}, elem_tag); break;
      default: launch(std::integral_constant<int, 128>{}, elem_tag); break;   // 128; callers check the depth
    }
  };
  if constexpr (sizeof(OutT) == 2) {
    if (bf16) return by_depth(bf16_t{});
  }
  by_depth(half_t{});
}
}  // namespace

bool AttentionDepthSupported(int depth) { return depth == 32 || depth == 64 || depth == 128; }

void LaunchAttention(const half_t* qkv, const half_t* bias, half_t* out, int batch, int heads, float scale,
                     hipStream_t stream, int depth, bool bf16) {
  LaunchAttentionT<half_t>(qkv, bias, out, 1.0f, batch, heads, depth, scale, stream, bf16);
}

void LaunchAttentionF8Out(const half_t* qkv, const half_t* bias, uint8_t* out, float out_mul, int batch, int heads,
                          float scale, hipStream_t stream, int depth) {
  LaunchAttentionT<uint8_t>(qkv, bias, out, out_mul, batch, heads, depth, scale, stream);
}

// ---------------------------------------------------------------------------
// Attention policy tail.
// ---------------------------------------------------------------------------
namespace {
template <typename T>   // element type of kq: half_t, bf16_t or float
__global__ __launch_bounds__(256) void attn_policy_gather_kernel(const float* __restrict__ logits,
                                                                 const T* __restrict__ kq, int ld_kq,
                                                                 int key_off, const float* __restrict__ ppo, int pd,
                                                                 const int16_t* __restrict__ inv_map,
                                                                 float* __restrict__ out) {
  __shared__ float off[4][8];
  const int b = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // Promotion offsets off[i][j] = key row (56 + j) . ppo row i: wave i takes ppo row i against all eight keys,
  // with the loads of the eight products in flight together.
  {
    const int i = wave;
    const T* krow = kq + (long long)(b * 64 + 56) * ld_kq + key_off;
    float s[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    bool done = false;
    if constexpr (sizeof(T) == 2) {
      if (((pd | ld_kq | key_off) & 7) == 0) {
        done = true;
      for (int c = lane; c < pd / 8; c += 64) {
        const floatx4 p0 = *reinterpret_cast<const floatx4*>(ppo + (long long)i * pd + c * 8);
        const floatx4 p1 = *reinterpret_cast<const floatx4*>(ppo + (long long)i * pd + c * 8 + 4);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const auto kv = *reinterpret_cast<const typename Vec16<T>::v8*>(krow + (long long)j * ld_kq + c * 8);
#pragma unroll
          for (int e = 0; e < 4; e++) s[j] += (float)kv[e] * p0[e] + (float)kv[4 + e] * p1[e];
        }
      }
      }
    }
    if (!done) {
      for (int k = lane; k < pd; k += 64) {
        const float pw = ppo[(long long)i * pd + k];
#pragma unroll
        for (int j = 0; j < 8; j++) s[j] += (float)krow[(long long)j * ld_kq + k] * pw;
      }
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float t = WaveSum(s[j]);
      if (lane == 0) off[i][j] = t;
    }
  }
  __syncthreads();
  const float* lg = logits + (long long)b * 4096;
  for (int o = threadIdx.x; o < 1858; o += 256) {
    int src = inv_map[o];
    float v;
    if (src < 4096) {
      v = lg[src];
    } else {
      int q = src - 4096;
      int k = q / 24, j = (q % 24) / 3, pc = q % 3;
      v = lg[(48 + k) * 64 + 56 + j] + off[pc][j] + off[3][j];
    }
    out[(long long)b * 1858 + o] = v;
  }
}
}  // namespace

template <typename T>
void LaunchAttnPolicyGather(const float* logits, const T* kq, int ld_kq, int key_off, const float* ppo, int pd,
                            const int16_t* inv_map, float* out, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  hipLaunchKernelGGL(attn_policy_gather_kernel<T>, dim3(batch), dim3(256), 0, stream, logits, kq, ld_kq, key_off, ppo,
                     pd, inv_map, out);
}
template void LaunchAttnPolicyGather<half_t>(const float*, const half_t*, int, int, const float*, int, const int16_t*,
                                             float*, int, hipStream_t);
template void LaunchAttnPolicyGather<bf16_t>(const float*, const bf16_t*, int, int, const float*, int, const int16_t*,
                                             float*, int, hipStream_t);
template void LaunchAttnPolicyGather<float>(const float*, const float*, int, int, const float*, int, const int16_t*,
                                            float*, int, hipStream_t);

// ---------------------------------------------------------------------------
// Layer norm and attention for any element type and any row length / head depth: the forms the float
// configuration runs on, and what 16-bit networks fall back to for shapes the tuned kernels above do not take
// (LayerNorm2DWithSkipConnection, blas/encoder.h:29-66; per-head attention, blas/network_blas.cc:352-439).
// Plain vector-ALU arithmetic in float; written for generality, not for speed.
// ---------------------------------------------------------------------------
namespace {
// One workgroup per row: y = beta + gamma * (t - mean) / sqrt(var + eps), t = act(x) * alpha + skip.
template <typename T>
__global__ __launch_bounds__(256) void layer_norm_generic_kernel(const T* __restrict__ x, const T* skip, T* y,
                                                                 const float* __restrict__ gamma,
                                                                 const float* __restrict__ beta, int C, float alpha,
                                                                 float eps, int pre_act) {
  __shared__ float red[4];
  const long long row = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* xr = x + row * C;
  const T* sr = skip != nullptr ? skip + row * C : nullptr;
  auto value = [&](int c) {
    const float t = Activate((float)xr[c], pre_act) * alpha;
    return sr != nullptr ? t + (float)sr[c] : t;
  };
  float sum = 0.0f;
  for (int c = tid; c < C; c += 256) sum += value(c);
  sum = WaveSum(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  const float mean = (red[0] + red[1] + red[2] + red[3]) / (float)C;
  __syncthreads();
  float var = 0.0f;
  for (int c = tid; c < C; c += 256) {
    const float d = value(c) - mean;
    var += d * d;
  }
  var = WaveSum(var);
  if (lane == 0) red[wave] = var;
  __syncthreads();
  const float den = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)C + eps);
  // (x, skip and y may alias: every element is read for the last time by the thread that writes it)
  for (int c = tid; c < C; c += 256) y[row * C + c] = (T)(beta[c] + gamma[c] * (value(c) - mean) * den);
}

// One workgroup per (sample, head): Q, K, V of the head in LDS as floats, the 64 x 64 scores in LDS, softmax by
// rows, then P.V. MAXD bounds the head depth (LDS: 64 x (3 MAXD + 66) floats).
template <typename T, int MAXD>
__global__ __launch_bounds__(256) void attention_generic_kernel(const T* __restrict__ qkv, const T* __restrict__ bias,
                                                                T* __restrict__ out, int heads, int depth,
                                                                float scale) {
  constexpr int LD = MAXD + 1;
  __shared__ float Qs[64 * LD], Ks[64 * LD], Vs[64 * MAXD], S[64 * 65];
  const int gh = blockIdx.x, b = gh / heads, h = gh - b * heads;
  const int d_model = heads * depth, ld = 3 * d_model;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* base = qkv + (long long)b * 64 * ld + h * depth;
  for (int i = tid; i < 64 * depth; i += 256) {
    const int row = i / depth, d = i - row * depth;
    const T* src = base + (long long)row * ld + d;
    Qs[row * LD + d] = (float)src[0];
    Ks[row * LD + d] = (float)src[d_model];
    Vs[row * MAXD + d] = (float)src[2 * d_model];
  }
  __syncthreads();
  const T* bh = bias != nullptr ? bias + (long long)gh * 4096 : nullptr;
  for (int i = tid; i < 4096; i += 256) {
    const int q = i >> 6, k = i & 63;
    float acc = 0.0f;
    for (int d = 0; d < depth; d++) acc = fmaf(Qs[q * LD + d], Ks[k * LD + d], acc);
    acc *= scale;
    if (bh != nullptr) acc += (float)bh[SmolgenBiasIndex(q, k)];
    S[q * 65 + k] = acc;
  }
  __syncthreads();
  for (int q = wave; q < 64; q += 4) {   // lane = key
    const float v = S[q * 65 + lane];
    float mx = v;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    const float e = expf(v - mx);
    const float sum = WaveSum(e);
    S[q * 65 + lane] = e / sum;
  }
  __syncthreads();
  T* ob = out + (long long)b * 64 * d_model + h * depth;
  for (int i = tid; i < 64 * depth; i += 256) {
    const int q = i / depth, d = i - q * depth;
    float acc = 0.0f;
    for (int k = 0; k < 64; k++) acc = fmaf(S[q * 65 + k], Vs[k * MAXD + d], acc);
    ob[(long long)q * d_model + d] = (T)acc;
  }
}
}  // namespace

template <typename T>
void LaunchLayerNormGeneric(const T* x, const T* skip, T* y, const float* gamma, const float* beta, int rows, int C,
                            float alpha, float eps, int pre_act, hipStream_t stream) {
  if (rows <= 0) return;
  hipLaunchKernelGGL(layer_norm_generic_kernel<T>, dim3(rows), dim3(256), 0, stream, x, skip, y, gamma, beta, C, alpha,
                     eps, pre_act);
}

bool AttentionGenericDepthSupported(int depth) { return depth >= 1 && depth <= 128; }

template <typename T>
void LaunchAttentionGeneric(const T* qkv, const T* bias, T* out, int batch, int heads, int depth, float scale,
                            hipStream_t stream) {
  if (batch * heads <= 0) return;
  if (!AttentionGenericDepthSupported(depth)) throw std::runtime_error("LaunchAttentionGeneric: head depth above 128");
  const dim3 grid(batch * heads), block(256);
  if (depth <= 32) {
    hipLaunchKernelGGL((attention_generic_kernel<T, 32>), grid, block, 0, stream, qkv, bias, out, heads, depth, scale);
  } else if (depth <= 64) {
    hipLaunchKernelGGL((attention_generic_kernel<T, 64>), grid, block, 0, stream, qkv, bias, out, heads, depth, scale);
  } else {
    hipLaunchKernelGGL((attention_generic_kernel<T, 128>), grid, block, 0, stream, qkv, bias, out, heads, depth, scale);
  }
}
#define LC0MI_INSTANTIATE_GENERIC(T)                                                                                   \
  template void LaunchLayerNormGeneric<T>(const T*, const T*, T*, const float*, const float*, int, int, float, float, \
                                          int, hipStream_t);                                                          \
  template void LaunchAttentionGeneric<T>(const T*, const T*, T*, int, int, int, float, hipStream_t);
LC0MI_INSTANTIATE_GENERIC(half_t)
LC0MI_INSTANTIATE_GENERIC(bf16_t)
LC0MI_INSTANTIATE_GENERIC(float)
#undef LC0MI_INSTANTIATE_GENERIC

// ---------------------------------------------------------------------------
// Policy softmax over the legal moves of every sample: what lc0's search wrapper does on the host
// with the 1858 downloaded logits (NetworkAsBackendComputation::SoftmaxPolicy, src/neural/wrapper.cc:135-156,
// with FastExp of src/utils/fastmath.h:59-86), done here so that only the probabilities of the legal moves
// leave the device. Every float operation is a separately rounded IEEE operation in the reference's order
// (no fused multiply-add, the total is accumulated move by move by one lane).
// ---------------------------------------------------------------------------
namespace {
// 2^a for a <= 0 as a quadratic in the fractional part, exponent added to the float's bits.
// Contraction is switched off for the plain operators of these two functions: a fused multiply-add
// rounds once where the reference rounds twice.
__device__ __forceinline__ float FastExp2Ref(float a) {
#pragma clang fp contract(off)
  int e;
  if (a < 0.0f) {
    if (a < -126.0f) return 0.0f;
    e = (int)(a - 1.0f);   // truncation of a - 1 stands in for floor(a)
  } else {
    e = (int)a;
  }
  float out = a - (float)e;
  const float inner = 0.33976606f * out;
  const float lin = 0.6602339f + inner;
  const float prod = out * lin;
  out = 1.0f + prod;
  return __int_as_float(__float_as_int(out) + (int)((unsigned)e << 23));
}

__global__ __launch_bounds__(64) void legal_softmax_kernel(const float* __restrict__ policy,
                                                          const int* __restrict__ offsets,
                                                          const uint16_t* __restrict__ ids, float inv_temperature,
                                                          float* __restrict__ probs) {
#pragma clang fp contract(off)
  __shared__ float vals[kMaxLegalMoves];
  __shared__ float scale_s;
  const int b = blockIdx.x, lane = threadIdx.x;
  const int start = offsets[b], n = offsets[b + 1] - start;
  const float* row = policy + (long long)b * 1858;
  constexpr int kPerLane = kMaxLegalMoves / 64;
  float v[kPerLane];
  float mx = -__builtin_inff();
#pragma unroll
  for (int j = 0; j < kPerLane; j++) {
    const int i = lane + 64 * j;
    v[j] = i < n ? row[ids[start + i]] : -__builtin_inff();
    mx = fmaxf(mx, v[j]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
#pragma unroll
  for (int j = 0; j < kPerLane; j++) {
    const int i = lane + 64 * j;
    if (i < n) {
      const float scaled = (v[j] - mx) * inv_temperature;
      vals[i] = FastExp2Ref(1.442695040f * scaled);
    }
  }
  __syncthreads();
  if (lane == 0) {
    float total = 0.0f;
    for (int i = 0; i < n; i++) total = total + vals[i];
    scale_s = total > 0.0f ? 1.0f / total : 1.0f;
  }
  __syncthreads();
  const float scale = scale_s;
#pragma unroll
  for (int j = 0; j < kPerLane; j++) {
    const int i = lane + 64 * j;
    if (i < n) probs[start + i] = vals[i] * scale;
  }
}
}  // namespace

void LaunchLegalSoftmax(const float* policy, const int* offsets, const uint16_t* ids, float inv_temperature,
                        float* probs, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  hipLaunchKernelGGL(legal_softmax_kernel, dim3(batch), dim3(64), 0, stream, policy, offsets, ids, inv_temperature,
                     probs);
}

}  // namespace lc0mi
