// gfx950 kernels of the SE-ResNet tower (bandwidth-bound parts; the 36 batched
// GEMMs of each convolution run on the GEMM kernels of kernels.hip).
//
// What each kernel replaces in the reference CPU backend (file:line):
//   winograd_input_transform    WinogradConvolution3::TransformIn   blas/winograd_convolution3.cc:59-166
//   winograd_output_transform   TransformOut + BiasActivate / BiasResidual / ApplySEUnit
//                               blas/winograd_convolution3.cc:256-324, shared/activation.cc:166-267,
//                               blas/se_unit.cc:31-91
//   WinogradFilterTransform4x4  WinogradFilterTransformF            shared/winograd_filter.cc:54-90
//   conv_policy_gather          kConvPolicyMap gather               blas/network_blas.cc:931-942
// The reference uses F(2x2,3x3); this backend uses F(4x4,3x3) (4 tiles per board
// instead of 16): the same convolution with 2.25x fewer multiplications.
#include "kernels.h"

namespace lc0mi {
namespace {

__device__ __forceinline__ float RActivate(float v, int act) {
  switch (act) {
    case 1: {  // mish = v * n / (n + 2), n = e^v (e^v + 2); exponent clamped where the ratio rounds to 1
      const float e = __expf(__builtin_fminf(v, 20.0f));
      const float n = e * (e + 2.0f);
      return v * n * __builtin_amdgcn_rcpf(n + 2.0f);
    }
    case 2: return v > 0.0f ? v : 0.0f;
    case 4: return tanhf(v);
    case 5: return __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    case 6: return v > 0.0f ? 1.05070098f * v : 1.05070098f * 1.67326324f * (__expf(v) - 1.0f);
    case 7: return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    case 8: return v > 0.0f ? v * v : 0.0f;
    default: return v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void expand_planes_nhwc_kernel(const uint64_t* __restrict__ masks,
                                                                 const float* __restrict__ values,
                                                                 T* __restrict__ out) {
  const int b = blockIdx.x;
  __shared__ uint64_t smask[112];
  __shared__ float sval[112];
  if (threadIdx.x < 112) {
    smask[threadIdx.x] = masks[(long long)b * 112 + threadIdx.x];
    sval[threadIdx.x] = values[(long long)b * 112 + threadIdx.x];
  }
  __syncthreads();
  T* o = out + (long long)b * 64 * 112;
  for (int i = threadIdx.x; i < 64 * 112; i += 256) {
    int sq = i / 112, c = i - sq * 112;
    o[i] = ((smask[c] >> sq) & 1ull) ? (T)sval[c] : (T)0.0f;
  }
}

// One thread per (sample, tile, channel); channels are the fastest index so that
// loads and stores of neighbouring threads are contiguous.
template <typename T>
__global__ __launch_bounds__(256) void winograd_input_transform_kernel(const T* __restrict__ x, T* __restrict__ v,
                                                                       int batch, int C, int ldv) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  const int bt = blockIdx.y;  // b * 4 + tile
  if (c >= ldv) return;
  if (c >= C) {   // padding columns of a row longer than C: zeros, so that the GEMM may reduce over ldv
#pragma unroll
    for (int k = 0; k < 36; k++) v[((long long)k * batch * 4 + bt) * ldv + c] = (T)0.0f;
    return;
  }
  const int b = bt >> 2, tile = bt & 3;
  const int y0 = (tile >> 1) * 4 - 1, x0 = (tile & 1) * 4 - 1;
  const T* xb = x + (long long)b * 64 * C + c;
  float d[6][6];
#pragma unroll
  for (int i = 0; i < 6; i++)
#pragma unroll
    for (int j = 0; j < 6; j++) {
      const int yy = y0 + i, xx = x0 + j;
      d[i][j] = (yy >= 0 && yy < 8 && xx >= 0 && xx < 8) ? (float)xb[(long long)(yy * 8 + xx) * C] : 0.0f;
    }
  // t = B^T d (rows), then v = t B (columns); B^T rows scaled by 1/(4,6,6,24,24,1).
  float t[6][6];
#pragma unroll
  for (int j = 0; j < 6; j++) {
    const float d0 = d[0][j], d1 = d[1][j], d2 = d[2][j], d3 = d[3][j], d4 = d[4][j], d5 = d[5][j];
    t[0][j] = d0 - 1.25f * d2 + 0.25f * d4;
    t[1][j] = (-4.0f * (d1 + d2) + d3 + d4) * (1.0f / 6.0f);
    t[2][j] = (4.0f * (d1 - d2) - d3 + d4) * (1.0f / 6.0f);
    t[3][j] = (-2.0f * d1 - d2 + 2.0f * d3 + d4) * (1.0f / 24.0f);
    t[4][j] = (2.0f * d1 - d2 - 2.0f * d3 + d4) * (1.0f / 24.0f);
    t[5][j] = 4.0f * d1 - 5.0f * d3 + d5;
  }
  T* vo = v + (long long)bt * ldv + c;
  const long long kstride = (long long)batch * 4 * ldv;
#pragma unroll
  for (int i = 0; i < 6; i++) {
    const float t0 = t[i][0], t1 = t[i][1], t2 = t[i][2], t3 = t[i][3], t4 = t[i][4], t5 = t[i][5];
    float r[6];
    r[0] = t0 - 1.25f * t2 + 0.25f * t4;
    r[1] = (-4.0f * (t1 + t2) + t3 + t4) * (1.0f / 6.0f);
    r[2] = (4.0f * (t1 - t2) - t3 + t4) * (1.0f / 6.0f);
    r[3] = (-2.0f * t1 - t2 + 2.0f * t3 + t4) * (1.0f / 24.0f);
    r[4] = (2.0f * t1 - t2 - 2.0f * t3 + t4) * (1.0f / 24.0f);
    r[5] = 4.0f * t1 - 5.0f * t3 + t5;
#pragma unroll
    for (int j = 0; j < 6; j++) vo[(long long)(i * 6 + j) * kstride] = (T)r[j];
  }
}

// One workgroup per sample, one thread per channel (channels beyond blockDim loop).
// Shared memory: pool[C] | hidden[K] floats.
template <typename T, typename MT>
__global__ void winograd_output_transform_kernel(const MT* __restrict__ m, const float* __restrict__ bias,
                                                 const T* skip, const float* __restrict__ se_w1,
                                                 const float* __restrict__ se_b1,
                                                 const float* __restrict__ se_w2,
                                                 const float* __restrict__ se_b2, int se_k, T* out, int batch,
                                                 int C, int act) {
  extern __shared__ float shm[];
  float* pool = shm;
  float* hidden = shm + C;
  const int b = blockIdx.x;
  const int c = threadIdx.x;  // blockDim.x == C (C <= 1024)
  const long long kstride = (long long)batch * 4 * C;
  float y[64];
  float sum = 0.0f;
#pragma unroll
  for (int tile = 0; tile < 4; tile++) {
    const MT* mp = m + (long long)(b * 4 + tile) * C + c;
    // s = A^T mm (4x6), then o = s A (4x4); A^T = [1 1 1 1 1 0; 0 1 -1 2 -2 0; 0 1 1 4 4 0; 0 1 -1 8 -8 1].
    float s[4][6];
#pragma unroll
    for (int j = 0; j < 6; j++) {
      const float m0 = (float)mp[(long long)(0 * 6 + j) * kstride], m1 = (float)mp[(long long)(1 * 6 + j) * kstride];
      const float m2 = (float)mp[(long long)(2 * 6 + j) * kstride], m3 = (float)mp[(long long)(3 * 6 + j) * kstride];
      const float m4 = (float)mp[(long long)(4 * 6 + j) * kstride], m5 = (float)mp[(long long)(5 * 6 + j) * kstride];
      s[0][j] = m0 + m1 + m2 + m3 + m4;
      s[1][j] = m1 - m2 + 2.0f * (m3 - m4);
      s[2][j] = m1 + m2 + 4.0f * (m3 + m4);
      s[3][j] = m1 - m2 + 8.0f * (m3 - m4) + m5;
    }
    const int ty = (tile >> 1) * 4, tx = (tile & 1) * 4;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const float s0 = s[i][0], s1 = s[i][1], s2 = s[i][2], s3 = s[i][3], s4 = s[i][4], s5 = s[i][5];
      const float o0 = s0 + s1 + s2 + s3 + s4;
      const float o1 = s1 - s2 + 2.0f * (s3 - s4);
      const float o2 = s1 + s2 + 4.0f * (s3 + s4);
      const float o3 = s1 - s2 + 8.0f * (s3 - s4) + s5;
      y[(ty + i) * 8 + tx + 0] = o0;
      y[(ty + i) * 8 + tx + 1] = o1;
      y[(ty + i) * 8 + tx + 2] = o2;
      y[(ty + i) * 8 + tx + 3] = o3;
      sum += o0 + o1 + o2 + o3;
    }
  }
  const float bc = bias[c];
  float gamma = 1.0f, beta = bc;
  if (se_k > 0) {
    pool[c] = sum * (1.0f / 64.0f) + bc;
    __syncthreads();
    for (int k = c; k < se_k; k += blockDim.x) {
      float h = se_b1[k];
      const float* w = se_w1 + (long long)k * C;
      for (int i = 0; i < C; i++) h += w[i] * pool[i];
      hidden[k] = RActivate(h, act);
    }
    __syncthreads();
    float sg = se_b2[c], sb = se_b2[C + c];
    for (int k = 0; k < se_k; k++) {   // se_w2 is stored [K][2C]: neighbouring channels, neighbouring addresses
      sg += se_w2[(long long)k * 2 * C + c] * hidden[k];
      sb += se_w2[(long long)k * 2 * C + C + c] * hidden[k];
    }
    gamma = 1.0f / (1.0f + __expf(-sg));
    beta = sb + gamma * bc;
  }
  const T* sk = skip ? skip + (long long)b * 64 * C + c : nullptr;
  T* o = out + (long long)b * 64 * C + c;
#pragma unroll
  for (int sq = 0; sq < 64; sq++) {
    float v = gamma * y[sq] + beta;
    if (sk) v += (float)sk[(long long)sq * C];
    o[(long long)sq * C] = (T)RActivate(v, act);
  }
}

// Same for C <= 256 with four times the parallelism: one thread per (tile, channel),
// blockDim.x == 4 * C. Shared memory: part[4][C] | hidden[K] | fc2[4][2][C] floats.
// The squeeze-and-excitation layers sit on the critical path of every workgroup (nothing moves through memory while
// they run), so they are spread over all threads: every wave pools the channels it needs itself, the second layer is
// split four ways over k with the weights of a thread's share asked for at once, and every thread adds the four
// partial sums of its own channel.
template <typename T, typename MT>
// (eight waves per SIMD, i.e. two workgroups of 1024 threads per CU: at most 64 registers)
__global__ __launch_bounds__(1024, 8) void winograd_output_transform_tiles_kernel(
    const MT* __restrict__ m, const float* __restrict__ bias, const T* skip, const float* __restrict__ se_w1,
    const float* __restrict__ se_b1, const float* __restrict__ se_w2, const float* __restrict__ se_b2, int se_k,
    T* out, T* __restrict__ v_next, int ldv, int batch, int C, int act) {
  extern __shared__ float shm[];
  float* part = shm;               // [4][C], then pool[C] in its first row
  float* hidden = shm + 4 * C;     // [K]
  float* fc2 = hidden + se_k;      // [4][gamma | beta][C] partial sums of the second layer
  T* xs = reinterpret_cast<T*>(fc2 + 8 * C + ((se_k & 1) ? 1 : 0));   // [64][C] activations for the fused input transform
  const int b = blockIdx.x;
  const int tile = threadIdx.x / C, c = threadIdx.x - tile * C;
  const long long kstride = (long long)batch * 4 * C;
  const MT* mp = m + (long long)(b * 4 + tile) * C + c;
  float mm[36];
#pragma unroll
  for (int k = 0; k < 36; k++) mm[k] = (float)mp[(long long)k * kstride];
  float s[4][6];
#pragma unroll
  for (int j = 0; j < 6; j++) {
    const float m0 = mm[j], m1 = mm[6 + j], m2 = mm[12 + j], m3 = mm[18 + j], m4 = mm[24 + j], m5 = mm[30 + j];
    s[0][j] = m0 + m1 + m2 + m3 + m4;
    s[1][j] = m1 - m2 + 2.0f * (m3 - m4);
    s[2][j] = m1 + m2 + 4.0f * (m3 + m4);
    s[3][j] = m1 - m2 + 8.0f * (m3 - m4) + m5;
  }
  float y[4][4];
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const float s0 = s[i][0], s1 = s[i][1], s2 = s[i][2], s3 = s[i][3], s4 = s[i][4], s5 = s[i][5];
    y[i][0] = s0 + s1 + s2 + s3 + s4;
    y[i][1] = s1 - s2 + 2.0f * (s3 - s4);
    y[i][2] = s1 + s2 + 4.0f * (s3 + s4);
    y[i][3] = s1 - s2 + 8.0f * (s3 - s4) + s5;
    sum += y[i][0] + y[i][1] + y[i][2] + y[i][3];
  }
  const float bc = bias[c];
  float gamma = 1.0f, beta = bc;
  if (se_k > 0) {
    part[tile * C + c] = sum;
    __syncthreads();
    // hidden[k] = act(w1[k] . pool + b1[k]): one wave per k, lanes stride over the channels (pooled on the way).
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    constexpr int kMaxPerLane = 4;   // C <= 256
    float pool[kMaxPerLane];
#pragma unroll
    for (int q = 0; q < kMaxPerLane; q++) {
      const int i = lane + 64 * q;
      pool[q] = i < C ? (part[i] + part[C + i] + part[2 * C + i] + part[3 * C + i]) * (1.0f / 64.0f) + bias[i] : 0.0f;
    }
    for (int k0 = wave; k0 < se_k; k0 += 2 * nwaves) {   // two k per round: their weights are asked for together
      float w[2][kMaxPerLane];
#pragma unroll
      for (int u = 0; u < 2; u++) {
        const int k = min(k0 + u * nwaves, se_k - 1);
#pragma unroll
        for (int q = 0; q < kMaxPerLane; q++) w[u][q] = se_w1[(long long)k * C + min(lane + 64 * q, C - 1)];
      }
#pragma unroll
      for (int u = 0; u < 2; u++) {
        const int k = k0 + u * nwaves;
        float h = 0.0f;
#pragma unroll
        for (int q = 0; q < kMaxPerLane; q++) h += w[u][q] * pool[q];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) h += __shfl_xor(h, off, 64);
        if (lane == 0 && k < se_k) hidden[k] = RActivate(h + se_b1[k], act);
      }
    }
    __syncthreads();
    // Second layer: this thread's share is k = tile, tile + 4, ...
    float sg = 0.0f, sb = 0.0f;
    for (int k0 = tile; k0 < se_k; k0 += 16) {
      float wg[4], wb[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int k = min(k0 + 4 * u, se_k - 1);
        wg[u] = se_w2[(long long)k * 2 * C + c];
        wb[u] = se_w2[(long long)k * 2 * C + C + c];
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int k = k0 + 4 * u;
        const float h = k < se_k ? hidden[k] : 0.0f;
        sg += wg[u] * h;
        sb += wb[u] * h;
      }
    }
    fc2[(tile * 2) * C + c] = sg;
    fc2[(tile * 2 + 1) * C + c] = sb;
    __syncthreads();
    sg = se_b2[c] + ((fc2[c] + fc2[2 * C + c]) + (fc2[4 * C + c] + fc2[6 * C + c]));
    sb = se_b2[C + c] + ((fc2[C + c] + fc2[3 * C + c]) + (fc2[5 * C + c] + fc2[7 * C + c]));
    gamma = 1.0f / (1.0f + __expf(-sg));
    beta = sb + gamma * bc;
  }
  const int ty = (tile >> 1) * 4, tx = (tile & 1) * 4;
  const T* sk = skip ? skip + (long long)b * 64 * C + c : nullptr;
  T* o = out ? out + (long long)b * 64 * C + c : nullptr;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int sq = (ty + i) * 8 + tx + j;
      float v = gamma * y[i][j] + beta;
      if (sk) v += (float)sk[(long long)sq * C];
      const T r = (T)RActivate(v, act);
      if (o) o[(long long)sq * C] = r;
      if (v_next) xs[sq * C + c] = r;
    }
  if (!v_next) return;
  // Fused input transform of the next convolution: this thread's tile reads its 6x6
  // patch (with the halo owned by the other three tiles) from LDS.
  __syncthreads();
  const int y0 = ty - 1, x0 = tx - 1;
  float d[6][6];
#pragma unroll
  for (int i = 0; i < 6; i++)
#pragma unroll
    for (int j = 0; j < 6; j++) {
      const int yy = y0 + i, xx = x0 + j;
      d[i][j] = (yy >= 0 && yy < 8 && xx >= 0 && xx < 8) ? (float)xs[(yy * 8 + xx) * C + c] : 0.0f;
    }
  float t[6][6];
#pragma unroll
  for (int j = 0; j < 6; j++) {
    const float d0 = d[0][j], d1 = d[1][j], d2 = d[2][j], d3 = d[3][j], d4 = d[4][j], d5 = d[5][j];
    t[0][j] = d0 - 1.25f * d2 + 0.25f * d4;
    t[1][j] = (-4.0f * (d1 + d2) + d3 + d4) * (1.0f / 6.0f);
    t[2][j] = (4.0f * (d1 - d2) - d3 + d4) * (1.0f / 6.0f);
    t[3][j] = (-2.0f * d1 - d2 + 2.0f * d3 + d4) * (1.0f / 24.0f);
    t[4][j] = (2.0f * d1 - d2 - 2.0f * d3 + d4) * (1.0f / 24.0f);
    t[5][j] = 4.0f * d1 - 5.0f * d3 + d5;
  }
  T* vo = v_next + (long long)(b * 4 + tile) * ldv + c;
  const long long vstride = (long long)batch * 4 * ldv;
#pragma unroll
  for (int i = 0; i < 6; i++) {
    const float t0 = t[i][0], t1 = t[i][1], t2 = t[i][2], t3 = t[i][3], t4 = t[i][4], t5 = t[i][5];
    float r[6];
    r[0] = t0 - 1.25f * t2 + 0.25f * t4;
    r[1] = (-4.0f * (t1 + t2) + t3 + t4) * (1.0f / 6.0f);
    r[2] = (4.0f * (t1 - t2) - t3 + t4) * (1.0f / 6.0f);
    r[3] = (-2.0f * t1 - t2 + 2.0f * t3 + t4) * (1.0f / 24.0f);
    r[4] = (2.0f * t1 - t2 - 2.0f * t3 + t4) * (1.0f / 24.0f);
    r[5] = 4.0f * t1 - 5.0f * t3 + t5;
#pragma unroll
    for (int j = 0; j < 6; j++) vo[(long long)(i * 6 + j) * vstride] = (T)r[j];
  }
}

template <typename T>
__global__ __launch_bounds__(256) void conv_policy_gather_kernel(const T* __restrict__ t, int ld,
                                                                 const int16_t* __restrict__ inv_map,
                                                                 float* __restrict__ out) {
  const int b = blockIdx.x;
  for (int o = threadIdx.x; o < 1858; o += 256) {
    const int src = inv_map[o];
    const int plane = src >> 6, sq = src & 63;
    out[(long long)b * 1858 + o] = (float)t[((long long)b * 64 + sq) * ld + plane];
  }
}

}  // namespace

template <typename T>
void LaunchExpandPlanesNhwc(const uint64_t* masks, const float* values, T* out, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  hipLaunchKernelGGL(expand_planes_nhwc_kernel<T>, dim3(batch), dim3(256), 0, stream, masks, values, out);
}
template void LaunchExpandPlanesNhwc<half_t>(const uint64_t*, const float*, half_t*, int, hipStream_t);
template void LaunchExpandPlanesNhwc<float>(const uint64_t*, const float*, float*, int, hipStream_t);

void WinogradFilterTransform4x4(const float* filter, int cout, int cin, int ld_cin, float* u) {
  static const float G[6][3] = {{1, 0, 0}, {-1, -1, -1}, {-1, 1, -1}, {1, 2, 4}, {1, -2, 4}, {0, 0, 1}};
  const size_t plane = (size_t)cout * ld_cin;
  for (size_t i = 0; i < 36 * plane; i++) u[i] = 0.0f;
  for (int o = 0; o < cout; o++)
    for (int c = 0; c < cin; c++) {
      const float* g = filter + ((size_t)o * cin + c) * 9;
      float tmp[6][3];
      for (int i = 0; i < 6; i++)
        for (int j = 0; j < 3; j++) tmp[i][j] = G[i][0] * g[0 * 3 + j] + G[i][1] * g[1 * 3 + j] + G[i][2] * g[2 * 3 + j];
      for (int i = 0; i < 6; i++)
        for (int j = 0; j < 6; j++)
          u[(size_t)(i * 6 + j) * plane + (size_t)o * ld_cin + c] =
              tmp[i][0] * G[j][0] + tmp[i][1] * G[j][1] + tmp[i][2] * G[j][2];
    }
}

template <typename T>
void LaunchWinogradInputTransform(const T* x, T* v, int batch, int C, int ldv, hipStream_t stream) {
  if (batch <= 0) return;
  hipLaunchKernelGGL(winograd_input_transform_kernel<T>, dim3((ldv + 255) / 256, batch * 4), dim3(256), 0, stream, x, v,
                     batch, C, ldv);
}
template void LaunchWinogradInputTransform<half_t>(const half_t*, half_t*, int, int, int, hipStream_t);
template void LaunchWinogradInputTransform<float>(const float*, float*, int, int, int, hipStream_t);

template <typename T, typename MT>
void LaunchWinogradOutputTransform(const MT* m, const float* bias, const T* skip, const float* se_w1,
                                   const float* se_b1, const float* se_w2, const float* se_b2, int se_k, T* out,
                                   int batch, int C, int act, hipStream_t stream, T* v_next, int ldv_next) {
  if (batch <= 0) return;
  const int k = se_k > 0 ? se_k : 0;
  if (C <= 256 && C % 16 == 0) {   // 4 * C threads in whole waves (the SE reduction shuffles across a wave)
    size_t shm = sizeof(float) * (size_t)(12 * C + k + (k & 1));
    if (v_next) shm += sizeof(T) * 64 * (size_t)C;
    hipLaunchKernelGGL((winograd_output_transform_tiles_kernel<T, MT>), dim3(batch), dim3(4 * C), shm, stream, m, bias,
                       skip, se_w1, se_b1, se_w2, se_b2, se_k, out, v_next, ldv_next, batch, C, act);
    return;
  }
  // Wide towers: separate kernels (the caller checks WinogradFusedInputTransform before asking for v_next).
  const size_t shm = sizeof(float) * (size_t)(C + k);
  hipLaunchKernelGGL((winograd_output_transform_kernel<T, MT>), dim3(batch), dim3(C), shm, stream, m, bias, skip,
                     se_w1, se_b1, se_w2, se_b2, se_k, out, batch, C, act);
}
// The fused kernel needs 4 * C threads and its staging area in the 64 KiB of dynamic LDS.
bool WinogradFusedInputTransform(int C, int elem_size, int se_k) {
  return C <= 256 && C % 16 == 0 && sizeof(float) * (12 * C + se_k + 1) + (size_t)elem_size * 64 * C <= 64 * 1024;
}

template void LaunchWinogradOutputTransform<half_t, half_t>(const half_t*, const float*, const half_t*, const float*,
                                                            const float*, const float*, const float*, int, half_t*,
                                                            int, int, int, hipStream_t, half_t*, int);
template void LaunchWinogradOutputTransform<half_t, float>(const float*, const float*, const half_t*, const float*,
                                                           const float*, const float*, const float*, int, half_t*, int,
                                                           int, int, hipStream_t, half_t*, int);
template void LaunchWinogradOutputTransform<float, float>(const float*, const float*, const float*, const float*,
                                                          const float*, const float*, const float*, int, float*, int,
                                                          int, int, hipStream_t, float*, int);

template <typename T>
void LaunchConvPolicyGather(const T* t, int ld, const int16_t* inv_map, float* out, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  hipLaunchKernelGGL(conv_policy_gather_kernel<T>, dim3(batch), dim3(256), 0, stream, t, ld, inv_map, out);
}
template void LaunchConvPolicyGather<half_t>(const half_t*, int, const int16_t*, float*, int, hipStream_t);
template void LaunchConvPolicyGather<float>(const float*, int, const int16_t*, float*, int, hipStream_t);

}  // namespace lc0mi
