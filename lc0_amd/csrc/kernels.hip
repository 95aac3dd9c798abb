// Hand-written gfx950 (CDNA4, wave64) kernels of the attention-body path.
//
// What each kernel replaces in the reference CPU backend (file:line):
//   gemm_kernel           FullyConnectedLayer::Forward1D  blas/fully_connected_layer.cc:49-106
//                         (+ bias/activation of shared/activation.cc:102-164) and the per-sample
//                         Q.K^T sgemm of the attention policy (blas/network_blas.cc:850-872)
//   expand_planes_*       BlasComputation::EncodePlanes + NCHW->NHWC + pos-enc concat
//                         blas/network_blas.cc:973-981, 630-652
//   layer_norm_kernel     LayerNorm2DWithSkipConnection   blas/encoder.h:29-66
//   attention_kernel      per-head QK^T, +smolgen, softmax, .V   blas/network_blas.cc:352-439
//   attn_policy_gather    promotion offsets + kAttnPolicyMap gather  blas/network_blas.cc:873-914
#include "kernels.h"

#include "device_math.h"

#include <algorithm>
#include <stdexcept>
#include <type_traits>
#include <utility>

namespace lc0mi {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx8 __attribute__((ext_vector_type(8)));

namespace {

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

// ---------------------------------------------------------------------------
// GEMM  C[m][n] = act(scale * sum_k A[m][k] W[n][k] + bias[n])
//
// 256 threads = 4 waves laid out WAVES_M x WAVES_N over a BM x BN block tile;
// each wave owns (BM/WAVES_M) x (BN/WAVES_N) as 32x32 MFMA tiles
// (v_mfma_f32_32x32x16_f16). The weight rows are the MFMA "A" operand and the
// activation rows the "B" operand, so a lane ends up holding 4 consecutive n
// for one m and stores 8 bytes at a time. Global tiles are fetched as 16-byte
// vectors into registers one k-tile ahead and staged through padded LDS.
// ---------------------------------------------------------------------------
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, typename OutT>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs p) {
  static_assert(WAVES_M * WAVES_N == 4, "four waves per block");
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int LDS_STRIDE = BK + 8;  // halves; 16-byte rows shifted by 4 banks per row
  constexpr int VEC_PER_ROW = BK / 8;
  constexpr int A_VECS = BM * VEC_PER_ROW / 256;
  constexpr int W_VECS = BN * VEC_PER_ROW / 256;
  static_assert(A_VECS >= 1 && W_VECS >= 1, "tile too small for 256 threads");

  __shared__ __attribute__((aligned(16))) half_t As[BM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) half_t Ws[BN * LDS_STRIDE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;
  const int zb = blockIdx.z / p.split_k, zs = blockIdx.z - zb * p.split_k;
  const half_t* A = p.A + (long long)zb * p.strideA;
  const half_t* W = p.W + (long long)zb * p.strideW;
  const int M = p.M, N = p.N;
  // This workgroup's slice of the reduction dimension.
  const int k_slice = ((p.K + p.split_k - 1) / p.split_k + BK - 1) / BK * BK;
  const int k_begin = zs * k_slice;
  const int K = min(p.K, k_begin + k_slice);

  uint4 ra[A_VECS], rw[W_VECS];
  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_VECS; i++) {
      int v = tid + i * 256;
      int row = v / VEC_PER_ROW, kv = v % VEC_PER_ROW;
      int gm = min(m0 + row, M - 1), k = k0 + kv * 8;
      ra[i] = k < K ? *reinterpret_cast<const uint4*>(A + (long long)gm * p.lda + k) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < W_VECS; i++) {
      int v = tid + i * 256;
      int row = v / VEC_PER_ROW, kv = v % VEC_PER_ROW;
      int gn = min(n0 + row, N - 1), k = k0 + kv * 8;
      rw[i] = k < K ? *reinterpret_cast<const uint4*>(W + (long long)gn * p.ldw + k) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < A_VECS; i++) {
      int v = tid + i * 256;
      int row = v / VEC_PER_ROW, kv = v % VEC_PER_ROW;
      *reinterpret_cast<uint4*>(&As[row * LDS_STRIDE + kv * 8]) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < W_VECS; i++) {
      int v = tid + i * 256;
      int row = v / VEC_PER_ROW, kv = v % VEC_PER_ROW;
      *reinterpret_cast<uint4*>(&Ws[row * LDS_STRIDE + kv * 8]) = rw[i];
    }
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

  const int nk = K > k_begin ? (K - k_begin + BK - 1) / BK : 0;
  const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
  if (nk > 0) load_tile(k_begin);
  for (int kt = 0; kt < nk; kt++) {
    store_tile();
    __syncthreads();
    if (kt + 1 < nk) load_tile(k_begin + (kt + 1) * BK);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      half8 af[TM], wf[TN];
#pragma unroll
      for (int i = 0; i < TM; i++)
        af[i] = *reinterpret_cast<const half8*>(&As[(wm * WM + i * 32 + frag_row) * LDS_STRIDE + ks * 16 + frag_k]);
#pragma unroll
      for (int j = 0; j < TN; j++)
        wf[j] = *reinterpret_cast<const half8*>(&Ws[(wn * WN + j * 32 + frag_row) * LDS_STRIDE + ks * 16 + frag_k]);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[j], af[i], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }

  // Epilogue. Accumulator element e of a tile: n = 8*(e/4) + 4*(lane/32) + e%4, m = lane%32.
  OutT* C = reinterpret_cast<OutT*>(p.C) + (long long)zb * p.strideC;
  if constexpr (sizeof(OutT) == 4) {
    if (p.split_k > 1) {
      // Every slice stores its own partial sums (no atomics: the consumer adds the
      // slices in a fixed order, so results do not depend on scheduling).
      C += (long long)zs * p.split_stride;
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int blk = 0; blk < 4; blk++) {
          const int n = n0 + wn * WN + j * 32 + blk * 8 + (lane >> 5) * 4;
          float b4[4];
          LoadBias4(zs == 0 ? p.bias : nullptr, n, N, b4);
#pragma unroll
          for (int i = 0; i < TM; i++) {
            const int m = m0 + wm * WM + i * 32 + frag_row;
#pragma unroll
            for (int r = 0; r < 4; r++)
              if (m < M && n + r < N) C[(long long)m * p.ldc + n + r] = acc[i][j][blk * 4 + r] * p.scale + b4[r];
          }
        }
      return;
    }
  }
  const bool vec_ok = (p.ldc % 4 == 0);
  // Consumer side of a folded layer norm (GemmArgs::row_stats): mean and rstd of this lane's rows.
  float row_mean[TM], row_rstd[TM];
#pragma unroll
  for (int i = 0; i < TM; i++) {
    row_mean[i] = 0.0f;
    row_rstd[i] = 1.0f;
    if (p.row_stats != nullptr) {
      RowMeanRstd(p.row_stats, p.row_parts, min(m0 + wm * WM + i * 32 + frag_row, M - 1), p.norm_n, p.norm_eps,
                  row_mean[i], row_rstd[i]);
    }
  }
  DispatchAct(p.act, [&](auto act_fn) {
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
      for (int blk = 0; blk < 4; blk++) {
        const int n = n0 + wn * WN + j * 32 + blk * 8 + (lane >> 5) * 4;
        if (n >= N) continue;
        float b4[4], c4[4];
        LoadBias4(p.bias, n, N, b4);
        LoadBias4(p.row_stats != nullptr ? p.col_c : nullptr, n, N, c4);
#pragma unroll
        for (int i = 0; i < TM; i++) {
          const int m = m0 + wm * WM + i * 32 + frag_row;
          if (m >= M) continue;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; r++)
            v[r] = act_fn(row_rstd[i] * (acc[i][j][blk * 4 + r] * p.scale - row_mean[i] * c4[r]) + b4[r]);
          OutT* dst = C + (long long)m * p.ldc + n;
          if (vec_ok && n + 3 < N) {
            if constexpr (sizeof(OutT) == 2) {
              half4 h = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
              *reinterpret_cast<half4*>(dst) = h;
            } else {
              floatx4 f = {v[0], v[1], v[2], v[3]};
              *reinterpret_cast<floatx4*>(dst) = f;
            }
          } else {
#pragma unroll
            for (int r = 0; r < 4; r++)
              if (n + r < N) dst[r] = (OutT)v[r];
          }
        }
      }
    }
  });
}

// ---------------------------------------------------------------------------
// Row-panel GEMM for small problems (few rows, or few columns): a workgroup owns a
// (16 RT) x (16 CT) output panel and its eight waves split the reduction dimension, so
// even a 16 x 16 x K problem keeps eight waves busy, the serial chain is K / 256 MFMA
// steps instead of K / 32, and U steps of operand loads are in flight per wave (these
// problems are bound by memory latency and by the 64 bytes per cycle at which a CU's
// address path takes loads, not by arithmetic: the time of a launch grows with the
// RT + CT operand rows a workgroup reads, so the launcher picks the smallest panel that
// still fits the problem into one workgroup per CU). Fragments of 16x16x32 tiles go from
// global memory straight into registers, 64 bytes of a row per load instruction; the
// eight partial sums are added in wave order through LDS, so results do not depend on
// timing.
// ---------------------------------------------------------------------------
template <int RT, int CT, int U, typename OutT>
__global__ __launch_bounds__(512) void gemm_rowpanel_kernel(GemmArgs p) {
  constexpr int NW = 8, ROWS = 16 * RT, COLS = 16 * CT, LD = COLS + 1;
  __shared__ float part[NW][ROWS * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int m0 = blockIdx.x * ROWS, n0 = blockIdx.y * COLS;
  const int M = p.M, N = p.N, K = p.K;
  const half_t* A = p.A + (long long)blockIdx.z * p.strideA;
  const half_t* W = p.W + (long long)blockIdx.z * p.strideW;
  // K range of this wave, in steps of 32. A last step of 8, 16 or 24 values goes to the last wave.
  const int steps = K / 32;
  const int per_wave = (steps + NW - 1) / NW;
  const int s_begin = min(steps, wave * per_wave), s_end = min(steps, s_begin + per_wave);
  const half_t* a_row[RT];
  const half_t* w_row[CT];
#pragma unroll
  for (int t = 0; t < RT; t++) a_row[t] = A + (long long)min(m0 + 16 * t + r, M - 1) * p.lda + 8 * g;
#pragma unroll
  for (int c = 0; c < CT; c++) w_row[c] = W + (long long)min(n0 + 16 * c + r, N - 1) * p.ldw + 8 * g;
  floatx4 acc[RT][CT];
#pragma unroll
  for (int t = 0; t < RT; t++)
#pragma unroll
    for (int c = 0; c < CT; c++) acc[t][c] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
  // Loads carry no predicate, so that the compiler can put the loads of U steps in flight at once.
  for (int st = s_begin; st < s_end; st += U) {
    half8 fa[RT][U], fw[CT][U];
#pragma unroll
    for (int u = 0; u < U; u++) {   // steps past the end re-read the last one (never used)
      const int k = min(st + u, s_end - 1) * 32;
#pragma unroll
      for (int t = 0; t < RT; t++) fa[t][u] = *reinterpret_cast<const half8*>(a_row[t] + k);
#pragma unroll
      for (int c = 0; c < CT; c++) fw[c][u] = *reinterpret_cast<const half8*>(w_row[c] + k);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (st + u < s_end) {
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
          for (int c = 0; c < CT; c++)
            acc[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fw[c][u], fa[t][u], acc[t][c], 0, 0, 0);
      }
    }
  }
  if (wave == NW - 1 && K % 32 != 0) {   // K is a multiple of 8: the missing part of the last step is zero-filled
    const int k = steps * 32;
    const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const bool in = k + 8 * g < K;
    half8 fa[RT], fw[CT];
#pragma unroll
    for (int t = 0; t < RT; t++) fa[t] = in ? *reinterpret_cast<const half8*>(a_row[t] + k) : zero;
#pragma unroll
    for (int c = 0; c < CT; c++) fw[c] = in ? *reinterpret_cast<const half8*>(w_row[c] + k) : zero;
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
      for (int c = 0; c < CT; c++) acc[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fw[c], fa[t], acc[t][c], 0, 0, 0);
  }
  // Accumulator lane (r, g) of tile (t, c) holds row m = 16 t + r, columns n = 16 c + 4 g + e.
  float* mine = part[wave];
#pragma unroll
  for (int t = 0; t < RT; t++)
#pragma unroll
    for (int c = 0; c < CT; c++)
#pragma unroll
      for (int e = 0; e < 4; e++) mine[(16 * t + r) * LD + 16 * c + 4 * g + e] = acc[t][c][e];
  __syncthreads();
  OutT* C = reinterpret_cast<OutT*>(p.C) + (long long)blockIdx.z * p.strideC;
  DispatchAct(p.act, [&](auto act_fn) {
#pragma unroll
    for (int i = 0; i < (ROWS * COLS + 511) / 512; i++) {
      const int idx = tid + 512 * i;        // consecutive threads along n
      const int row = idx / COLS, col = idx % COLS;
      const int m = m0 + row, n = n0 + col;
      if (row < ROWS && m < M && n < N) {
        float sum = part[0][row * LD + col];
#pragma unroll
        for (int w = 1; w < NW; w++) sum += part[w][row * LD + col];
        sum *= p.scale;
        if (p.row_stats != nullptr) {   // consumer side of a folded layer norm
          float mean, rstd;
          RowMeanRstd(p.row_stats, p.row_parts, m, p.norm_n, p.norm_eps, mean, rstd);
          sum = rstd * (sum - mean * p.col_c[n]);
        }
        const float v = act_fn(sum + (p.bias ? p.bias[n] : 0.0f));
        C[(long long)m * p.ldc + n] = (OutT)v;
      }
    }
  });
}

// The same panel scheme for e4m3 operands (v_mfma_f32_16x16x128_f8f6f4): a k-step is 128 values, a lane holds 32
// consecutive bytes of its row, so every fragment load covers sixteen full 128-byte lines.
template <int RT, int CT, int U, typename OutT>
__global__ __launch_bounds__(512) void gemm_f8_rowpanel_kernel(GemmF8Args p) {
  constexpr int NW = 8, ROWS = 16 * RT, COLS = 16 * CT, LD = COLS + 1;
  __shared__ float part[NW][ROWS * LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int m0 = blockIdx.x * ROWS, n0 = blockIdx.y * COLS;
  const int M = p.M, N = p.N;
  const int steps = p.K / 128;
  const int per_wave = (steps + NW - 1) / NW;
  const int s_begin = min(steps, wave * per_wave), s_end = min(steps, s_begin + per_wave);
  const uint8_t* a_row[RT];
  const uint8_t* w_row[CT];
#pragma unroll
  for (int t = 0; t < RT; t++) a_row[t] = p.A + (long long)min(m0 + 16 * t + r, M - 1) * p.lda + 32 * g;
#pragma unroll
  for (int c = 0; c < CT; c++) w_row[c] = p.W + (long long)min(n0 + 16 * c + r, N - 1) * p.ldw + 32 * g;
  floatx4 acc[RT][CT];
#pragma unroll
  for (int t = 0; t < RT; t++)
#pragma unroll
    for (int c = 0; c < CT; c++) acc[t][c] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
  auto load32 = [](const uint8_t* ptr) {
    const intx4 lo = *reinterpret_cast<const intx4*>(ptr);
    const intx4 hi = *reinterpret_cast<const intx4*>(ptr + 16);
    return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  for (int st = s_begin; st < s_end; st += U) {
    intx8 fa[RT][U], fw[CT][U];
#pragma unroll
    for (int u = 0; u < U; u++) {   // steps past the end re-read the last one (never used)
      const int k = min(st + u, s_end - 1) * 128;
#pragma unroll
      for (int t = 0; t < RT; t++) fa[t][u] = load32(a_row[t] + k);
#pragma unroll
      for (int c = 0; c < CT; c++) fw[c][u] = load32(w_row[c] + k);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (st + u < s_end) {
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
          for (int c = 0; c < CT; c++)
            acc[t][c] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fw[c][u], fa[t][u], acc[t][c], 0, 0, 0, 0, 0, 0);
      }
    }
  }
  float* mine = part[wave];
#pragma unroll
  for (int t = 0; t < RT; t++)
#pragma unroll
    for (int c = 0; c < CT; c++)
#pragma unroll
      for (int e = 0; e < 4; e++) mine[(16 * t + r) * LD + 16 * c + 4 * g + e] = acc[t][c][e];
  __syncthreads();
  OutT* C = reinterpret_cast<OutT*>(p.C);
  DispatchAct(p.act, [&](auto act_fn) {
#pragma unroll
    for (int i = 0; i < (ROWS * COLS + 511) / 512; i++) {
      const int idx = tid + 512 * i;        // consecutive threads along n
      const int row = idx / COLS, col = idx % COLS;
      const int m = m0 + row, n = n0 + col;
      if (row < ROWS && m < M && n < N) {
        float sum = part[0][row * LD + col];
#pragma unroll
        for (int w = 1; w < NW; w++) sum += part[w][row * LD + col];
        const float v = act_fn(sum * p.col_scale[n] + (p.bias ? p.bias[n] : 0.0f));
        if constexpr (sizeof(OutT) == 1) {
          C[(long long)m * p.ldc + n] = (uint8_t)(PackFp8x4(v * p.out_mul, 0.0f, 0.0f, 0.0f) & 0xFFu);
        } else {
          C[(long long)m * p.ldc + n] = (OutT)v;
        }
      }
    }
  });
}

// ---------------------------------------------------------------------------
// Large-shape GEMM: same contract as gemm_kernel for K % BK == 0 and half output.
//
// Operand tiles travel from global memory straight into LDS (16 bytes per lane,
// global_load_lds_dwordx4), double-buffered, with one barrier per k-tile: the
// fetch of k-tile t+1 is in flight while the MFMAs of k-tile t run, and no VGPR
// is spent on staging. One such instruction fills 1 KiB of LDS in lane order, so
// LDS rows are unpadded; the 16-byte chunk c of tile row r is stored at chunk
// slot c ^ swizzle(r), which makes the ds_read_b128 fragment reads (32 rows x
// one chunk column) hit all banks evenly. The epilogue applies scale, bias and
// activation in registers, stages 32-row strips through LDS and writes rows of
// the output as 16-byte vectors.
// ---------------------------------------------------------------------------
#define LC0MI_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// 16 bytes per lane from global memory into LDS at lds_base + lane * 16
// (lds_base must be wave-uniform). Completion is visible through vmcnt only:
// callers wait with s_waitcnt vmcnt(0) plus a barrier before reading the data.
// Two forms: inline assembly, which the compiler schedules nothing across, and the compiler's builtin, which sets M0
// itself and may be moved among the MFMAs and fragment reads of a k-tile (better for the 256-row tiles: +0.5 % of a
// pass at batch 256; worse for the small tiles: -1 % at batch 16).
template <bool BUILTIN>
__device__ __forceinline__ void DmaToLds16(const void* gptr, void* lds_base) {
  if constexpr (BUILTIN) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gptr, LC0MI_LDS_PTR(lds_base), 16,
                                     0, 0);
  } else {
    unsigned lds_addr = (unsigned)(size_t)LC0MI_LDS_PTR(lds_base);
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory", "m0");
  }
}

// The same kernel serves fp16 operands (Args = GemmArgs: BKB = 128 bytes = 64
// halves per tile row, v_mfma_f32_32x32x16_f16) and e4m3 operands (Args =
// GemmF8Args: 128 bytes = 128 values per row, v_mfma_f32_32x32x64_f8f6f4);
// BKB is the k-tile in bytes. OutT is half_t or uint8_t (e4m3, fp8 operands only).
// STREAM: the output is written with streaming (non-temporal) stores.
// EPI (fp16 operands only): 0 the plain epilogue, 1 the consumer and 2 the producer side of a folded layer norm
// (GemmArgs::row_stats / GemmArgs::skip).
// NSTAGES k-tiles of LDS: NSTAGES - 1 of them are in flight while one is consumed. Two stages suffice when the
// operands come from L2; with small tiles and operands that come from memory (a few hundred to a few thousand rows:
// every workgroup streams weights nobody has touched since the previous pass) a k-tile takes longer to arrive than
// to consume, and more stages hide that.
template <int BM, int BN, int BKB, int WAVES_M, int WAVES_N, typename Args, typename OutT, bool STREAM = false,
          int EPI = 0, int NSTAGES = 2>
// Second launch bound = waves per SIMD: with small wave tiles two workgroups share a CU
// (4 waves per SIMD, at most 128 VGPRs) and overlap each other's prologue and epilogue.
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64,
                             ((BM / WAVES_M / 32) * (BN / WAVES_N / 32) <= 4 && 2 * NSTAGES * (BM + BN) * BKB <= 160 * 1024)
                                 ? WAVES_M * WAVES_N / 2
                                 : WAVES_M * WAVES_N / 4)
void gemm_dma_kernel(Args p) {
  constexpr bool F8 = std::is_same<Args, GemmF8Args>::value;
  constexpr int ES = F8 ? 1 : 2;                  // bytes per operand element
  constexpr int NWAVES = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int CPR = BKB / 16;                   // 16-byte chunks per tile row
  constexpr int ROWS_PER_CHUNK = 64 / CPR;        // tile rows per 1 KiB transfer
  constexpr int SWZ_SHIFT = (BKB == 128) ? 1 : 2; // log2(rows per 256 bytes of LDS)
  constexpr int A_CPW = BM / ROWS_PER_CHUNK / NWAVES, W_CPW = BN / ROWS_PER_CHUNK / NWAVES;
  static_assert(BKB == 128 || BKB == 64, "k-tile must be 64 or 128 bytes");
  static_assert(F8 || sizeof(OutT) == 2, "fp8 output needs fp8 operands");
  static_assert(A_CPW >= 1 && W_CPW >= 1, "tile too small for the wave count");
  constexpr int STAGE = (BM + BN) * BKB;          // bytes
  constexpr int OV = 16 / sizeof(OutT);           // output elements per 16-byte vector
  constexpr int EPI_STRIDE = WN + OV;             // elements
  constexpr int EPI_BYTES = NWAVES * 32 * EPI_STRIDE * (int)sizeof(OutT);
  // Folded layer norm: (mean, rstd) of the tile's rows, and the producer's per-wave-column partial sums.
  constexpr int STAT_BYTES = (EPI != 0) ? BM * 8 : 0;
  constexpr int PART_BYTES = (EPI == 2) ? WAVES_N * BM * 8 : 0;
  constexpr int EPI_TOTAL = EPI_BYTES + STAT_BYTES + PART_BYTES;
  constexpr int SMEM = (NSTAGES * STAGE > EPI_TOTAL) ? NSTAGES * STAGE : EPI_TOTAL;
  static_assert(NSTAGES >= 2 && (NSTAGES - 2) * (A_CPW + W_CPW) <= 63, "transfers in flight must fit the counter");
  static_assert(EPI == 0 || (!F8 && sizeof(OutT) == 2), "folded layer norm: fp16 operands and output");
  // The tile's bias (and per-column scale, fp8 operands) waits in LDS behind the stages: fetched with the first k-tile,
  // so that the epilogue does not start with a round trip to memory.
  constexpr int COLV_BYTES = (F8 ? 2 : 1) * BN * 4;
  __shared__ __attribute__((aligned(1024))) char smem[SMEM + COLV_BYTES];
  float* colv = reinterpret_cast<float*>(smem + SMEM);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;
  const int M = p.M, N = p.N, K = p.K;
  float my_bias = 0.0f;
  [[maybe_unused]] float my_cscale = 0.0f;
  if (tid < BN && n0 + tid < N) {
    if (p.bias != nullptr) my_bias = p.bias[n0 + tid];
    if constexpr (F8) my_cscale = p.col_scale[n0 + tid];
  }
  const char* A = reinterpret_cast<const char*>(p.A);
  const char* W = reinterpret_cast<const char*>(p.W);
  if constexpr (!F8) {
    A += (long long)blockIdx.z * p.strideA * ES;
    W += (long long)blockIdx.z * p.strideW * ES;
  }

  const char* a_ptr[A_CPW];
  const char* w_ptr[W_CPW];
#pragma unroll
  for (int i = 0; i < A_CPW; i++) {
    const int row = (wave * A_CPW + i) * ROWS_PER_CHUNK + lane / CPR;
    const int c = (lane % CPR) ^ ((row >> SWZ_SHIFT) % CPR);
    a_ptr[i] = A + (long long)min(m0 + row, M - 1) * p.lda * ES + c * 16;
  }
#pragma unroll
  for (int i = 0; i < W_CPW; i++) {
    const int row = (wave * W_CPW + i) * ROWS_PER_CHUNK + lane / CPR;
    const int c = (lane % CPR) ^ ((row >> SWZ_SHIFT) % CPR);
    w_ptr[i] = W + (long long)min(n0 + row, N - 1) * p.ldw * ES + c * 16;
  }
  auto issue = [&](char* As, char* Ws, int kbyte) {
#pragma unroll
    for (int i = 0; i < A_CPW; i++) DmaToLds16<BM == 256>(a_ptr[i] + kbyte, As + (wave * A_CPW + i) * 1024);
#pragma unroll
    for (int i = 0; i < W_CPW; i++) DmaToLds16<BM == 256>(w_ptr[i] + kbyte, Ws + (wave * W_CPW + i) * 1024);
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

  const int r = lane & 31, g = lane >> 5;
  const int swz = (r >> SWZ_SHIFT) % CPR;
  const int a_row = (wm * WM + r) * BKB, w_row = (wn * WN + r) * BKB;

  const int nk = K * ES / BKB;
  issue(smem, smem + BM * BKB, 0);
#pragma unroll
  for (int st = 1; st < NSTAGES - 1; st++) {
    if (st < nk) issue(smem + st * STAGE, smem + st * STAGE + BM * BKB, st * BKB);
  }
  if (tid < BN) {
    colv[tid] = my_bias;
    if constexpr (F8) colv[BN + tid] = my_cscale;
  }
  // Folded layer norm: (mean, rstd) of tile row `tid` (of the A operand for a consumer, of the residual for a
  // producer), fetched while the first k-tile is on its way and kept in two registers until the epilogue.
  [[maybe_unused]] float2 my_ms = make_float2(0.0f, 1.0f);
  [[maybe_unused]] bool norm_skip = false;
  if constexpr (EPI != 0) {
    const float* st = (EPI == 1) ? p.row_stats : p.skip_stats;
    norm_skip = st != nullptr;
    if (st != nullptr && tid < BM) {
      RowMeanRstd(st, (EPI == 1) ? p.row_parts : p.skip_parts, min(m0 + tid, M - 1), p.norm_n, p.norm_eps, my_ms.x,
                  my_ms.y);
    }
  }
  // Producer: the residual tile is touched early (one dword per 128-byte line, values unused), so that the
  // epilogue finds it in cache instead of reading memory in the same burst in which every workgroup writes.
  [[maybe_unused]] int touch[(BM * BN * 2 / 128 + NWAVES * 64 - 1) / (NWAVES * 64)] = {};
  for (int kt = 0; kt < nk; kt++) {
    const char* As = smem + (NSTAGES == 2 ? (kt & 1) : kt % NSTAGES) * STAGE;
    const char* Ws = As + BM * BKB;
    char* nxt = smem + (NSTAGES == 2 ? ((kt + 1) & 1) : (kt + NSTAGES - 1) % NSTAGES) * STAGE;
    // This wave's pieces of k-tile kt have landed: the transfers of the NSTAGES - 2 k-tiles behind it may still be
    // in flight (near the end of K fewer are, and the wait is for all of them).
    constexpr int IN_FLIGHT = (NSTAGES - 2) * (A_CPW + W_CPW);
    if constexpr (NSTAGES > 2) {
      if (kt + NSTAGES - 2 < nk) {
        __builtin_amdgcn_s_waitcnt(0x0F70 | (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14));
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      }
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    }
    __syncthreads();                     // ... and everybody's; everybody is done reading the stage filled next
    if (kt + NSTAGES - 1 < nk) issue(nxt, nxt + BM * BKB, (kt + NSTAGES - 1) * BKB);
    if constexpr (EPI == 2) {
      if (kt == 1) {
        constexpr int LINES_PER_ROW = (BN * 2 + 127) / 128;
        constexpr int LINES = BM * LINES_PER_ROW;
#pragma unroll
        for (int q = 0; q < (LINES + NWAVES * 64 - 1) / (NWAVES * 64); q++) {
          const int line = q * NWAVES * 64 + tid;
          const int row = line / LINES_PER_ROW, seg = line % LINES_PER_ROW;
          const half_t* src = p.skip + (long long)min(m0 + row, M - 1) * p.ldskip + min(n0 + seg * 64, N - 2);
          if (line < LINES) touch[q] = *reinterpret_cast<const volatile int*>(src);
        }
      }
    }
    if constexpr (F8) {
      // One MFMA consumes 64 k-values: lane half g holds 32 consecutive bytes = 2 chunks.
#pragma unroll
      for (int ks = 0; ks < BKB / 64; ks++) {
        const int c0 = ((4 * ks + 2 * g) ^ swz) * 16, c1 = ((4 * ks + 2 * g + 1) ^ swz) * 16;
        intx8 af[TM], wf[TN];
#pragma unroll
        for (int i = 0; i < TM; i++) {
          const intx4 lo = *reinterpret_cast<const intx4*>(As + a_row + i * 32 * BKB + c0);
          const intx4 hi = *reinterpret_cast<const intx4*>(As + a_row + i * 32 * BKB + c1);
          af[i] = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const intx4 lo = *reinterpret_cast<const intx4*>(Ws + w_row + j * 32 * BKB + c0);
          const intx4 hi = *reinterpret_cast<const intx4*>(Ws + w_row + j * 32 * BKB + c1);
          wf[j] = intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[j], af[i], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < BKB / 32; ks++) {
        const int coff = ((2 * ks + g) ^ swz) * 16;
        half8 af[TM], wf[TN];
#pragma unroll
        for (int i = 0; i < TM; i++) af[i] = *reinterpret_cast<const half8*>(As + a_row + i * 32 * BKB + coff);
#pragma unroll
        for (int j = 0; j < TN; j++) wf[j] = *reinterpret_cast<const half8*>(Ws + w_row + j * 32 * BKB + coff);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[j], af[i], acc[i][j], 0, 0, 0);
      }
      if constexpr ((BM / WAVES_M / 32) * (BN / WAVES_N / 32) >= (BM / WAVES_M / 32) + (BN / WAVES_N / 32) && EPI == 0) {
        // Order of the k-tile's 32 MFMAs and 24 fragment reads: the reads of a k-step one by one between the MFMAs
        // of the step before it.
        constexpr int KS = BKB / 32, RD = TM + TN, MF = TM * TN;
        __builtin_amdgcn_sched_group_barrier(0x100, RD, 0);
#pragma unroll
        for (int ks = 0; ks + 1 < KS; ks++) {
#pragma unroll
          for (int q = 0; q < RD; q++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, MF - RD, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, MF, 0);
      }
    }
  }

  // Epilogue through LDS (the stage buffers are free after the barrier).
  __syncthreads();
  if constexpr (EPI == 2) {
    // (the early touches are consumed here: every wait of the loop has covered them)
#pragma unroll
    for (int q = 0; q < (int)(sizeof(touch) / sizeof(touch[0])); q++) asm volatile("" ::"v"(touch[q]));
  }
  OutT* C = reinterpret_cast<OutT*>(p.C);
  if constexpr (!F8) C += (long long)blockIdx.z * p.strideC;
  OutT* strip = reinterpret_cast<OutT*>(smem) + wave * 32 * EPI_STRIDE;
  constexpr int CHUNKS_PER_ROW = WN / OV;
  constexpr int STRIP_CHUNKS = 32 * CHUNKS_PER_ROW;
  constexpr int NPASS = (STRIP_CHUNKS + 63) / 64;
  const bool vec_ok = (p.ldc % OV == 0);
  float bias_v[TN][4][4];
#pragma unroll
  for (int j = 0; j < TN; j++)
#pragma unroll
    for (int blk = 0; blk < 4; blk++) {
      const floatx4 b4 = *reinterpret_cast<const floatx4*>(colv + wn * WN + j * 32 + blk * 8 + g * 4);
#pragma unroll
      for (int rr = 0; rr < 4; rr++) bias_v[j][blk][rr] = b4[rr];
    }
  // Folded layer norm: statistics of this tile's rows (of the A operand for a consumer, of the residual for a
  // producer), one row per thread, shared through LDS.
  [[maybe_unused]] float2* row_ms = reinterpret_cast<float2*>(smem + EPI_BYTES);                 // [BM] (mean, rstd)
  [[maybe_unused]] float2* part_lds = reinterpret_cast<float2*>(smem + EPI_BYTES + STAT_BYTES);  // [WAVES_N][BM]
  [[maybe_unused]] float col_c[TN][4][4];
  auto load_skip = [&](int i, intx4 (&sk)[NPASS]) {
#pragma unroll
    for (int pass = 0; pass < NPASS; pass++) {
      const int idx = pass * 64 + lane;
      const int row = idx / CHUNKS_PER_ROW;
      const int ch = idx - row * CHUNKS_PER_ROW;
      const int m = m0 + wm * WM + i * 32 + row;
      const int n = n0 + wn * WN + ch * OV;
      if constexpr (EPI == 2) {
        sk[pass] = (idx < STRIP_CHUNKS && m < M && n + OV - 1 < N)
                       ? *reinterpret_cast<const intx4*>(p.skip + (long long)m * p.ldskip + n)
                       : intx4{0, 0, 0, 0};
      }
    }
  };
  // Producer: the residual chunks of a strip are fetched one strip ahead.
  [[maybe_unused]] intx4 sk_cur[NPASS], sk_nxt[NPASS];
  if constexpr (EPI == 2) load_skip(0, sk_cur);
  if constexpr (EPI != 0) {
    if (norm_skip) {
      if (tid < BM) row_ms[tid] = my_ms;
      __syncthreads();
    }
    if constexpr (EPI == 1) {
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int blk = 0; blk < 4; blk++) LoadBias4(p.col_c, n0 + wn * WN + j * 32 + blk * 8 + g * 4, N, col_c[j][blk]);
    }
  }
  // Producer: gamma and beta of the residual's layer norm for this lane's eight columns (the same in every pass).
  [[maybe_unused]] float sk_gamma[8], sk_beta[8];
  if constexpr (EPI == 2) {
    static_assert(64 % CHUNKS_PER_ROW == 0, "a lane must keep its columns over the passes of a strip");
    const int n = n0 + wn * WN + (lane % CHUNKS_PER_ROW) * OV;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      sk_gamma[e] = (norm_skip && n + e < N) ? p.skip_gamma[n + e] : 1.0f;
      sk_beta[e] = (norm_skip && n + e < N) ? p.skip_beta[n + e] : 0.0f;
    }
  }
  DispatchAct(p.act, [&](auto act_fn) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      // Consumer: v = rstd * (scale * acc - mean * c) + bias = acc * (rstd * scale) + (bias - (rstd * mean) * c)
      [[maybe_unused]] float rs_scale = 1.0f, rs_mean = 0.0f;
      if constexpr (EPI == 1) {
        const float2 ms = row_ms[wm * WM + i * 32 + r];
        rs_scale = ms.y * p.scale;
        rs_mean = -ms.y * ms.x;
      }
#pragma unroll
      for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int blk = 0; blk < 4; blk++) {
          float v[4];
          if constexpr (F8) {
            // Per-column dequantisation factor (activation scale x weight-row scale).
            float cs[4];
            const floatx4 c4 = *reinterpret_cast<const floatx4*>(colv + BN + wn * WN + j * 32 + blk * 8 + g * 4);
#pragma unroll
            for (int rr = 0; rr < 4; rr++) cs[rr] = c4[rr];
#pragma unroll
            for (int rr = 0; rr < 4; rr++) v[rr] = act_fn(acc[i][j][blk * 4 + rr] * cs[rr] + bias_v[j][blk][rr]);
          } else if constexpr (EPI == 1) {
#pragma unroll
            for (int rr = 0; rr < 4; rr++)
              v[rr] = act_fn(fmaf(acc[i][j][blk * 4 + rr], rs_scale, fmaf(rs_mean, col_c[j][blk][rr], bias_v[j][blk][rr])));
          } else {
#pragma unroll
            for (int rr = 0; rr < 4; rr++) v[rr] = act_fn(acc[i][j][blk * 4 + rr] * p.scale + bias_v[j][blk][rr]);
          }
          OutT* dst = &strip[r * EPI_STRIDE + j * 32 + blk * 8 + g * 4];
          if constexpr (sizeof(OutT) == 1) {
            *reinterpret_cast<unsigned*>(dst) =
                PackFp8x4(v[0] * p.out_mul, v[1] * p.out_mul, v[2] * p.out_mul, v[3] * p.out_mul);
          } else {
            half4 h;
#pragma unroll
            for (int rr = 0; rr < 4; rr++) h[rr] = (half_t)v[rr];
            *reinterpret_cast<half4*>(dst) = h;
          }
        }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0); the strip is private to this wave
      __builtin_amdgcn_wave_barrier();
      if constexpr (EPI == 2) {
        if (i + 1 < TM) load_skip(i + 1, sk_nxt);
      }
#pragma unroll
      for (int pass = 0; pass < NPASS; pass++) {
        const int idx = pass * 64 + lane;
        const int row = idx / CHUNKS_PER_ROW;
        const int ch = idx - row * CHUNKS_PER_ROW;
        const int m = m0 + wm * WM + i * 32 + row;
        const int n = n0 + wn * WN + ch * OV;
        if constexpr (EPI == 2) {
          // C = (scale * acc + bias, already rounded to half) + residual, the residual normalised on the way when
          // it is itself an un-normalised sum; then the partial sums of the stored values over this wave's columns.
          const bool ok = idx < STRIP_CHUNKS && m < M && n + OV - 1 < N;
          const half8 hv = *reinterpret_cast<const half8*>(&strip[row * EPI_STRIDE + ch * OV]);
          const half8 hs = __builtin_bit_cast(half8, sk_cur[pass]);
          float2 rm = make_float2(0.0f, 1.0f);
          if (norm_skip) rm = row_ms[wm * WM + i * 32 + min(row, 31)];
          const float neg_mean_rstd = -rm.x * rm.y;
          half8 o;
          float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float t = fmaf((float)hs[e], rm.y, neg_mean_rstd);
            const float u = fmaf(t, sk_gamma[e], sk_beta[e]) + (float)hv[e];
            o[e] = (half_t)u;
            s1 += u;            // (of the sums before rounding to half: the difference is far below the rounding
            s2 = fmaf(u, u, s2);   //  of the normalised values themselves)
          }
          if (ok) {
            half_t* dst = reinterpret_cast<half_t*>(C) + (long long)m * p.ldc + n;
            if constexpr (STREAM) {
              __builtin_nontemporal_store(__builtin_bit_cast(intx4, o), reinterpret_cast<intx4*>(dst));
            } else {
              *reinterpret_cast<half8*>(dst) = o;
            }
          }
          // Sum over the CHUNKS_PER_ROW (4 or 8) neighbouring lanes of a row, with data-parallel-primitive moves.
          static_assert(CHUNKS_PER_ROW == 4 || CHUNKS_PER_ROW == 8, "row reduction written for 4 or 8 lanes per row");
          s1 += DppMove<0xB1>(s1);   // lane ^ 1
          s2 += DppMove<0xB1>(s2);
          s1 += DppMove<0x4E>(s1);   // lane ^ 2
          s2 += DppMove<0x4E>(s2);
          if constexpr (CHUNKS_PER_ROW == 8) {
            s1 += DppMove<0x141>(s1);   // mirror within 8 lanes: the other quad's sum
            s2 += DppMove<0x141>(s2);
          }
          if (ch == 0 && idx < STRIP_CHUNKS) part_lds[wn * BM + wm * WM + i * 32 + row] = make_float2(s1, s2);
          if (pass + 1 == NPASS && i + 1 < TM) {
#pragma unroll
            for (int q = 0; q < NPASS; q++) sk_cur[q] = sk_nxt[q];
          }
          continue;
        }
        if (idx < STRIP_CHUNKS && m < M && n < N) {
          OutT* dst = C + (long long)m * p.ldc + n;
          if (vec_ok && n + OV - 1 < N) {
            const intx4 val = *reinterpret_cast<const intx4*>(&strip[row * EPI_STRIDE + ch * OV]);
            if constexpr (STREAM) {
              __builtin_nontemporal_store(val, reinterpret_cast<intx4*>(dst));
            } else {
              *reinterpret_cast<intx4*>(dst) = val;
            }
          } else {
            for (int e = 0; e < OV && n + e < N; e++) dst[e] = strip[row * EPI_STRIDE + ch * OV + e];
          }
        }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
    }
  });
  if constexpr (EPI == 2) {
    // Partial sums of this column tile: the WAVES_N wave columns added in a fixed order.
    if (p.stats_out != nullptr) {
      __syncthreads();
      if (tid < BM && m0 + tid < M) {
        float2 t = part_lds[tid];
#pragma unroll
        for (int w = 1; w < WAVES_N; w++) {
          t.x += part_lds[w * BM + tid].x;
          t.y += part_lds[w * BM + tid].y;
        }
        reinterpret_cast<float2*>(p.stats_out)[(long long)(m0 + tid) * gridDim.y + blockIdx.y] = t;
      }
    }
  }
}

// Outputs of at least 64 MiB, or of 32 MiB (the size of L2) from at least 16384 rows, are written with streaming stores:
// cached, each round of output tiles would push out the operand rows that the next round reads again
// (measured on the same machine: BT4 batch 256 +0.7 %, fp8 batch 1024 +5 %). Smaller launches keep cached
// stores for the kernel that consumes the output (batch 128 loses 2.6 % with streaming, a 10x256 net at
// batch 64 loses 8 %). Only the BM = 256 tiles carry the variant: nothing else is picked for such outputs.
inline bool StreamOutput(long long m, long long n, long long batch, int elem_bytes) {
  const long long bytes = m * n * batch * elem_bytes;
  return bytes >= (64LL << 20) || (m >= 16384 && bytes >= (32LL << 20));
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int NSTAGES = 2>
void LaunchGemmDma(const GemmArgs& a, hipStream_t stream) {
  dim3 grid((a.M + BM - 1) / BM, (a.N + BN - 1) / BN, a.batch);
  const dim3 block(WAVES_M * WAVES_N * 64);
  auto launch = [&](auto stream_tag) {
    constexpr bool S = decltype(stream_tag)::value;
    // The folded-layer-norm epilogues exist with two stages only (LaunchGemmDmaStaged sends them there).
    if (a.skip != nullptr) {
      if constexpr (((BN / WAVES_N) % 64 == 0 || BN / WAVES_N == 32) && NSTAGES == 2) {
        hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BK * 2, WAVES_M, WAVES_N, GemmArgs, half_t, S, 2, 2>), grid, block, 0,
                           stream, a);
      }
    } else if (a.row_stats != nullptr) {
      if constexpr (NSTAGES == 2) {
        hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BK * 2, WAVES_M, WAVES_N, GemmArgs, half_t, S, 1, 2>), grid, block, 0,
                           stream, a);
      }
    } else {
      hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BK * 2, WAVES_M, WAVES_N, GemmArgs, half_t, S, 0, NSTAGES>), grid, block, 0,
                         stream, a);
    }
  };
  if constexpr (BM == 256) {
    if (StreamOutput(a.M, a.N, a.batch, 2)) {
      launch(std::true_type{});
      return;
    }
  }
  launch(std::false_type{});
}

// As many LDS stages (2 to 4) as leave room on the CUs for all of the launch's workgroups at once: with one
// workgroup per CU nothing else hides the time a k-tile takes to arrive from memory, with several per CU they hide it
// for each other and more stages would only lower their number (15x1024 net, per pass: 16 positions 1.91 -> 1.67 ms
// with four stages; 64 positions 2.59 -> 2.93 ms if forced there).
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
void LaunchGemmDmaStaged(const GemmArgs& a, hipStream_t stream) {
  constexpr int kStage = (BM + BN) * BK * 2, kLds = 160 * 1024, kCus = 256;
  const long long wgs = (long long)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN) * a.batch;
  if (a.skip != nullptr || a.row_stats != nullptr) return LaunchGemmDma<BM, BN, BK, WAVES_M, WAVES_N, 2>(a, stream);
  if constexpr (4 * kStage + 4096 <= kLds) {
    if (wgs <= (long long)kCus * (kLds / (4 * kStage + 4096))) return LaunchGemmDma<BM, BN, BK, WAVES_M, WAVES_N, 4>(a, stream);
  }
  if constexpr (3 * kStage + 4096 <= kLds) {
    if (wgs <= (long long)kCus * (kLds / (3 * kStage + 4096))) return LaunchGemmDma<BM, BN, BK, WAVES_M, WAVES_N, 3>(a, stream);
  }
  LaunchGemmDma<BM, BN, BK, WAVES_M, WAVES_N, 2>(a, stream);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int BKB = 128, int NSTAGES = 2>
void LaunchGemmDmaF8(const GemmF8Args& a, hipStream_t stream) {
  dim3 grid((a.M + BM - 1) / BM, (a.N + BN - 1) / BN, 1);
  const dim3 block(WAVES_M * WAVES_N * 64);
  if constexpr (BM == 256) {
    if (StreamOutput(a.M, a.N, 1, a.out_f8 ? 1 : 2)) {
      if (a.out_f8) {
        hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BKB, WAVES_M, WAVES_N, GemmF8Args, uint8_t, true>), grid, block, 0,
                           stream, a);
      } else {
        hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BKB, WAVES_M, WAVES_N, GemmF8Args, half_t, true>), grid, block, 0,
                           stream, a);
      }
      return;
    }
  }
  if (a.out_f8) {
    hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BKB, WAVES_M, WAVES_N, GemmF8Args, uint8_t, false, 0, NSTAGES>), grid,
                       block, 0, stream, a);
  } else {
    hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BKB, WAVES_M, WAVES_N, GemmF8Args, half_t, false, 0, NSTAGES>), grid,
                       block, 0, stream, a);
  }
}

// Stage count by the launch's workgroup count, as LaunchGemmDmaStaged does for fp16 operands.
template <int BM, int BN, int WAVES_M, int WAVES_N>
void LaunchGemmDmaF8Staged(const GemmF8Args& a, hipStream_t stream) {
  constexpr int kStage = (BM + BN) * 128, kLds = 160 * 1024, kCus = 256;
  const long long wgs = (long long)((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  if constexpr (4 * kStage + 4096 <= kLds) {
    if (wgs <= (long long)kCus * (kLds / (4 * kStage + 4096))) return LaunchGemmDmaF8<BM, BN, WAVES_M, WAVES_N, 128, 4>(a, stream);
  }
  if constexpr (3 * kStage + 4096 <= kLds) {
    if (wgs <= (long long)kCus * (kLds / (3 * kStage + 4096))) return LaunchGemmDmaF8<BM, BN, WAVES_M, WAVES_N, 128, 3>(a, stream);
  }
  LaunchGemmDmaF8<BM, BN, WAVES_M, WAVES_N, 128, 2>(a, stream);
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
void LaunchGemmTile(const GemmArgs& a, hipStream_t stream) {
  dim3 grid((a.M + BM - 1) / BM, (a.N + BN - 1) / BN, a.batch * a.split_k);
  if (a.out_f32) {
    hipLaunchKernelGGL((gemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, float>), grid, dim3(256), 0, stream, a);
  } else {
    hipLaunchKernelGGL((gemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, half_t>), grid, dim3(256), 0, stream, a);
  }
}

}  // namespace

namespace {
// The smallest panel (in operand rows a workgroup reads) with which the problem still fits into one workgroup per
// CU; the largest one otherwise. 64x1024xK runs as 256 panels of 16x16 (64x1024x1536: 4.6 us against 14.3 with 64x32
// panels), 64x3072xK as 192 panels of 32x32.
struct RowPanelShape { int rt, ct; };
constexpr RowPanelShape kRowPanelShapes[] = {{1, 1}, {2, 1}, {1, 2}, {2, 2}, {4, 2}};
constexpr long long kRowPanelWorkgroups = 256;   // one per CU
inline long long RowPanelWorkgroups(const GemmArgs& a, const RowPanelShape& c) {
  return (long long)((a.M + 16 * c.rt - 1) / (16 * c.rt)) * ((a.N + 16 * c.ct - 1) / (16 * c.ct)) * a.batch;
}
inline RowPanelShape PickRowPanelShape(const GemmArgs& a) {
  for (const RowPanelShape& c : kRowPanelShapes) {
    if (RowPanelWorkgroups(a, c) <= kRowPanelWorkgroups) return c;
  }
  return kRowPanelShapes[4];
}

template <int RT, int CT, int U>
void LaunchGemmRowPanelShape(const GemmArgs& a, hipStream_t stream) {
  dim3 grid((a.M + 16 * RT - 1) / (16 * RT), (a.N + 16 * CT - 1) / (16 * CT), a.batch);
  if (a.out_f32) {
    hipLaunchKernelGGL((gemm_rowpanel_kernel<RT, CT, U, float>), grid, dim3(512), 0, stream, a);
  } else {
    hipLaunchKernelGGL((gemm_rowpanel_kernel<RT, CT, U, half_t>), grid, dim3(512), 0, stream, a);
  }
}

template <int RT, int CT>
void LaunchGemmRowPanelSteps(const GemmArgs& a, hipStream_t stream) {
  // Steps of 32 per wave; U of them are loaded at once (registers: 4 (RT + CT) U), in as few rounds as possible
  // with as few steps loaded in vain as possible.
  constexpr int kMaxU = (RT + CT >= 6) ? 6 : 8;
  const int per_wave = (a.K / 32 + 7) / 8;
  int u = 2;
  if (per_wave > 2) {
    int best_waste = 1 << 30;
    for (int cand = kMaxU; cand >= 4; cand -= 2) {
      const int rounds = (per_wave + cand - 1) / cand;
      const int waste = rounds * cand - per_wave + 4 * (rounds - 1);   // a further round costs about four steps
      if (waste < best_waste) { best_waste = waste; u = cand; }
    }
  }
  switch (u) {
    case 2: LaunchGemmRowPanelShape<RT, CT, 2>(a, stream); break;
    case 4: LaunchGemmRowPanelShape<RT, CT, 4>(a, stream); break;
    case 6: LaunchGemmRowPanelShape<RT, CT, 6>(a, stream); break;
    default:
      if constexpr (kMaxU >= 8) LaunchGemmRowPanelShape<RT, CT, 8>(a, stream);
      else LaunchGemmRowPanelShape<RT, CT, 6>(a, stream);
      break;
  }
}

inline void LaunchGemmRowPanel(const GemmArgs& a, hipStream_t stream) {
  const RowPanelShape c = PickRowPanelShape(a);
  if (c.rt == 1 && c.ct == 1) LaunchGemmRowPanelSteps<1, 1>(a, stream);
  else if (c.rt == 2 && c.ct == 1) LaunchGemmRowPanelSteps<2, 1>(a, stream);
  else if (c.rt == 1 && c.ct == 2) LaunchGemmRowPanelSteps<1, 2>(a, stream);
  else if (c.rt == 2 && c.ct == 2) LaunchGemmRowPanelSteps<2, 2>(a, stream);
  else LaunchGemmRowPanelSteps<4, 2>(a, stream);
}

enum GemmVariant { kDma256x256, kDma256x192, kDma256x128, kTile128, kTile64, kDma128x128, kRowPanel, kDma128x64, kPersist256,
                   kDma128x32, kDma64x64 };

int g_variant_override = -1;

GemmVariant PickGemmVariant(const GemmArgs& a) {
  if (g_variant_override >= 0) {
    const bool dma_ok = !a.out_f32 && a.split_k == 1 && a.K % 64 == 0;
    const bool is_dma = g_variant_override <= kDma256x128 || g_variant_override == kDma128x128 ||
                        g_variant_override == kDma128x64 || g_variant_override == kDma128x32 ||
                        g_variant_override == kDma64x64;
    bool ok = is_dma ? dma_ok : (g_variant_override != kRowPanel || a.split_k == 1);
    if (g_variant_override == kPersist256) ok = GemmPersistentSupports(a);
    if (ok) return static_cast<GemmVariant>(g_variant_override);
  }
  const long long tiles128 = (long long)((a.M + 127) / 128) * ((a.N + 127) / 128) * a.batch;
  if (!a.out_f32 && a.split_k == 1 && a.K % 64 == 0 && a.K >= 128 && a.N >= 128 && a.M >= (a.latency_first ? 256 : 1024) && tiles128 >= 64) {
    // Direct-to-LDS kernels. Cost = rounds over the 256 CUs x tile area x a measured cost per
    // output element and round (ns per element at K = 1024): 0.60 for 256x256, 0.61 for 256x192;
    // the two small shapes run two workgroups per CU, 0.68 (256x128) and 0.75 (128x128) per element
    // while sharing a CU, 0.84 and 0.95 when a single round leaves every workgroup alone on its CU.
    auto rounds = [&](int bm, int bn) {
      const long long tiles = (long long)((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn) * a.batch;
      return (double)((tiles + 255) / 256);
    };
    const double r256 = rounds(256, 256), r192 = rounds(256, 192), r128 = rounds(256, 128), rs = rounds(128, 128);
    const double c256 = r256 * 256 * 256 * 0.60;
    const double c192 = r192 * 256 * 192 * 0.61;
    const double c128 = r128 * 256 * 128 * (r128 > 1 ? 0.68 : 0.84);
    // (short reductions are dominated by the epilogue, where the smallest tile loses a little more)
    const double cs = rs * 128 * 128 * (rs > 1 ? 0.75 : 0.95) * (a.K <= 256 ? 1.12 : 1.0);
    GemmVariant best = kDma256x256;
    double cost = c256;
    // (The persistent kernel of gemm_persistent.hip is not part of this choice: alone it is level with the 256x256
    // kernel on these shapes (16384x3072x1024: 107 against 112 us, single-round shapes equal), but its one
    // workgroup per CU holds every CU for the whole launch, so the smolgen chain on the second stream no longer
    // slips in between rounds of tiles: a 15x1024 pass at batch 256 takes 6.66 ms with it against 5.91 ms.
    // It is reachable through SetGemmVariantOverride(kPersist256).)
    // (a producer of a folded layer norm needs a power-of-two column count per wave: not the 192-wide tile)
    if (c192 < cost && a.skip == nullptr) { best = kDma256x192; cost = c192; }
    if (c128 < cost) { best = kDma256x128; cost = c128; }
    if (cs < cost) { best = kDma128x128; cost = cs; }
    // 128x64 tiles (three workgroups per CU, so partial rounds are counted as fractions) move more operand
    // bytes from L2 per flop, but they split small problems over all CUs and odd tile counts evenly
    // (4096x512x1024: 10.5 us against 14.6 for 128x128; 36 x 2048x256x256: 23.1 us against 26.0 for 256x128).
    {
      const double tiles = (double)((a.M + 127) / 128) * ((a.N + 63) / 64) * a.batch;
      const double c64 = std::max(1.0, tiles / 256.0) * 128 * 64 * 0.80;
      if (c64 < cost) { best = kDma128x64; cost = c64; }
    }
    return best;
  }
  // Very many rows, at most 32 columns (the smolgen compression at 512 positions and more): a memory-bound stream of
  // the activation rows. 128x32 direct-to-LDS tiles (four workgroups per CU) read them once at full line width
  // (65536x32x1024: 34 us against 96 for the row-panel kernel).
  if (!a.out_f32 && a.split_k == 1 && a.batch == 1 && a.N <= 32 && a.K % 64 == 0 && a.K >= 128 && a.M >= 32768) {
    return kDma128x32;
  }
  // Small problems: the 64x64 kernel walks K serially in one workgroup; when it would start at most 64 workgroups,
  // the row-panel kernel (8-way K split inside the workgroup, panels sized to give every CU one) is faster
  // (64x3072x1024: 6.4 vs 9.7 us; 32x4096x256: 3.1 vs 5.1 us). With a short K and more panels than CUs it loses
  // (128x8192x256 in 64x32 panels: 15.8 vs 5.6 us).
  // The same holds for a handful of rows with thousands of columns, as long as panels of at most 32x32 cover them
  // with one workgroup per CU (1x8192x256: 2.9 vs 5.0 us).
  const long long tiles64 = (long long)((a.M + 63) / 64) * ((a.N + 63) / 64) * a.batch;
  if (a.split_k == 1 && a.K >= 256 &&
      (tiles64 <= 64 || (a.M <= 128 && tiles64 <= 128) ||
       RowPanelWorkgroups(a, kRowPanelShapes[3]) <= kRowPanelWorkgroups)) {
    return kRowPanel;
  }
  // A few hundred rows (3 to 12 positions), or few columns: too small for the cost model above, too large for row
  // panels. Small direct-to-LDS tiles with three or four stages in flight stream the weights, which come from
  // memory, better than the register-staged tiles below (512x1024x1024: 6.8 against 9.9 us; a pass of 8 positions
  // 1.94 -> 1.46 ms). 128x64 tiles once they fill most CUs (512x3072x1024: 9.6 against 11.1 us), 64x64 before.
  // (With a short reduction only on request: beside a large GEMM on the other stream the register-staged tiles
  // disturb it less.)
  if (!a.out_f32 && a.split_k == 1 && a.K % 64 == 0 && a.K >= (a.latency_first ? 256 : 512) && a.N >= 64 && a.M >= 192) {
    const long long wg128 = (long long)((a.M + 127) / 128) * ((a.N + 63) / 64) * a.batch;
    return wg128 >= 192 ? kDma128x64 : kDma64x64;
  }
  // A single 32-column panel (the smolgen compression): one workgroup per 64 rows, K split over its waves
  // (16384x32x1024: 9.5 us against 12.3 for the 64x64 tiles, but with twice the threads on every CU).
  if (a.latency_first && a.split_k == 1 && a.N <= 32 && a.K >= 512) return kRowPanel;
  const long long big_tiles = tiles128;
  return big_tiles >= 192 ? kTile128 : kTile64;
}
}  // namespace

void SetGemmVariantOverride(int variant) { g_variant_override = variant; }

namespace {
// Column-tile width of the direct-to-LDS variants (0 for the others).
int DmaTileN(GemmVariant v) {
  switch (v) {
    case kDma256x256: return 256;
    case kDma256x192: return 192;
    case kDma256x128: case kDma128x128: return 128;
    case kDma128x64: case kDma64x64: return 64;
    case kDma128x32: return 32;
    default: return 0;
  }
}
}  // namespace

bool GemmSupportsNormFolding(const GemmArgs& a) {
  const GemmVariant v = PickGemmVariant(a);
  if (a.skip != nullptr) {
    return DmaTileN(v) != 0 && v != kDma256x192 && !a.out_f32 && a.act == 3 && a.batch == 1 && a.N % 8 == 0 &&
           a.ldc % 8 == 0 && a.ldskip % 8 == 0 && a.row_stats == nullptr;
  }
  if (a.row_stats != nullptr) {
    if (a.split_k != 1 || a.batch != 1 || a.col_c == nullptr) return false;
    return DmaTileN(v) != 0 || v == kTile128 || v == kTile64 || v == kRowPanel;
  }
  return true;
}

int GemmStatsParts(const GemmArgs& a) {
  const int bn = DmaTileN(PickGemmVariant(a));
  return bn == 0 ? 0 : (a.N + bn - 1) / bn;
}

const char* GemmVariantName(const GemmArgs& a) {
  switch (PickGemmVariant(a)) {
    case kPersist256: return "gemm_persistent_256x256x64";
    case kDma256x256: return "gemm_dma_256x256x64";
    case kDma256x192: return "gemm_dma_256x192x64";
    case kDma256x128: return "gemm_dma_256x128x32";
    case kDma128x128: return "gemm_dma_128x128x64";
    case kDma128x64: return "gemm_dma_128x64x64";
    case kDma128x32: return "gemm_dma_128x32x64";
    case kDma64x64: return "gemm_dma_64x64x64";
    case kRowPanel: return "gemm_rowpanel";
    case kTile128: return "gemm_128x128x64";
    default: return a.split_k > 1 ? "gemm_64x64x64_splitk" : "gemm_64x64x64";
  }
}

void LaunchGemm(const GemmArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0 || a.batch <= 0) return;
  if ((a.skip != nullptr || a.row_stats != nullptr) && !GemmSupportsNormFolding(a)) {
    throw std::runtime_error("LaunchGemm: no kernel variant with the folded layer-norm epilogue for this shape");
  }
  switch (PickGemmVariant(a)) {
    case kPersist256: LaunchGemmPersistent(a, StreamOutput(a.M, a.N, a.batch, 2), stream); break;
    case kDma256x256: LaunchGemmDma<256, 256, 64, 2, 4>(a, stream); break;
    case kDma256x192: LaunchGemmDma<256, 192, 64, 4, 2>(a, stream); break;
    case kDma256x128: LaunchGemmDmaStaged<256, 128, 32, 4, 2>(a, stream); break;
    case kDma128x128: LaunchGemmDmaStaged<128, 128, 64, 2, 2>(a, stream); break;
    case kDma128x64: LaunchGemmDmaStaged<128, 64, 64, 2, 2>(a, stream); break;
    case kDma128x32: LaunchGemmDma<128, 32, 64, 4, 1>(a, stream); break;
    case kDma64x64: LaunchGemmDmaStaged<64, 64, 64, 2, 2>(a, stream); break;
    case kRowPanel: LaunchGemmRowPanel(a, stream); break;
    case kTile128: LaunchGemmTile<128, 128, 64, 2, 2>(a, stream); break;
    default: LaunchGemmTile<64, 64, 64, 2, 2>(a, stream); break;
  }
}

namespace {
// 0: 256x256, 1: 256x192, 2: 256x128, 5: 128x128 and 7: 128x64 with 4 waves (two / three workgroups per CU); chosen by
// the cost model of the fp16 kernels (the k-tile structure is the same).
template <int RT, int CT>
void LaunchGemmF8RowPanelSteps(const GemmF8Args& a, hipStream_t stream) {
  dim3 grid((a.M + 16 * RT - 1) / (16 * RT), (a.N + 16 * CT - 1) / (16 * CT), 1);
  const int per_wave = (a.K / 128 + 7) / 8;   // steps of 128 per wave: all of them in flight, up to four
  auto launch = [&](auto u_tag) {
    constexpr int U = decltype(u_tag)::value;
    if (a.out_f8) {
      hipLaunchKernelGGL((gemm_f8_rowpanel_kernel<RT, CT, U, uint8_t>), grid, dim3(512), 0, stream, a);
    } else {
      hipLaunchKernelGGL((gemm_f8_rowpanel_kernel<RT, CT, U, half_t>), grid, dim3(512), 0, stream, a);
    }
  };
  if (per_wave <= 1) launch(std::integral_constant<int, 1>{});
  else if (per_wave == 2) launch(std::integral_constant<int, 2>{});
  else launch(std::integral_constant<int, 4>{});
}

GemmArgs PanelShapeArgs(const GemmF8Args& a) {
  GemmArgs g;
  g.M = a.M; g.N = a.N; g.K = a.K; g.batch = 1;
  return g;
}

void LaunchGemmF8RowPanel(const GemmF8Args& a, hipStream_t stream) {
  const RowPanelShape c = PickRowPanelShape(PanelShapeArgs(a));
  if (c.rt == 1 && c.ct == 1) LaunchGemmF8RowPanelSteps<1, 1>(a, stream);
  else if (c.rt == 2 && c.ct == 1) LaunchGemmF8RowPanelSteps<2, 1>(a, stream);
  else if (c.rt == 1 && c.ct == 2) LaunchGemmF8RowPanelSteps<1, 2>(a, stream);
  else if (c.rt == 2 && c.ct == 2) LaunchGemmF8RowPanelSteps<2, 2>(a, stream);
  else LaunchGemmF8RowPanelSteps<4, 2>(a, stream);
}

// Few rows: row panels, as for fp16 operands.
bool GemmF8TakesRowPanels(const GemmF8Args& a) {
  const long long tiles64 = (long long)((a.M + 63) / 64) * ((a.N + 63) / 64);
  return a.K >= 256 &&
         (tiles64 <= 64 || RowPanelWorkgroups(PanelShapeArgs(a), kRowPanelShapes[3]) <= kRowPanelWorkgroups);
}

int PickGemmF8Variant(const GemmF8Args& a) {
  if (g_variant_override >= 0 && (g_variant_override <= 2 || g_variant_override == kDma128x128 ||
                                  g_variant_override == kDma128x64 || g_variant_override == kRowPanel ||
                                  g_variant_override == kDma64x64)) {
    return g_variant_override;
  }
  if (GemmF8TakesRowPanels(a)) return kRowPanel;
  // A few hundred rows: small tiles with three or four stages in flight, as for fp16 operands.
  if (a.M < 1024 && a.N >= 64) {
    const long long wg128 = (long long)((a.M + 127) / 128) * ((a.N + 63) / 64);
    return wg128 >= 192 ? kDma128x64 : kDma64x64;
  }
  auto rounds = [&](int bm, int bn) {
    const long long tiles = (long long)((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn);
    return (double)((tiles + 255) / 256);
  };
  const double r128 = rounds(256, 128), rs = rounds(128, 128);
  const double c256 = rounds(256, 256) * 256 * 256 * 0.60;
  const double c192 = rounds(256, 192) * 256 * 192 * 0.61;
  const double c128 = r128 * 256 * 128 * 0.84;   // 96 KiB of LDS: one workgroup per CU
  const double cs = rs * 128 * 128 * (rs > 1 ? 0.75 : 0.95);
  int best = 0;
  double cost = c256;
  if (c192 < cost) { best = 1; cost = c192; }
  if (c128 < cost) { best = 2; cost = c128; }
  if (cs < cost) { best = kDma128x128; cost = cs; }
  const double tiles64 = (double)((a.M + 127) / 128) * ((a.N + 63) / 64);
  const double c64 = std::max(1.0, tiles64 / 256.0) * 128 * 64 * 0.80;
  if (c64 < cost) { best = kDma128x64; cost = c64; }
  return best;
}
}  // namespace

const char* GemmF8VariantName(const GemmF8Args& a) {
  switch (PickGemmF8Variant(a)) {
    case 0: return "gemm_f8_256x256x128";
    case 1: return "gemm_f8_256x192x128";
    case 2: return "gemm_f8_256x128x128";
    case kDma128x64: return "gemm_f8_128x64x128";
    case kRowPanel: return "gemm_f8_rowpanel";
    case kDma64x64: return "gemm_f8_64x64x128";
    default: return "gemm_f8_128x128x128";
  }
}

void LaunchGemmF8(const GemmF8Args& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0) return;
  switch (PickGemmF8Variant(a)) {
    case 0: LaunchGemmDmaF8<256, 256, 2, 4>(a, stream); break;
    case 1: LaunchGemmDmaF8<256, 192, 4, 2>(a, stream); break;
    case 2: LaunchGemmDmaF8<256, 128, 4, 2>(a, stream); break;
    case kDma128x64: LaunchGemmDmaF8Staged<128, 64, 2, 2>(a, stream); break;
    case kDma64x64: LaunchGemmDmaF8Staged<64, 64, 2, 2>(a, stream); break;
    case kRowPanel: LaunchGemmF8RowPanel(a, stream); break;
    default: LaunchGemmDmaF8Staged<128, 128, 2, 2>(a, stream); break;
  }
}

// ---------------------------------------------------------------------------
// float GEMM (fp32 configuration): same contract on fp32 operands with the fp32 matrix instruction
// v_mfma_f32_32x32x2_f32 (fp32 products, fp32 accumulation).
//
// Eight waves per workgroup, laid out TILES_M x TILES_N x KSPLIT: every wave owns one 32x32 accumulator tile over
// its share of the reduction and reads its 32 + 32 operand rows straight from global memory, 16 bytes per lane
// and k-step (lane half g takes k = 8s + 4g .. 8s + 4g + 3; the four MFMAs of a step pair equal offsets of both
// operands, so every k is used exactly once). Sixteen such loads are kept in flight per wave. The KSPLIT partial
// tiles are added through LDS in wave order, then scale, bias and activation are applied.
//   <1,1,8>: 32x32 tile, the reduction split eight ways -- few output tiles, long K (the heads' dense layers at
//            small batch: 32x128x2048 used to run on two workgroups);
//   <2,2,2>: 64x64 tile for launches with many tiles.
// ---------------------------------------------------------------------------
namespace {
template <int TILES_M, int TILES_N, int KSPLIT>
__global__ __launch_bounds__(512) void gemm_f32_mfma_kernel(GemmArgsF32 p) {
  static_assert(TILES_M * TILES_N * KSPLIT == 8, "eight waves");
  constexpr int UNROLL = 8;   // k-steps (of 8) whose loads are issued together
  __shared__ float red[8][32][33];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ks = wave % KSPLIT, tile = wave / KSPLIT;
  const int tm = tile / TILES_N, tn = tile % TILES_N;
  const int r = lane & 31, g = lane >> 5;
  const int m0 = (blockIdx.x * TILES_M + tm) * 32, n0 = (blockIdx.y * TILES_N + tn) * 32;
  const float* A = p.A + (long long)blockIdx.z * p.strideA + (long long)min(m0 + r, p.M - 1) * p.lda + g * 4;
  const float* W = p.W + (long long)blockIdx.z * p.strideW + (long long)min(n0 + r, p.N - 1) * p.ldw + g * 4;
  float* C = p.C + (long long)blockIdx.z * p.strideC;
  const int K = p.K;
  floatx16 acc;
#pragma unroll
  for (int e = 0; e < 16; e++) acc[e] = 0.0f;
  const int steps = (K + 7) / 8;
  // this wave's k-steps: ks, ks + KSPLIT, ...
  for (int s0 = ks; s0 < steps; s0 += KSPLIT * UNROLL) {
    floatx4 va[UNROLL], vw[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      const int k = (s0 + u * KSPLIT) * 8;
      const bool ok = k + g * 4 < K;   // K % 4 == 0: a 16-byte piece is inside or outside as a whole
      va[u] = ok ? *reinterpret_cast<const floatx4*>(A + k) : floatx4{0, 0, 0, 0};
      vw[u] = ok ? *reinterpret_cast<const floatx4*>(W + k) : floatx4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++)
#pragma unroll
      for (int e = 0; e < 4; e++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(vw[u][e], va[u][e], acc, 0, 0, 0);
  }
  // accumulator element e: n = 8*(e/4) + 4*g + e%4, m = r
#pragma unroll
  for (int e = 0; e < 16; e++) red[wave][r][8 * (e / 4) + 4 * g + (e & 3)] = acc[e];
  __syncthreads();
  constexpr int OUT = TILES_M * TILES_N * 1024;
  for (int idx = tid; idx < OUT; idx += 512) {
    const int t = idx >> 10, mm = (idx >> 5) & 31, nn = idx & 31;
    float x = 0.0f;
#pragma unroll
    for (int z = 0; z < KSPLIT; z++) x += red[t * KSPLIT + z][mm][nn];
    const int m = (blockIdx.x * TILES_M + t / TILES_N) * 32 + mm, n = (blockIdx.y * TILES_N + t % TILES_N) * 32 + nn;
    if (m < p.M && n < p.N) {
      x *= p.scale;
      if (p.bias != nullptr) x += p.bias[n];
      C[(long long)m * p.ldc + n] = Activate(x, p.act);
    }
  }
}
}  // namespace

void LaunchGemmF32(const GemmArgsF32& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0 || a.batch <= 0) return;
  const long long tiles64 = (long long)((a.M + 63) / 64) * ((a.N + 63) / 64) * a.batch;
  if (tiles64 >= 256) {
    dim3 grid((a.M + 63) / 64, (a.N + 63) / 64, a.batch);
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<2, 2, 2>), grid, dim3(512), 0, stream, a);
  } else {
    dim3 grid((a.M + 31) / 32, (a.N + 31) / 32, a.batch);
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<1, 1, 8>), grid, dim3(512), 0, stream, a);
  }
}

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
  for (int i = threadIdx.x; i < 64 * chunks; i += 256) {
    const int sq = i / chunks, c0 = (i - sq * chunks) * V;
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
__global__ __launch_bounds__(256) void piece_planes_kernel(const uint64_t* __restrict__ masks,
                                                           const float* __restrict__ values,
                                                           half_t* __restrict__ out) {
  const int b = blockIdx.x;
  for (int i = threadIdx.x; i < 64 * 12; i += 256) {
    const int sq = i / 12, j = i - sq * 12;
    const bool bit = (masks[(long long)b * 112 + j] >> sq) & 1ull;
    out[(long long)b * 768 + i] = bit ? (half_t)values[(long long)b * 112 + j] : (half_t)0.0f;
  }
}

// x[b][sq][c] = x * mult[sq][c] + add[sq][c]
__global__ __launch_bounds__(256) void input_gating_kernel(half_t* __restrict__ x, const float* __restrict__ mult,
                                                           const float* __restrict__ add, int per_sample,
                                                           long long total) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int j = (int)(i % per_sample);
  x[i] = (half_t)((float)x[i] * mult[j] + add[j]);
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
    hipLaunchKernelGGL((expand_planes_attn_kernel<T, 8>), dim3(batch), dim3(256), 0, stream, masks, values, pos_enc, 64,
                       0LL, out, ld);
  } else {
    hipLaunchKernelGGL((expand_planes_attn_kernel<T, 1>), dim3(batch), dim3(256), 0, stream, masks, values, pos_enc, 64,
                       0LL, out, ld);
  }
}

void LaunchExpandPlanesDense(const uint64_t* masks, const float* values, const half_t* extra, int n_extra,
                             half_t* out, int ld, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  if (ld % 8 == 0) {
    hipLaunchKernelGGL((expand_planes_attn_kernel<half_t, 8>), dim3(batch), dim3(256), 0, stream, masks, values, extra,
                       n_extra, 64LL * n_extra, out, ld);
  } else {
    hipLaunchKernelGGL((expand_planes_attn_kernel<half_t, 1>), dim3(batch), dim3(256), 0, stream, masks, values, extra,
                       n_extra, 64LL * n_extra, out, ld);
  }
}

void LaunchPiecePlanes(const uint64_t* masks, const float* values, half_t* out, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  hipLaunchKernelGGL(piece_planes_kernel, dim3(batch), dim3(256), 0, stream, masks, values, out);
}

void LaunchInputGating(half_t* x, const float* mult, const float* add, int batch, int per_sample, hipStream_t stream) {
  const long long total = (long long)batch * per_sample;
  if (total <= 0) return;
  hipLaunchKernelGGL(input_gating_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, x, mult, add,
                     per_sample, total);
}
template void LaunchExpandPlanesAttn<half_t>(const uint64_t*, const float*, const half_t*, half_t*, int, int,
                                             hipStream_t);
template void LaunchExpandPlanesAttn<float>(const uint64_t*, const float*, const float*, float*, int, int,
                                            hipStream_t);

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
template <int NV>  // 16-byte vectors per lane; covers C <= 512 * NV
__global__ __launch_bounds__(256) void layer_norm_kernel(const half_t* __restrict__ x, const half_t* skip,
                                                         half_t* y, uint8_t* yq, float q_mul,
                                                         const float* __restrict__ gamma,
                                                         const float* __restrict__ beta, int rows, int C,
                                                         float alpha, float eps) {
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
      half8 hx = *reinterpret_cast<const half8*>(xr + v * 8);
      if (sr) {
        half8 hs = *reinterpret_cast<const half8*>(sr + v * 8);
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
      half8 o;
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; e++) {
        f[e] = beta[v * 8 + e] + gamma[v * 8 + e] * (t[i][e] - mean) * den;
        o[e] = (half_t)f[e];
      }
      *reinterpret_cast<half8*>(yr + v * 8) = o;
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
template <bool EARLY>
__global__ __launch_bounds__(256) void layer_norm_rows_kernel(const float* __restrict__ xf, int n_partials,
                                                              long long partial_stride, const half_t* xh,
                                                              int pre_act, const half_t* skip, half_t* y,
                                                              const float* __restrict__ gamma,
                                                              const float* __restrict__ beta, int C, float alpha,
                                                              float eps) {
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
          half8 h = *reinterpret_cast<const half8*>(xh + off);
#pragma unroll
          for (int e = 0; e < 8; e++) t[i][e] = (float)h[e];
        }
#pragma unroll
        for (int e = 0; e < 8; e++) t[i][e] = act_fn(t[i][e]) * alpha;
        if (skip != nullptr) {
          half8 hs = *reinterpret_cast<const half8*>(skip + off);
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
      half8 o;
#pragma unroll
      for (int e = 0; e < 8; e++) o[e] = (half_t)(bt[i][e / 4][e % 4] + gm[i][e / 4][e % 4] * (t[i][e] - mean) * den);
      *reinterpret_cast<half8*>(y + (long long)row * C + v * 8) = o;
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
                         int C, float alpha, float eps, hipStream_t stream) {
  if (rows <= 0) return;
  if (rows <= 64) {
    hipLaunchKernelGGL(layer_norm_rows_kernel<true>, dim3(rows), dim3(256), 0, stream, x_f32, n_partials,
                       partial_stride, x_f16, pre_act, skip, y, gamma, beta, C, alpha, eps);
  } else {
    hipLaunchKernelGGL(layer_norm_rows_kernel<false>, dim3(rows), dim3(256), 0, stream, x_f32, n_partials,
                       partial_stride, x_f16, pre_act, skip, y, gamma, beta, C, alpha, eps);
  }
}

void LaunchLayerNorm(const half_t* x, const half_t* skip, half_t* y, const float* gamma, const float* beta,
                     int rows, int C, float alpha, float eps, hipStream_t stream, uint8_t* y_f8, float f8_mul) {
  if (rows <= 0) return;
  dim3 grid((rows + 3) / 4), block(256);
  if (C <= 512) {
    hipLaunchKernelGGL(layer_norm_kernel<1>, grid, block, 0, stream, x, skip, y, y_f8, f8_mul, gamma, beta, rows, C,
                       alpha, eps);
  } else if (C <= 1024) {
    hipLaunchKernelGGL(layer_norm_kernel<2>, grid, block, 0, stream, x, skip, y, y_f8, f8_mul, gamma, beta, rows, C,
                       alpha, eps);
  } else if (C <= 2048) {
    hipLaunchKernelGGL(layer_norm_kernel<4>, grid, block, 0, stream, x, skip, y, y_f8, f8_mul, gamma, beta, rows, C,
                       alpha, eps);
  } else {  // callers guarantee C <= 8192
    hipLaunchKernelGGL(layer_norm_kernel<16>, grid, block, 0, stream, x, skip, y, y_f8, f8_mul, gamma, beta, rows, C,
                       alpha, eps);
  }
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
template <int DEPTH, typename OutT>
__global__ __launch_bounds__(256, DEPTH == 32 ? 4 : DEPTH == 64 ? 3 : 1) void attention_kernel(const half_t* __restrict__ qkv,
                                                        const half_t* __restrict__ bias,
                                                        OutT* __restrict__ out, int total_heads, int heads,
                                                        float scale, float out_mul) {
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
    half8 kf[2], qf[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
      kf[t] = *reinterpret_cast<const half8*>(Kp + (long long)(32 * t + r) * ld + 16 * ks + 8 * g);
      qf[t] = *reinterpret_cast<const half8*>(Q + (long long)(32 * t + r) * ld + 16 * ks + 8 * g);
    }
#pragma unroll
    for (int mt = 0; mt < 2; mt++)
#pragma unroll
      for (int nt = 0; nt < 2; nt++)
        st[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[mt], qf[nt], st[mt][nt], 0, 0, 0);
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
        half8 bv = {0, 0, 0, 0, 0, 0, 0, 0};
        if (bh) bv = *reinterpret_cast<const half8*>(bh + ((nt * 2 + mt) * 2 + bp) * 512 + lane * 8);
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
    half8 pf[2];
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int e = 0; e < 8; e++) pf[nt][e] = (half_t)st[s / 2][nt][8 * (s % 2) + e];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      half8 vf;
#pragma unroll
      for (int e = 0; e < 8; e++) vf[e] = vs[(16 * s + 8 * (e / 4) + 4 * g + (e % 4)) * kVStride + dt * 32 + r];
#pragma unroll
      for (int nt = 0; nt < 2; nt++) o[nt][dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(pf[nt], vf, o[nt][dt], 0, 0, 0);
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
          *dst = (half_t)o[nt][dt][e];
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

int SmolgenBiasIndex(int q, int k) {
  int nt = q / 32, r = q % 32, mt = k / 32, kk = k % 32;
  int blk = kk / 8, g = (kk % 8) / 4, j = kk % 4;
  int lane = g * 32 + r;
  return ((nt * 2 + mt) * 2 + blk / 2) * 512 + lane * 8 + (blk % 2) * 4 + j;
}

namespace {
template <typename OutT>
void LaunchAttentionT(const half_t* qkv, const half_t* bias, OutT* out, float out_mul, int batch, int heads, int depth,
                      float scale, hipStream_t stream) {
  const int total = batch * heads;
  if (total <= 0) return;
  const dim3 grid((total + 3) / 4), block(256);
  switch (depth) {
    case 32:
      hipLaunchKernelGGL((attention_kernel<32, OutT>), grid, block, 0, stream, qkv, bias, out, total, heads, scale, out_mul);
      break;
    case 64:
      hipLaunchKernelGGL((attention_kernel<64, OutT>), grid, block, 0, stream, qkv, bias, out, total, heads, scale, out_mul);
      break;
    default:  // 128; callers check the depth
      hipLaunchKernelGGL((attention_kernel<128, OutT>), grid, block, 0, stream, qkv, bias, out, total, heads, scale, out_mul);
      break;
  }
}
}  // namespace

bool AttentionDepthSupported(int depth) { return depth == 32 || depth == 64 || depth == 128; }

void LaunchAttention(const half_t* qkv, const half_t* bias, half_t* out, int batch, int heads, float scale,
                     hipStream_t stream, int depth) {
  LaunchAttentionT<half_t>(qkv, bias, out, 1.0f, batch, heads, depth, scale, stream);
}

void LaunchAttentionF8Out(const half_t* qkv, const half_t* bias, uint8_t* out, float out_mul, int batch, int heads,
                          float scale, hipStream_t stream, int depth) {
  LaunchAttentionT<uint8_t>(qkv, bias, out, out_mul, batch, heads, depth, scale, stream);
}

// ---------------------------------------------------------------------------
// Attention policy tail.
// ---------------------------------------------------------------------------
namespace {
__global__ __launch_bounds__(256) void attn_policy_gather_kernel(const float* __restrict__ logits,
                                                                 const half_t* __restrict__ kq, int ld_kq,
                                                                 int key_off, const float* __restrict__ ppo, int pd,
                                                                 const int16_t* __restrict__ inv_map,
                                                                 float* __restrict__ out) {
  __shared__ float off[4][8];
  const int b = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // Promotion offsets off[i][j] = key row (56 + j) . ppo row i: wave i takes ppo row i against all eight keys,
  // with the loads of the eight products in flight together.
  {
    const int i = wave;
    const half_t* krow = kq + (long long)(b * 64 + 56) * ld_kq + key_off;
    float s[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    if (((pd | ld_kq | key_off) & 7) == 0) {
      for (int c = lane; c < pd / 8; c += 64) {
        const floatx4 p0 = *reinterpret_cast<const floatx4*>(ppo + (long long)i * pd + c * 8);
        const floatx4 p1 = *reinterpret_cast<const floatx4*>(ppo + (long long)i * pd + c * 8 + 4);
#pragma unroll
        for (int j = 0; j < 8; j++) {
          const half8 kv = *reinterpret_cast<const half8*>(krow + (long long)j * ld_kq + c * 8);
#pragma unroll
          for (int e = 0; e < 4; e++) s[j] += (float)kv[e] * p0[e] + (float)kv[4 + e] * p1[e];
        }
      }
    } else {
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

void LaunchAttnPolicyGather(const float* logits, const half_t* kq, int ld_kq, int key_off, const float* ppo, int pd,
                            const int16_t* inv_map, float* out, int batch, hipStream_t stream) {
  if (batch <= 0) return;
  hipLaunchKernelGGL(attn_policy_gather_kernel, dim3(batch), dim3(256), 0, stream, logits, kq, ld_kq, key_off, ppo,
                     pd, inv_map, out);
}

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
