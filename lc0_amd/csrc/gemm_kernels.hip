// Hand-written gfx950 (CDNA4, wave64) matrix-product kernels of the dense layers.
//
// What each kernel replaces in the reference CPU backend (file:line):
//   gemm_kernel, gemm_dma_kernel, gemm_rowpanel_kernel, gemm_f32_mfma_kernel
//                         FullyConnectedLayer::Forward1D  blas/fully_connected_layer.cc:49-106
//                         (+ bias/activation of shared/activation.cc:102-164), the per-sample
//                         Q.K^T sgemm of the attention policy (blas/network_blas.cc:850-872) and the
//                         winograd-domain products of WinogradConvolution3 (blas/winograd_convolution3.cc:47-324)
#include "kernel_common.h"

#include <algorithm>
#include <cmath>
#include <stdexcept>
#include <type_traits>
#include <utility>

namespace lc0mi {

namespace {

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
// ET: type of the operands (half_t or bf16_t); OutT: float, or ET.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, typename OutT, typename ET = half_t>
__global__ __launch_bounds__(256) void gemm_kernel(GemmArgs p) {
  using ev8 = typename Vec16<ET>::v8;
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
      ev8 af[TM], wf[TN];
#pragma unroll
      for (int i = 0; i < TM; i++)
        af[i] = *reinterpret_cast<const ev8*>(&As[(wm * WM + i * 32 + frag_row) * LDS_STRIDE + ks * 16 + frag_k]);
#pragma unroll
      for (int j = 0; j < TN; j++)
        wf[j] = *reinterpret_cast<const ev8*>(&Ws[(wn * WN + j * 32 + frag_row) * LDS_STRIDE + ks * 16 + frag_k]);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = Mfma32(wf[j], af[i], acc[i][j]);
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
              using ov4 = typename Vec16<OutT>::v4;
              ov4 h = {(OutT)v[0], (OutT)v[1], (OutT)v[2], (OutT)v[3]};
              *reinterpret_cast<ov4*>(dst) = h;
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
template <int RT, int CT, int U, typename OutT, typename ET = half_t>
__global__ __launch_bounds__(512) void gemm_rowpanel_kernel(GemmArgs p) {
  using ev8 = typename Vec16<ET>::v8;
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
    ev8 fa[RT][U], fw[CT][U];
#pragma unroll
    for (int u = 0; u < U; u++) {   // steps past the end re-read the last one (never used)
      const int k = min(st + u, s_end - 1) * 32;
#pragma unroll
      for (int t = 0; t < RT; t++) fa[t][u] = *reinterpret_cast<const ev8*>(a_row[t] + k);
#pragma unroll
      for (int c = 0; c < CT; c++) fw[c][u] = *reinterpret_cast<const ev8*>(w_row[c] + k);
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (st + u < s_end) {
#pragma unroll
        for (int t = 0; t < RT; t++)
#pragma unroll
          for (int c = 0; c < CT; c++)
            acc[t][c] = Mfma16(fw[c][u], fa[t][u], acc[t][c]);
      }
    }
  }
  if (wave == NW - 1 && K % 32 != 0) {   // K is a multiple of 8: the missing part of the last step is zero-filled
    const int k = steps * 32;
    const ev8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const bool in = k + 8 * g < K;
    ev8 fa[RT], fw[CT];
#pragma unroll
    for (int t = 0; t < RT; t++) fa[t] = in ? *reinterpret_cast<const ev8*>(a_row[t] + k) : zero;
#pragma unroll
    for (int c = 0; c < CT; c++) fw[c] = in ? *reinterpret_cast<const ev8*>(w_row[c] + k) : zero;
#pragma unroll
    for (int t = 0; t < RT; t++)
#pragma unroll
      for (int c = 0; c < CT; c++) acc[t][c] = Mfma16(fw[c], fa[t], acc[t][c]);
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

template <int STORES>
__device__ __forceinline__ void StoreOut16(void* dst, intx4 val) {
  if constexpr (STORES == 1) {
    __builtin_nontemporal_store(val, reinterpret_cast<intx4*>(dst));
  } else if constexpr (STORES == 2) {
    // (the no-op covers the wait states that the hardware needs between a store of more than eight bytes and a vector
    // ALU write to its data registers - two on this part; the compiler adds them after its own stores and does not
    // look into this one: without them the 256x128 tiles, which reuse the registers at once, stored wrong values)
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 2" ::"v"(dst), "v"(val) : "memory");
  } else {
    *reinterpret_cast<intx4*>(dst) = val;
  }
}

// The same kernel serves fp16 operands (Args = GemmArgs: BKB = 128 bytes = 64
// halves per tile row, v_mfma_f32_32x32x16_f16) and e4m3 operands (Args =
// GemmF8Args: 128 bytes = 128 values per row, v_mfma_f32_32x32x64_f8f6f4);
// BKB is the k-tile in bytes. OutT is half_t or uint8_t (e4m3, fp8 operands only).
// STORES: how the 16-byte output vectors are stored: 0 ordinary stores (the output stays in L2 and the memory-side
// cache), 1 streaming (non-temporal) stores, 2 stores written through at system scope (they leave L2 alone like the
// streaming ones, but what they wrote is found faster by the next kernel; plain epilogue only).
// EPI (fp16 operands only): 0 the plain epilogue, 1 the consumer and 2 the producer side of a folded layer norm
// (GemmArgs::row_stats / GemmArgs::skip).
// NSTAGES k-tiles of LDS: NSTAGES - 1 of them are in flight while one is consumed. Two stages suffice when the
// operands come from L2; with small tiles and operands that come from memory (a few hundred to a few thousand rows:
// every workgroup streams weights nobody has touched since the previous pass) a k-tile takes longer to arrive than
// to consume, and more stages hide that.
// ET (fp16-type operands only): half_t or bf16_t; the output type is then ET as well.
template <int BM, int BN, int BKB, int WAVES_M, int WAVES_N, typename Args, typename OutT, int STORES = 0,
          int EPI = 0, int NSTAGES = 2, typename ET = half_t>
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
  static_assert(EPI == 0 || (!F8 && std::is_same<OutT, half_t>::value && std::is_same<ET, half_t>::value),
                "folded layer norm: fp16 operands and output");
  static_assert(std::is_same<ET, half_t>::value || (!F8 && std::is_same<OutT, ET>::value),
                "bfloat16 operands go with bfloat16 output");
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
        using ev8 = typename Vec16<ET>::v8;
        ev8 af[TM], wf[TN];
#pragma unroll
        for (int i = 0; i < TM; i++) af[i] = *reinterpret_cast<const ev8*>(As + a_row + i * 32 * BKB + coff);
#pragma unroll
        for (int j = 0; j < TN; j++) wf[j] = *reinterpret_cast<const ev8*>(Ws + w_row + j * 32 * BKB + coff);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++) acc[i][j] = Mfma32(wf[j], af[i], acc[i][j]);
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
            using ov4 = typename Vec16<OutT>::v4;
            ov4 h;
#pragma unroll
            for (int rr = 0; rr < 4; rr++) h[rr] = (OutT)v[rr];
            *reinterpret_cast<ov4*>(dst) = h;
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
          // Columns past N (a last column tile that N does not fill) and rows past M hold products of clamped
          // operand rows: they are neither stored nor counted in the row statistics.
          if (!ok) s1 = s2 = 0.0f;
          if (ok) {
            half_t* dst = reinterpret_cast<half_t*>(C) + (long long)m * p.ldc + n;
            StoreOut16<STORES>(dst, __builtin_bit_cast(intx4, o));
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
            StoreOut16<STORES>(dst, val);
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

// The STORES instance for a launch: what the caller asked for (GemmArgs::out_stores), or by the size rule above.
inline int OutputStores(int requested, long long m, long long n, long long batch, int elem_bytes) {
  if (requested == kStoresCached) return 0;
  if (requested == kStoresStream) return 1;
  if (requested == kStoresWriteThrough) return 2;
  if (!StreamOutput(m, n, batch, elem_bytes)) return 0;
  return requested == kStoresAutoKeep ? 2 : 1;
}
// The same as a value of GemmArgs::out_stores that no longer depends on the size (for the parts of a product).
inline int ResolvedOutStores(const GemmArgs& a) {
  const int s = OutputStores(a.out_stores, a.M, a.N, a.batch, 2);
  return s == 1 ? kStoresStream : s == 2 ? kStoresWriteThrough : kStoresCached;
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int NSTAGES = 2>
void LaunchGemmDma(const GemmArgs& a, hipStream_t stream) {
  dim3 grid((a.M + BM - 1) / BM, (a.N + BN - 1) / BN, a.batch);
  const dim3 block(WAVES_M * WAVES_N * 64);
  auto launch = [&](auto stores_tag) {
    constexpr int S = decltype(stores_tag)::value;
    constexpr int SF = S == 2 ? 1 : S;   // (the folded-layer-norm epilogues know cached and streaming stores only)
    // The folded-layer-norm epilogues exist with two stages only (LaunchGemmDmaStaged sends them there).
    if (a.skip != nullptr) {
      if constexpr (((BN / WAVES_N) % 64 == 0 || BN / WAVES_N == 32) && NSTAGES == 2) {
        hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BK * 2, WAVES_M, WAVES_N, GemmArgs, half_t, SF, 2, 2>), grid, block, 0,
                           stream, a);
      }
    } else if (a.row_stats != nullptr) {
      if constexpr (NSTAGES == 2) {
        hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BK * 2, WAVES_M, WAVES_N, GemmArgs, half_t, SF, 1, 2>), grid, block, 0,
                           stream, a);
      }
    } else if (a.bf16) {
      hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BK * 2, WAVES_M, WAVES_N, GemmArgs, bf16_t, S, 0, NSTAGES, bf16_t>), grid,
                         block, 0, stream, a);
    } else {
      hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BK * 2, WAVES_M, WAVES_N, GemmArgs, half_t, S, 0, NSTAGES>), grid, block, 0,
                         stream, a);
    }
  };
  if constexpr (BM == 256) {
    const int stores = OutputStores(a.out_stores, a.M, a.N, a.batch, 2);
    if (stores == 1) return launch(std::integral_constant<int, 1>{});
    if (stores == 2) return launch(std::integral_constant<int, 2>{});
  }
  launch(std::integral_constant<int, 0>{});
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
    const int stores = OutputStores(a.out_stores, a.M, a.N, 1, a.out_f8 ? 1 : 2);
    auto launch = [&](auto stores_tag) {
      constexpr int S = decltype(stores_tag)::value;
      if (a.out_f8) {
        hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BKB, WAVES_M, WAVES_N, GemmF8Args, uint8_t, S>), grid, block, 0,
                           stream, a);
      } else {
        hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BKB, WAVES_M, WAVES_N, GemmF8Args, half_t, S>), grid, block, 0,
                           stream, a);
      }
    };
    if (stores == 1) return launch(std::integral_constant<int, 1>{});
    if (stores == 2) return launch(std::integral_constant<int, 2>{});
  }
  if (a.out_f8) {
    hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BKB, WAVES_M, WAVES_N, GemmF8Args, uint8_t, 0, 0, NSTAGES>), grid,
                       block, 0, stream, a);
  } else {
    hipLaunchKernelGGL((gemm_dma_kernel<BM, BN, BKB, WAVES_M, WAVES_N, GemmF8Args, half_t, 0, 0, NSTAGES>), grid,
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
  if (a.bf16) {
    if (a.out_f32) {
      hipLaunchKernelGGL((gemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, float, bf16_t>), grid, dim3(256), 0, stream, a);
    } else {
      hipLaunchKernelGGL((gemm_kernel<BM, BN, BK, WAVES_M, WAVES_N, bf16_t, bf16_t>), grid, dim3(256), 0, stream, a);
    }
  } else if (a.out_f32) {
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

enum GemmVariant { kDma256x256, kDma256x192, kDma256x128, kTile128, kTile64, kDma128x128, kRowPanel, kDma128x64, kUnused8 /* keeps the numbering of the variants after it */,
                   kDma128x32, kDma64x64 };

int g_variant_override = -1;

GemmVariant PickGemmVariantHalf(const GemmArgs& a);

// Fitted cost model of the five direct-to-LDS tile shapes, in microseconds per launch (see PickGemmVariantHalf).
struct FittedCosts {
  double t256, t192, t128, ts, t64;
  double Best() const { return std::min(std::min(std::min(t256, t192), std::min(t128, ts)), t64); }
};
inline bool InFittedDomain(const GemmArgs& a) { return a.batch == 1 && a.M >= 4096 && a.K >= 512 && a.N >= 512; }
inline FittedCosts FitCosts(int M, int N, int K) {
  const double kt = K / 64.0;
  auto tiles = [&](int bm, int bn) { return (double)((M + bm - 1) / bm) * (double)((N + bn - 1) / bn); };
  auto rounds_of = [](double x) {
    const double whole = std::floor(x + 1e-9), frac = x - whole;
    return whole + (frac > 1e-9 ? 0.55 + 0.45 * frac : 0.0);
  };
  FittedCosts c;
  c.t256 = 1.6 + rounds_of(tiles(256, 256) / 256.0) * (6.93 + 1.814 * kt);
  c.t192 = 1.6 + rounds_of(tiles(256, 192) / 256.0) * (5.37 + 1.444 * kt);
  c.t128 = 1.08 * (1.6 + rounds_of(tiles(256, 128) / 256.0) * (2.53 + 1.215 * kt));
  c.ts = 2.62 + std::max(0.5, tiles(128, 128) / 512.0) * (3.62 + 1.140 * kt);
  c.t64 = 1.19 + std::max(0.34, tiles(128, 64) / 768.0) * (2.75 + 1.119 * kt);
  return c;
}

// A large product whose tiles do not fill whole rounds of the 256 CUs, cut along its rows: the rows that make whole
// rounds of 256x256 (or 256x192) tiles go to one launch and the rest to a second launch on whatever shape suits it
// (20480x1024x1536: 87 us on 320 tiles of 256x256, one and a quarter rounds, or 78 us on 128x128 tiles, against
// 49 + 19 us for 16384 rows on one full round of large tiles and 4096 rows on small ones). Returns the rows of the
// first launch (0: one launch) when the model above prices the pair at least 3 % below the best single shape.
bool g_row_split = true;   // (profiling and tests switch it off through SetGemmRowSplit)
int PlanRowSplit(const GemmArgs& a, GemmVariant* first) {
  if (!g_row_split || g_variant_override >= 0 || !InFittedDomain(a) || a.out_f32 || a.split_k != 1 || a.K % 64 != 0 ||
      a.skip != nullptr || a.row_stats != nullptr) {
    return 0;
  }
  double best = FitCosts(a.M, a.N, a.K).Best() * 0.97;
  int best_m1 = 0;
  for (int v = 0; v < 2; v++) {
    const int bn = v == 0 ? 256 : 192;
    const int col_tiles = (a.N + bn - 1) / bn;
    if (col_tiles > 256) continue;
    const int rows_per_round = (256 / col_tiles) * 256;
    // (the rest stays inside the range of sizes the model was fitted on: cut at 2048 rows, a 15x1024 pass at 96
    //  positions lost 4 %)
    for (int m1 = rows_per_round; m1 + 4096 <= a.M; m1 += rows_per_round) {
      const FittedCosts top = FitCosts(m1, a.N, a.K);
      const double c = (v == 0 ? top.t256 : top.t192) + FitCosts(a.M - m1, a.N, a.K).Best() + 1.0;
      if (c < best) { best = c; best_m1 = m1; *first = v == 0 ? kDma256x256 : kDma256x192; }
    }
  }
  return best_m1;
}

// bfloat16 operands run every variant except the row panels (kept out to bound the number of kernel instances):
// such shapes take the register-staged 64x64 tiles.
GemmVariant PickGemmVariant(const GemmArgs& a) {
  const GemmVariant v = PickGemmVariantHalf(a);
  return (a.bf16 && v == kRowPanel) ? kTile64 : v;
}

GemmVariant PickGemmVariantHalf(const GemmArgs& a) {
  if (g_variant_override >= 0) {
    const bool dma_ok = !a.out_f32 && a.split_k == 1 && a.K % 64 == 0;
    const bool is_dma = g_variant_override <= kDma256x128 || g_variant_override == kDma128x128 ||
                        g_variant_override == kDma128x64 || g_variant_override == kDma128x32 ||
                        g_variant_override == kDma64x64;
    bool ok = is_dma ? dma_ok : (g_variant_override != kRowPanel || a.split_k == 1);
    if (g_variant_override == kUnused8) ok = false;
    if (ok) return static_cast<GemmVariant>(g_variant_override);
  }
  const long long tiles128 = (long long)((a.M + 127) / 128) * ((a.N + 127) / 128) * a.batch;
  if (!a.out_f32 && a.split_k == 1 && a.K % 64 == 0 && a.K >= 128 && a.N >= 128 && a.M >= (a.latency_first ? 256 : 1024) && tiles128 >= 64) {
    // Direct-to-LDS kernels. Cost = rounds over the 256 CUs x tile area x a measured cost per
    // output element and round (ns per element at K = 1024): 0.60 for 256x256, 0.61 for 256x192;
    // the two small shapes run two workgroups per CU, 0.68 (256x128) and 0.75 (128x128) per element
    // while sharing a CU, 0.84 and 0.95 when a single round leaves every workgroup alone on its CU.
    // One product of at least 4096 rows with K and N of at least 512 (the encoder layers of the attention bodies
    // from 64 positions up): a cost model in microseconds fitted to launches of all five shapes on 92 problems
    // (M 4096 to 65536, N 512 to 3072, K 512 to 2048; the variant it picks is 0.6 % behind the fastest measured one
    // on average and 9 % at worst, against 3 % and 24 % for the per-element model below, which was set when the
    // large tiles were slower than they are now). A round of the one-workgroup-per-CU shapes costs a fixed part and
    // a part per k-tile of 64; a last round that fills only a fraction f of the CUs costs 0.55 + 0.45 f of a full
    // one (its workgroups find L2 and the memory system less contended); the shapes that share a CU are priced by
    // tile count.
    if (InFittedDomain(a)) {
      const FittedCosts c = FitCosts(a.M, a.N, a.K);
      GemmVariant best = kDma256x256;
      double cost = c.t256;
      if (c.t192 < cost && a.skip == nullptr) { best = kDma256x192; cost = c.t192; }
      if (c.t128 < cost) { best = kDma256x128; cost = c.t128; }
      if (c.ts < cost) { best = kDma128x128; cost = c.ts; }
      if (c.t64 < cost) { best = kDma128x64; cost = c.t64; }
      return best;
    }
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
  // Many products that each fit a 64x64 tile (the policy head's Q.K^T per position) would leave three quarters of
  // every 128x128 tile empty (256 x 64x64x1024: 14.5 against 21.4 us).
  if (a.M <= 64 && a.N <= 64) return kTile64;
  const long long big_tiles = tiles128;
  return big_tiles >= 192 ? kTile128 : kTile64;
}
}  // namespace

void SetGemmVariantOverride(int variant) { g_variant_override = variant; }
void SetGemmRowSplit(bool on) { g_row_split = on; }

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
  if (a.bf16 && (a.skip != nullptr || a.row_stats != nullptr)) return false;
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

int GemmRowSplit(const GemmArgs& a) {
  GemmVariant first = kDma256x256;
  return PlanRowSplit(a, &first);
}

const char* GemmVariantName(const GemmArgs& a) {
  GemmVariant first = kDma256x256;
  if (PlanRowSplit(a, &first) > 0) return first == kDma256x256 ? "gemm_dma_256x256x64+rest" : "gemm_dma_256x192x64+rest";
  switch (PickGemmVariant(a)) {
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

namespace {
void LaunchGemmOne(const GemmArgs& a, hipStream_t stream) {
  switch (PickGemmVariant(a)) {
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
}  // namespace

void LaunchGemm(const GemmArgs& a, hipStream_t stream) {
  if (a.M <= 0 || a.N <= 0 || a.batch <= 0) return;
  if ((a.skip != nullptr || a.row_stats != nullptr) && !GemmSupportsNormFolding(a)) {
    throw std::runtime_error("LaunchGemm: no kernel variant with the folded layer-norm epilogue for this shape");
  }
  GemmVariant first = kDma256x256;
  const int m1 = PlanRowSplit(a, &first);
  if (m1 > 0) {
    GemmArgs top = a, rest = a;
    top.out_stores = rest.out_stores = ResolvedOutStores(a);   // as for the whole product
    top.M = m1;
    rest.M = a.M - m1;
    rest.A = a.A + static_cast<long long>(m1) * a.lda;
    rest.C = static_cast<half_t*>(a.C) + static_cast<long long>(m1) * a.ldc;
    if (first == kDma256x256) LaunchGemmDma<256, 256, 64, 2, 4>(top, stream);
    else LaunchGemmDma<256, 192, 64, 4, 2>(top, stream);
    LaunchGemmOne(rest, stream);   // (the rest is below one round of the large tiles: one launch)
    return;
  }
  LaunchGemmOne(a, stream);
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

}  // namespace lc0mi
