// Host-pointer wrappers around single kernels (see include/lc0mi_kernels.h).
#include "../../include/lc0mi_kernels.h"

#include <hip/hip_runtime.h>

#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "kernels.h"
#include "tables.h"
#include "weights.h"

extern "C" const char* lc0mi_last_error(void);
namespace lc0mi {
void SetLastError(const std::string& msg);
}

namespace {
using lc0mi::Error;
using lc0mi::half_t;

#define K_CHECK(expr)                                                                              \
  do {                                                                                             \
    hipError_t e__ = (expr);                                                                       \
    if (e__ != hipSuccess) throw Error(std::string("HIP error: ") + hipGetErrorString(e__) + " (" #expr ")"); \
  } while (0)

struct Dev {
  std::vector<void*> ptrs;
  ~Dev() {
    for (void* p : ptrs) (void)hipFree(p);
  }
  void* Alloc(size_t bytes) {
    void* p = nullptr;
    K_CHECK(hipMalloc(&p, bytes < 256 ? 256 : bytes));
    ptrs.push_back(p);
    return p;
  }
  template <typename T>
  T* Put(const T* host, size_t n) {
    T* d = static_cast<T*>(Alloc(n * sizeof(T)));
    if (n) K_CHECK(hipMemcpy(d, host, n * sizeof(T), hipMemcpyHostToDevice));
    return d;
  }
};

void RequireDevice() {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n == 0) throw Error("No HIP device is available.");
}

// Profiling hook (lc0mi_k_set_cold_cache): when > 0, every timed launch is preceded by an untimed copy of this many
// MiB, which pushes the kernel's operands out of L2 and the memory-side cache, as the kernels between two launches of
// the same kernel do inside a forward pass. Timed launches in a loop otherwise find their operands cached.
int g_cold_mib = 0;

template <typename F>
double TimeLaunches(int iters, F&& launch) {
  hipEvent_t a, b;
  K_CHECK(hipEventCreate(&a));
  K_CHECK(hipEventCreate(&b));
  launch();  // warm-up
  double total_ms = 0.0;
  if (g_cold_mib > 0) {
    const size_t bytes = (size_t)g_cold_mib << 20;
    void *src = nullptr, *dst = nullptr;
    K_CHECK(hipMalloc(&src, bytes));
    K_CHECK(hipMalloc(&dst, bytes));
    K_CHECK(hipMemset(src, 1, bytes));
    for (int i = 0; i < iters; i++) {
      lc0mi::LaunchCopy(src, dst, (long long)(bytes / 16), nullptr);
      K_CHECK(hipEventRecord(a, nullptr));
      launch();
      K_CHECK(hipEventRecord(b, nullptr));
      K_CHECK(hipEventSynchronize(b));
      float ms = 0;
      K_CHECK(hipEventElapsedTime(&ms, a, b));
      total_ms += ms;
    }
    (void)hipFree(src);
    (void)hipFree(dst);
  } else {
    K_CHECK(hipEventRecord(a, nullptr));
    for (int i = 0; i < iters; i++) launch();
    K_CHECK(hipEventRecord(b, nullptr));
    K_CHECK(hipEventSynchronize(b));
    float ms = 0;
    K_CHECK(hipEventElapsedTime(&ms, a, b));
    total_ms = ms;
  }
  (void)hipEventDestroy(a);
  (void)hipEventDestroy(b);
  return total_ms / iters;
}

template <typename F>
int Guard(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    lc0mi::SetLastError(e.what());
    return 1;
  }
}
}  // namespace

namespace {
// Test hook (lc0mi_k_set_bf16): the 16-bit buffers of the entry points that say so hold bfloat16 instead of half.
bool g_bf16 = false;
// Test hook (lc0mi_k_set_out_stores): the kind of output stores of lc0mi_k_gemm, lc0mi_k_gemm_f8 and lc0mi_k_layer_norm.
int g_out_stores = lc0mi::kStoresAuto;
}  // namespace

extern "C" {

int lc0mi_k_set_cold_cache(int mib) {
  g_cold_mib = mib > 0 ? mib : 0;
  return 0;
}

int lc0mi_k_set_out_stores(int kind) {
  return Guard([&] {
    if (kind < lc0mi::kStoresAuto || kind > lc0mi::kStoresWriteThrough) throw Error("bad kind of output stores");
    g_out_stores = kind;
  });
}

int lc0mi_k_set_bf16(int on) {
  g_bf16 = on != 0;
  return 0;
}

int lc0mi_k_gemm(const uint16_t* A, int lda, long long strideA, const uint16_t* W, int ldw, long long strideW,
                 const float* bias, int M, int N, int K, int batch, float scale, int act, int out_f32, void* C,
                 int ldc, long long strideC, int time_iters, double* ms) {
  return Guard([&] {
    RequireDevice();
    if (K % 8 || lda % 8 || ldw % 8 || strideA % 8 || strideW % 8) throw Error("K, lda, ldw and strides must be multiples of 8");
    if (M < 1 || N < 1 || batch < 1 || lda < K || ldw < K || ldc < N) throw Error("bad gemm shape");
    Dev dev;
    const size_t a_elems = (size_t)(batch - 1) * strideA + (size_t)(M - 1) * lda + K;
    const size_t w_elems = (size_t)(batch - 1) * strideW + (size_t)(N - 1) * ldw + K;
    const size_t c_elems = (size_t)(batch - 1) * strideC + (size_t)(M - 1) * ldc + N;
    const size_t c_size = out_f32 ? 4 : 2;
    lc0mi::GemmArgs g;
    g.A = reinterpret_cast<const half_t*>(dev.Put(A, a_elems)); g.lda = lda; g.strideA = strideA;
    g.W = reinterpret_cast<const half_t*>(dev.Put(W, w_elems)); g.ldw = ldw; g.strideW = strideW;
    g.C = dev.Alloc(c_elems * c_size); g.ldc = ldc; g.strideC = strideC;
    K_CHECK(hipMemcpy(g.C, C, c_elems * c_size, hipMemcpyHostToDevice));
    g.bias = bias ? dev.Put(bias, (size_t)N) : nullptr;
    g.M = M; g.N = N; g.K = K; g.batch = batch; g.scale = scale; g.act = act; g.out_f32 = out_f32 != 0;
    g.bf16 = g_bf16;
    g.out_stores = g_out_stores;
    lc0mi::LaunchGemm(g, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(C, g.C, c_elems * c_size, hipMemcpyDeviceToHost));
    if (time_iters > 0 && ms) *ms = TimeLaunches(time_iters, [&] { lc0mi::LaunchGemm(g, nullptr); });
  });
}

const char* lc0mi_k_gemm_variant_name(int M, int N, int K, int batch, int latency_first) {
  lc0mi::GemmArgs g;
  g.M = M; g.N = N; g.K = K; g.batch = batch < 1 ? 1 : batch;
  g.lda = K; g.ldw = K; g.ldc = N;
  g.latency_first = latency_first != 0;
  return lc0mi::GemmVariantName(g);
}

void lc0mi_k_set_gemm_row_split(int on) { lc0mi::SetGemmRowSplit(on != 0); }

int lc0mi_k_gemm_row_split(int M, int N, int K) {
  lc0mi::GemmArgs g;
  g.M = M; g.N = N; g.K = K; g.batch = 1;
  g.lda = K; g.ldw = K; g.ldc = N;
  return lc0mi::GemmRowSplit(g);
}

int lc0mi_k_gemm_norm_producer(const uint16_t* A, int lda, const uint16_t* W, int ldw, const float* bias, int M, int N,
                               int K, float scale, const uint16_t* skip, const float* skip_stats, int skip_parts,
                               const float* skip_gamma, const float* skip_beta, float eps, uint16_t* U,
                               float* stats_out, int stats_cap, int* parts_out, int time_iters, double* ms) {
  return Guard([&] {
    RequireDevice();
    if (K % 8 || lda % 8 || ldw % 8 || N % 8) throw Error("K, lda, ldw and N must be multiples of 8");
    if (M < 1 || N < 1 || lda < K || ldw < K) throw Error("bad gemm shape");
    Dev dev;
    lc0mi::GemmArgs g;
    g.A = reinterpret_cast<const half_t*>(dev.Put(A, (size_t)(M - 1) * lda + K)); g.lda = lda;
    g.W = reinterpret_cast<const half_t*>(dev.Put(W, (size_t)(N - 1) * ldw + K)); g.ldw = ldw;
    // the residual is added in place, as the network does it
    half_t* u = reinterpret_cast<half_t*>(const_cast<uint16_t*>(dev.Put(skip, (size_t)M * N)));
    g.C = u; g.ldc = N;
    g.skip = u; g.ldskip = N;
    g.bias = bias ? dev.Put(bias, (size_t)N) : nullptr;
    g.M = M; g.N = N; g.K = K; g.scale = scale; g.act = 3;
    if (skip_stats != nullptr) {
      g.skip_stats = dev.Put(skip_stats, (size_t)M * skip_parts * 2);
      g.skip_parts = skip_parts;
      g.skip_gamma = dev.Put(skip_gamma, (size_t)N);
      g.skip_beta = dev.Put(skip_beta, (size_t)N);
    }
    g.norm_n = N; g.norm_eps = eps;
    if (!lc0mi::GemmSupportsNormFolding(g)) throw Error("no kernel variant with the producer epilogue for this shape");
    const int parts = lc0mi::GemmStatsParts(g);
    if (parts < 1 || (size_t)M * parts * 2 > (size_t)stats_cap) throw Error("stats_out is too small");
    float* d_stats = static_cast<float*>(dev.Alloc((size_t)M * parts * 2 * sizeof(float)));
    g.stats_out = d_stats;
    *parts_out = parts;
    lc0mi::LaunchGemm(g, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(U, u, (size_t)M * N * 2, hipMemcpyDeviceToHost));
    K_CHECK(hipMemcpy(stats_out, d_stats, (size_t)M * parts * 2 * sizeof(float), hipMemcpyDeviceToHost));
    if (time_iters > 0 && ms) *ms = TimeLaunches(time_iters, [&] { lc0mi::LaunchGemm(g, nullptr); });
  });
}

int lc0mi_k_gemm_norm_consumer(const uint16_t* U, int ldu, const uint16_t* W, int ldw, const float* col_c,
                               const float* bias, int M, int N, int K, const float* stats, int parts, float eps,
                               int act, int latency_first, uint16_t* C, int ldc, int time_iters, double* ms) {
  return Guard([&] {
    RequireDevice();
    if (K % 8 || ldu % 8 || ldw % 8) throw Error("K, ldu and ldw must be multiples of 8");
    if (M < 1 || N < 1 || ldu < K || ldw < K || ldc < N || parts < 1 || col_c == nullptr) throw Error("bad gemm shape");
    Dev dev;
    lc0mi::GemmArgs g;
    g.A = reinterpret_cast<const half_t*>(dev.Put(U, (size_t)(M - 1) * ldu + K)); g.lda = ldu;
    g.W = reinterpret_cast<const half_t*>(dev.Put(W, (size_t)(N - 1) * ldw + K)); g.ldw = ldw;
    const size_t c_elems = (size_t)(M - 1) * ldc + N;
    g.C = dev.Alloc(c_elems * 2); g.ldc = ldc;
    K_CHECK(hipMemcpy(g.C, C, c_elems * 2, hipMemcpyHostToDevice));
    g.bias = bias ? dev.Put(bias, (size_t)N) : nullptr;
    g.col_c = dev.Put(col_c, (size_t)N);
    g.row_stats = dev.Put(stats, (size_t)M * parts * 2);
    g.row_parts = parts;
    g.norm_n = K; g.norm_eps = eps;
    g.M = M; g.N = N; g.K = K; g.act = act;
    g.latency_first = latency_first != 0;
    if (!lc0mi::GemmSupportsNormFolding(g)) throw Error("no kernel variant with the consumer epilogue for this shape");
    lc0mi::LaunchGemm(g, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(C, g.C, c_elems * 2, hipMemcpyDeviceToHost));
    if (time_iters > 0 && ms) *ms = TimeLaunches(time_iters, [&] { lc0mi::LaunchGemm(g, nullptr); });
  });
}

int lc0mi_k_gemm_splitk(const uint16_t* A, int lda, const uint16_t* W, int ldw, const float* bias, int M, int N,
                        int K, int split_k, float scale, float* C, int ldc) {
  return Guard([&] {
    RequireDevice();
    if (K % 8 || lda % 8 || ldw % 8) throw Error("K, lda and ldw must be multiples of 8");
    if (M < 1 || N < 1 || split_k < 1 || lda < K || ldw < K || ldc < N) throw Error("bad gemm shape");
    Dev dev;
    lc0mi::GemmArgs g;
    g.A = reinterpret_cast<const half_t*>(dev.Put(A, (size_t)(M - 1) * lda + K)); g.lda = lda;
    g.W = reinterpret_cast<const half_t*>(dev.Put(W, (size_t)(N - 1) * ldw + K)); g.ldw = ldw;
    const size_t c_elems = (size_t)M * ldc;
    float* dC = static_cast<float*>(dev.Alloc(c_elems * 4 * split_k));
    g.C = dC; g.ldc = ldc;
    g.bias = bias ? dev.Put(bias, (size_t)N) : nullptr;
    g.M = M; g.N = N; g.K = K; g.scale = scale; g.act = 3; g.out_f32 = true;
    g.split_k = split_k; g.split_stride = (long long)c_elems;
    lc0mi::LaunchGemm(g, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    // Add the slices on the host in slice order.
    std::vector<float> part(c_elems * split_k);
    K_CHECK(hipMemcpy(part.data(), dC, part.size() * 4, hipMemcpyDeviceToHost));
    for (int m = 0; m < M; m++)
      for (int n = 0; n < N; n++) {
        float s = 0.0f;
        for (int z = 0; z < split_k; z++) s += part[(size_t)z * c_elems + (size_t)m * ldc + n];
        C[(size_t)m * ldc + n] = s;
      }
  });
}

int lc0mi_k_layer_norm_rows(const float* x_f32, const uint16_t* x_f16, int pre_act, const uint16_t* skip,
                            const float* gamma, const float* beta, int rows, int C, float alpha, float eps,
                            uint16_t* y) {
  return Guard([&] {
    RequireDevice();
    if (C % 8 || C < 8 || C > 8192 || rows < 1) throw Error("bad layer norm shape");
    if ((x_f32 == nullptr) == (x_f16 == nullptr)) throw Error("exactly one of x_f32 / x_f16 must be given");
    Dev dev;
    const size_t n = (size_t)rows * C;
    const float* dxf = x_f32 ? dev.Put(x_f32, n) : nullptr;
    const half_t* dxh = x_f16 ? reinterpret_cast<const half_t*>(dev.Put(x_f16, n)) : nullptr;
    const half_t* ds = skip ? reinterpret_cast<const half_t*>(dev.Put(skip, n)) : nullptr;
    auto* dy = reinterpret_cast<half_t*>(dev.Alloc(n * 2));
    float* dg = dev.Put(gamma, (size_t)C);
    float* db = dev.Put(beta, (size_t)C);
    lc0mi::LaunchLayerNormRows(dxf, dxf ? 1 : 0, 0, dxh, pre_act, ds, dy, dg, db, rows, C, alpha, eps, nullptr, g_bf16);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(y, dy, n * 2, hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_set_gemm_variant(int variant) {
  lc0mi::SetGemmVariantOverride(variant);
  return 0;
}

int lc0mi_k_gemm_f32(const float* A, int lda, const float* W, int ldw, const float* bias, int M, int N, int K,
                     float scale, int act, float* C, int ldc) {
  return Guard([&] {
    RequireDevice();
    if (K % 4 || lda % 4 || ldw % 4) throw Error("K, lda and ldw must be multiples of 4");
    if (M < 1 || N < 1 || lda < K || ldw < K || ldc < N) throw Error("bad gemm shape");
    Dev dev;
    lc0mi::GemmArgsF32 g;
    g.A = dev.Put(A, (size_t)(M - 1) * lda + K); g.lda = lda;
    g.W = dev.Put(W, (size_t)(N - 1) * ldw + K); g.ldw = ldw;
    const size_t c_elems = (size_t)(M - 1) * ldc + N;
    g.C = dev.Put(C, c_elems); g.ldc = ldc;
    g.bias = bias ? dev.Put(bias, (size_t)N) : nullptr;
    g.M = M; g.N = N; g.K = K; g.scale = scale; g.act = act;
    lc0mi::LaunchGemmF32(g, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(C, g.C, c_elems * sizeof(float), hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_layer_norm(const uint16_t* x, const uint16_t* skip, const float* gamma, const float* beta, int rows,
                       int C, float alpha, float eps, uint16_t* y, int time_iters, double* ms) {
  return Guard([&] {
    RequireDevice();
    if (C % 8 || C < 8 || C > 8192 || rows < 1) throw Error("bad layer norm shape");
    Dev dev;
    const size_t n = (size_t)rows * C;
    auto* dx = reinterpret_cast<half_t*>(dev.Put(x, n));
    auto* ds = skip ? reinterpret_cast<half_t*>(dev.Put(skip, n)) : nullptr;
    auto* dy = reinterpret_cast<half_t*>(dev.Alloc(n * 2));
    float* dg = dev.Put(gamma, (size_t)C);
    float* db = dev.Put(beta, (size_t)C);
    const bool through = g_out_stores == lc0mi::kStoresWriteThrough;
    lc0mi::LaunchLayerNorm(dx, ds, dy, dg, db, rows, C, alpha, eps, nullptr, nullptr, 1.0f, g_bf16, through);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(y, dy, n * 2, hipMemcpyDeviceToHost));
    if (time_iters > 0 && ms) {
      *ms = TimeLaunches(time_iters, [&] {
        lc0mi::LaunchLayerNorm(dx, ds, dy, dg, db, rows, C, alpha, eps, nullptr, nullptr, 1.0f, g_bf16, through);
      });
    }
  });
}

int lc0mi_k_attention(const uint16_t* qkv, const uint16_t* bias, int batch, int heads, int depth, float scale,
                      uint16_t* out, int time_iters, double* ms) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1 || heads < 1 || !lc0mi::AttentionDepthSupported(depth)) throw Error("bad attention shape");
    Dev dev;
    const int d = heads * depth;
    auto* dq = reinterpret_cast<half_t*>(dev.Put(qkv, (size_t)batch * 64 * 3 * d));
    half_t* db = nullptr;
    if (bias) {
      std::vector<uint16_t> perm((size_t)batch * heads * 4096);
      for (size_t bh = 0; bh < (size_t)batch * heads; bh++)
        for (int q = 0; q < 64; q++)
          for (int k = 0; k < 64; k++) perm[bh * 4096 + lc0mi::SmolgenBiasIndex(q, k)] = bias[bh * 4096 + q * 64 + k];
      db = reinterpret_cast<half_t*>(dev.Put(perm.data(), perm.size()));
    }
    auto* dout = reinterpret_cast<half_t*>(dev.Alloc((size_t)batch * 64 * d * 2));
    lc0mi::LaunchAttention(dq, db, dout, batch, heads, scale, nullptr, depth, g_bf16);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(out, dout, (size_t)batch * 64 * d * 2, hipMemcpyDeviceToHost));
    if (time_iters > 0 && ms) {
      *ms = TimeLaunches(time_iters, [&] { lc0mi::LaunchAttention(dq, db, dout, batch, heads, scale, nullptr, depth); });
    }
  });
}

int lc0mi_k_attention_generic(int dtype, const void* qkv, const void* bias, int batch, int heads, int depth, float scale,
                              void* out) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1 || heads < 1 || !lc0mi::AttentionGenericDepthSupported(depth) || dtype < 0 || dtype > 2) {
      throw Error("bad attention shape");
    }
    Dev dev;
    const size_t es = dtype == 2 ? 4 : 2;
    const size_t d = (size_t)heads * depth;
    void* dq = dev.Alloc((size_t)batch * 64 * 3 * d * es);
    K_CHECK(hipMemcpy(dq, qkv, (size_t)batch * 64 * 3 * d * es, hipMemcpyHostToDevice));
    void* db = nullptr;
    if (bias) {   // natural [b][h][q][k] order in, the kernels' order on the device
      std::vector<char> perm((size_t)batch * heads * 4096 * es);
      const char* src = static_cast<const char*>(bias);
      for (size_t bh = 0; bh < (size_t)batch * heads; bh++)
        for (int q = 0; q < 64; q++)
          for (int k = 0; k < 64; k++)
            std::memcpy(&perm[(bh * 4096 + lc0mi::SmolgenBiasIndex(q, k)) * es], src + (bh * 4096 + q * 64 + k) * es, es);
      db = dev.Alloc(perm.size());
      K_CHECK(hipMemcpy(db, perm.data(), perm.size(), hipMemcpyHostToDevice));
    }
    void* dout = dev.Alloc((size_t)batch * 64 * d * es);
    if (dtype == 2) {
      lc0mi::LaunchAttentionGeneric(static_cast<const float*>(dq), static_cast<const float*>(db), static_cast<float*>(dout),
                                    batch, heads, depth, scale, nullptr);
    } else if (dtype == 1) {
      lc0mi::LaunchAttentionGeneric(static_cast<const lc0mi::bf16_t*>(dq), static_cast<const lc0mi::bf16_t*>(db),
                                    static_cast<lc0mi::bf16_t*>(dout), batch, heads, depth, scale, nullptr);
    } else {
      lc0mi::LaunchAttentionGeneric(static_cast<const half_t*>(dq), static_cast<const half_t*>(db),
                                    static_cast<half_t*>(dout), batch, heads, depth, scale, nullptr);
    }
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(out, dout, (size_t)batch * 64 * d * es, hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_layer_norm_generic(int dtype, const void* x, const void* skip, const float* gamma, const float* beta, int rows,
                               int C, float alpha, float eps, int pre_act, void* y) {
  return Guard([&] {
    RequireDevice();
    if (rows < 1 || C < 1 || dtype < 0 || dtype > 2) throw Error("bad layer norm shape");
    Dev dev;
    const size_t bytes = (size_t)rows * C * (dtype == 2 ? 4 : 2);
    void* dx = dev.Alloc(bytes);
    K_CHECK(hipMemcpy(dx, x, bytes, hipMemcpyHostToDevice));
    void* ds = nullptr;
    if (skip) {
      ds = dev.Alloc(bytes);
      K_CHECK(hipMemcpy(ds, skip, bytes, hipMemcpyHostToDevice));
    }
    const float* dg = dev.Put(gamma, (size_t)C);
    const float* db = dev.Put(beta, (size_t)C);
    void* dy = dev.Alloc(bytes);
    if (dtype == 2) {
      lc0mi::LaunchLayerNormGeneric(static_cast<const float*>(dx), static_cast<const float*>(ds), static_cast<float*>(dy), dg,
                                    db, rows, C, alpha, eps, pre_act, nullptr);
    } else if (dtype == 1) {
      lc0mi::LaunchLayerNormGeneric(static_cast<const lc0mi::bf16_t*>(dx), static_cast<const lc0mi::bf16_t*>(ds),
                                    static_cast<lc0mi::bf16_t*>(dy), dg, db, rows, C, alpha, eps, pre_act, nullptr);
    } else {
      lc0mi::LaunchLayerNormGeneric(static_cast<const half_t*>(dx), static_cast<const half_t*>(ds),
                                    static_cast<half_t*>(dy), dg, db, rows, C, alpha, eps, pre_act, nullptr);
    }
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(y, dy, bytes, hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_expand_planes_attn(const uint64_t* masks, const float* values, int batch, int ld, uint16_t* out,
                               int time_iters, double* ms) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1 || ld < 176) throw Error("bad expand shape");
    Dev dev;
    uint64_t* dm = dev.Put(masks, (size_t)batch * 112);
    float* dv = dev.Put(values, (size_t)batch * 112);
    const std::vector<float>& pe = lc0mi::PosEncoding();
    std::vector<half_t> peh(pe.size());
    for (size_t i = 0; i < pe.size(); i++) peh[i] = (half_t)pe[i];
    half_t* dpe = dev.Put(peh.data(), peh.size());
    auto* dout = reinterpret_cast<half_t*>(dev.Alloc((size_t)batch * 64 * ld * 2));
    lc0mi::LaunchExpandPlanesAttn<half_t>(dm, dv, dpe, dout, ld, batch, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(out, dout, (size_t)batch * 64 * ld * 2, hipMemcpyDeviceToHost));
    if (time_iters > 0 && ms) {
      *ms = TimeLaunches(time_iters, [&] { lc0mi::LaunchExpandPlanesAttn<half_t>(dm, dv, dpe, dout, ld, batch, nullptr); });
    }
  });
}

int lc0mi_k_expand_planes_nchw(const uint64_t* masks, const float* values, int batch, float* out) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1) throw Error("bad expand shape");
    Dev dev;
    uint64_t* dm = dev.Put(masks, (size_t)batch * 112);
    float* dv = dev.Put(values, (size_t)batch * 112);
    auto* dout = static_cast<float*>(dev.Alloc((size_t)batch * 112 * 64 * 4));
    lc0mi::LaunchExpandPlanesNchw<float>(dm, dv, dout, batch, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(out, dout, (size_t)batch * 112 * 64 * 4, hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_attn_policy_gather(const float* logits, const uint16_t* keys, const float* ppo, int pd, int batch,
                               float* out) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1 || pd < 1) throw Error("bad policy shape");
    Dev dev;
    float* dl = dev.Put(logits, (size_t)batch * 4096);
    auto* dk = reinterpret_cast<half_t*>(dev.Put(keys, (size_t)batch * 64 * pd));
    float* dp = dev.Put(ppo, (size_t)4 * pd);
    const auto& inv = lc0mi::AttnPolicyInverseMap();
    int16_t* di = dev.Put(inv.data(), inv.size());
    auto* dout = static_cast<float*>(dev.Alloc((size_t)batch * 1858 * 4));
    lc0mi::LaunchAttnPolicyGather(dl, dk, pd, 0, dp, pd, di, dout, batch, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(out, dout, (size_t)batch * 1858 * 4, hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_legal_softmax(const float* policy, const int* offsets, const uint16_t* ids, float inv_temperature,
                          int batch, float* probs) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1) throw Error("bad batch");
    if (offsets[0] != 0) throw Error("offsets must start at 0");
    for (int b = 0; b < batch; b++) {
      const int n = offsets[b + 1] - offsets[b];
      if (n < 0 || n > lc0mi::kMaxLegalMoves) throw Error("bad move count");
    }
    const int total = offsets[batch];
    for (int i = 0; i < total; i++) {
      if (ids[i] >= 1858) throw Error("move id out of range");
    }
    Dev dev;
    float* dp = dev.Put(policy, (size_t)batch * 1858);
    int* doff = dev.Put(offsets, (size_t)batch + 1);
    uint16_t* di = dev.Put(ids, (size_t)total);
    auto* dout = static_cast<float*>(dev.Alloc((size_t)std::max(total, 1) * 4));
    lc0mi::LaunchLegalSoftmax(dp, doff, di, inv_temperature, dout, batch, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    if (total > 0) K_CHECK(hipMemcpy(probs, dout, (size_t)total * 4, hipMemcpyDeviceToHost));
  });
}

}  // extern "C"

namespace {
template <typename T>
void WinogradConvHost(const float* x, const float* filter, const float* bias, const float* skip, const float* se_w1,
                      const float* se_b1, const float* se_w2, const float* se_b2, int se_k, int batch, int cin,
                      int cout, int act, float* out, float* v_fused, float* v_separate) {
  Dev dev;
  const int ld = (cin + 7) / 8 * 8;
  const size_t nx = (size_t)batch * 64 * cin, no = (size_t)batch * 64 * cout;
  std::vector<T> hx(nx);
  for (size_t i = 0; i < nx; i++) hx[i] = (T)x[i];
  T* dx = dev.Put(hx.data(), nx);
  T* dskip = nullptr;
  if (skip) {
    std::vector<T> hs(no);
    for (size_t i = 0; i < no; i++) hs[i] = (T)skip[i];
    dskip = dev.Put(hs.data(), no);
  }
  std::vector<float> u((size_t)36 * cout * ld);
  lc0mi::WinogradFilterTransform4x4(filter, cout, cin, ld, u.data());
  std::vector<T> ut(u.size());
  for (size_t i = 0; i < u.size(); i++) ut[i] = (T)u[i];
  T* du = dev.Put(ut.data(), ut.size());
  float* dbias = dev.Put(bias, (size_t)cout);
  float *w1 = nullptr, *b1 = nullptr, *w2 = nullptr, *b2 = nullptr;
  if (se_k > 0) {
    w1 = dev.Put(se_w1, (size_t)se_k * cout); b1 = dev.Put(se_b1, (size_t)se_k);
    std::vector<float> w2t((size_t)2 * cout * se_k);   // [2C][K] -> [K][2C], the layout the kernels read
    for (int o = 0; o < 2 * cout; o++)
      for (int k = 0; k < se_k; k++) w2t[(size_t)k * 2 * cout + o] = se_w2[(size_t)o * se_k + k];
    w2 = dev.Put(w2t.data(), w2t.size()); b2 = dev.Put(se_b2, (size_t)2 * cout);
  }
  const int tiles = batch * 4;
  T* dv = static_cast<T*>(dev.Alloc(sizeof(T) * 36 * tiles * ld));
  K_CHECK(hipMemset(dv, 0, sizeof(T) * 36 * tiles * ld));
  T* dm = static_cast<T*>(dev.Alloc(sizeof(T) * 36 * tiles * cout));   // winograd-domain products, in the tower's type
  T* dout = static_cast<T*>(dev.Alloc(sizeof(T) * no));
  lc0mi::LaunchWinogradInputTransform<T>(dx, dv, batch, cin, ld, nullptr);
  if constexpr (sizeof(T) == 2) {
    lc0mi::GemmArgs g;
    g.A = dv; g.lda = ld; g.strideA = (long long)tiles * ld;
    g.W = du; g.ldw = ld; g.strideW = (long long)cout * ld;
    g.C = dm; g.ldc = cout; g.strideC = (long long)tiles * cout;
    g.M = tiles; g.N = cout; g.K = ld; g.batch = 36; g.out_f32 = false;
    lc0mi::LaunchGemm(g, nullptr);
  } else {
    lc0mi::GemmArgsF32 g;
    g.A = dv; g.lda = ld; g.strideA = (long long)tiles * ld;
    g.W = du; g.ldw = ld; g.strideW = (long long)cout * ld;
    g.C = dm; g.ldc = cout; g.strideC = (long long)tiles * cout;
    g.M = tiles; g.N = cout; g.K = ld; g.batch = 36;
    lc0mi::LaunchGemmF32(g, nullptr);
  }
  // Optionally also the next convolution's transformed input, once from the fused kernel and
  // once from the stand-alone input transform applied to the output (they must be identical).
  T *dvf = nullptr, *dvs = nullptr;
  const size_t nv = (size_t)36 * tiles * cout;
  if (v_fused) {
    if (cout % 8 || !lc0mi::WinogradFusedInputTransform(cout, sizeof(T), se_k)) throw Error("shape cannot be fused");
    dvf = static_cast<T*>(dev.Alloc(sizeof(T) * nv));
    dvs = static_cast<T*>(dev.Alloc(sizeof(T) * nv));
  }
  lc0mi::LaunchWinogradOutputTransform<T, T>(dm, dbias, dskip, w1, b1, w2, b2, se_k, dout, batch, cout, act, nullptr,
                                             dvf, cout);
  if (v_fused) lc0mi::LaunchWinogradInputTransform<T>(dout, dvs, batch, cout, cout, nullptr);
  K_CHECK(hipDeviceSynchronize());
  K_CHECK(hipGetLastError());
  std::vector<T> ho(no);
  K_CHECK(hipMemcpy(ho.data(), dout, sizeof(T) * no, hipMemcpyDeviceToHost));
  for (size_t i = 0; i < no; i++) out[i] = (float)ho[i];
  if (v_fused) {
    std::vector<T> hv(nv);
    K_CHECK(hipMemcpy(hv.data(), dvf, sizeof(T) * nv, hipMemcpyDeviceToHost));
    for (size_t i = 0; i < nv; i++) v_fused[i] = (float)hv[i];
    K_CHECK(hipMemcpy(hv.data(), dvs, sizeof(T) * nv, hipMemcpyDeviceToHost));
    for (size_t i = 0; i < nv; i++) v_separate[i] = (float)hv[i];
  }
}
}  // namespace

extern "C" {

int lc0mi_k_winograd_conv(const float* x, const float* filter, const float* bias, const float* skip,
                          const float* se_w1, const float* se_b1, const float* se_w2, const float* se_b2, int se_k,
                          int batch, int cin, int cout, int act, int use_fp16, float* out, float* v_fused,
                          float* v_separate) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1 || cin < 1 || cout < 1 || cout > 1024 || se_k < 0 || se_k > 256) throw Error("bad convolution shape");
    if ((v_fused == nullptr) != (v_separate == nullptr)) throw Error("v_fused and v_separate go together");
    if (use_fp16) {
      WinogradConvHost<half_t>(x, filter, bias, skip, se_w1, se_b1, se_w2, se_b2, se_k, batch, cin, cout, act, out,
                               v_fused, v_separate);
    } else {
      WinogradConvHost<float>(x, filter, bias, skip, se_w1, se_b1, se_w2, se_b2, se_k, batch, cin, cout, act, out,
                              v_fused, v_separate);
    }
  });
}

int lc0mi_k_gemm_f8(const uint8_t* A, int lda, const uint8_t* W, int ldw, const float* col_scale, const float* bias,
                    int M, int N, int K, int act, int out_f8, float out_mul, void* C, int ldc, int time_iters,
                    double* ms) {
  return Guard([&] {
    RequireDevice();
    if (K % 128 || lda % 16 || ldw % 16) throw Error("K must be a multiple of 128, lda and ldw of 16");
    if (M < 1 || N < 1 || lda < K || ldw < K || ldc < N || !col_scale) throw Error("bad gemm shape");
    Dev dev;
    lc0mi::GemmF8Args g;
    g.A = dev.Put(A, (size_t)(M - 1) * lda + K); g.lda = lda;
    g.W = dev.Put(W, (size_t)(N - 1) * ldw + K); g.ldw = ldw;
    const size_t c_bytes = ((size_t)(M - 1) * ldc + N) * (out_f8 ? 1 : 2);
    g.C = dev.Alloc(c_bytes); g.ldc = ldc;
    K_CHECK(hipMemcpy(g.C, C, c_bytes, hipMemcpyHostToDevice));
    g.col_scale = dev.Put(col_scale, (size_t)N);
    g.bias = bias ? dev.Put(bias, (size_t)N) : nullptr;
    g.M = M; g.N = N; g.K = K; g.act = act; g.out_f8 = out_f8 != 0; g.out_mul = out_mul;
    g.out_stores = g_out_stores;
    lc0mi::LaunchGemmF8(g, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(C, g.C, c_bytes, hipMemcpyDeviceToHost));
    if (time_iters > 0 && ms) *ms = TimeLaunches(time_iters, [&] { lc0mi::LaunchGemmF8(g, nullptr); });
  });
}

int lc0mi_k_quantize_f8(const uint16_t* x, long long n, float mul, uint8_t* y) {
  return Guard([&] {
    RequireDevice();
    if (n < 8 || n % 8) throw Error("n must be a positive multiple of 8");
    Dev dev;
    auto* dx = reinterpret_cast<half_t*>(dev.Put(x, (size_t)n));
    auto* dy = static_cast<uint8_t*>(dev.Alloc((size_t)n));
    lc0mi::LaunchQuantizeF8(dx, dy, n, mul, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(y, dy, (size_t)n, hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_layer_norm_f8(const uint16_t* x, const uint16_t* skip, const float* gamma, const float* beta, int rows,
                          int C, float alpha, float eps, float f8_mul, uint16_t* y, uint8_t* y_f8) {
  return Guard([&] {
    RequireDevice();
    if (C % 8 || C < 8 || C > 8192 || rows < 1) throw Error("bad layer norm shape");
    Dev dev;
    const size_t n = (size_t)rows * C;
    auto* dx = reinterpret_cast<half_t*>(dev.Put(x, n));
    auto* ds = skip ? reinterpret_cast<half_t*>(dev.Put(skip, n)) : nullptr;
    auto* dy = reinterpret_cast<half_t*>(dev.Alloc(n * 2));
    auto* dq = static_cast<uint8_t*>(dev.Alloc(n));
    float* dg = dev.Put(gamma, (size_t)C);
    float* db = dev.Put(beta, (size_t)C);
    lc0mi::LaunchLayerNorm(dx, ds, dy, dg, db, rows, C, alpha, eps, nullptr, dq, f8_mul);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(y, dy, n * 2, hipMemcpyDeviceToHost));
    K_CHECK(hipMemcpy(y_f8, dq, n, hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_attention_f8(const uint16_t* qkv, const uint16_t* bias, int batch, int heads, float scale, float out_mul,
                         uint8_t* out) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1 || heads < 1) throw Error("bad attention shape");
    Dev dev;
    const int d = heads * 32;
    auto* dq = reinterpret_cast<half_t*>(dev.Put(qkv, (size_t)batch * 64 * 3 * d));
    half_t* db = nullptr;
    if (bias) {
      std::vector<uint16_t> perm((size_t)batch * heads * 4096);
      for (size_t bh = 0; bh < (size_t)batch * heads; bh++)
        for (int q = 0; q < 64; q++)
          for (int k = 0; k < 64; k++) perm[bh * 4096 + lc0mi::SmolgenBiasIndex(q, k)] = bias[bh * 4096 + q * 64 + k];
      db = reinterpret_cast<half_t*>(dev.Put(perm.data(), perm.size()));
    }
    auto* dout = static_cast<uint8_t*>(dev.Alloc((size_t)batch * 64 * d));
    lc0mi::LaunchAttentionF8Out(dq, db, dout, out_mul, batch, heads, scale, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(out, dout, (size_t)batch * 64 * d, hipMemcpyDeviceToHost));
  });
}

int lc0mi_k_smolgen_attention(const uint16_t* qkv, const uint16_t* gen, const uint16_t* w, int batch, int heads,
                              int gen_sz, float scale, int f8_out, float out_mul, void* out, int time_iters,
                              double* ms) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1 || !lc0mi::SmolgenAttentionSupported(heads, 32, gen_sz)) throw Error("bad smolgen attention shape");
    Dev dev;
    const int d = heads * 32;
    auto* dq = reinterpret_cast<half_t*>(dev.Put(qkv, (size_t)batch * 64 * 3 * d));
    auto* dg = reinterpret_cast<half_t*>(dev.Put(gen, (size_t)batch * heads * gen_sz));
    std::vector<uint16_t> frag((size_t)4096 * gen_sz);
    for (int row = 0; row < 4096; row++)
      for (int col = 0; col < gen_sz; col++)
        frag[lc0mi::SmolgenFragmentIndex(row, col, gen_sz)] = w[(size_t)row * gen_sz + col];
    auto* dw = reinterpret_cast<half_t*>(dev.Put(frag.data(), frag.size()));
    const size_t out_bytes = (size_t)batch * 64 * d * (f8_out ? 1 : 2);
    void* dout = dev.Alloc(out_bytes);
    auto launch = [&] {
      if (f8_out) {
        lc0mi::LaunchSmolgenAttentionF8Out(dq, dg, dw, static_cast<uint8_t*>(dout), out_mul, batch, heads, 32, gen_sz,
                                           scale, nullptr);
      } else {
        lc0mi::LaunchSmolgenAttention(dq, dg, dw, static_cast<half_t*>(dout), batch, heads, 32, gen_sz, scale, nullptr,
                                      g_bf16);
      }
    };
    launch();
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(out, dout, out_bytes, hipMemcpyDeviceToHost));
    if (time_iters > 0 && ms) *ms = TimeLaunches(time_iters, launch);
  });
}

int lc0mi_k_copy(long long bytes, int iters, double* ms) {
  return Guard([&] {
    RequireDevice();
    if (bytes < 16 || iters < 1) throw Error("bad copy size");
    Dev dev;
    void* src = dev.Alloc((size_t)bytes);
    void* dst = dev.Alloc((size_t)bytes);
    K_CHECK(hipMemset(src, 1, (size_t)bytes));
    double t = TimeLaunches(iters, [&] { lc0mi::LaunchCopy(src, dst, bytes / 16, nullptr); });
    if (ms) *ms = t;
  });
}

int lc0mi_k_expand_planes_nhwc(const uint64_t* masks, const float* values, int batch, float* out) {
  return Guard([&] {
    RequireDevice();
    if (batch < 1) throw Error("bad expand shape");
    Dev dev;
    uint64_t* dm = dev.Put(masks, (size_t)batch * 112);
    float* dv = dev.Put(values, (size_t)batch * 112);
    auto* dout = static_cast<float*>(dev.Alloc((size_t)batch * 64 * 112 * 4));
    lc0mi::LaunchExpandPlanesNhwc<float>(dm, dv, dout, batch, nullptr);
    K_CHECK(hipDeviceSynchronize());
    K_CHECK(hipGetLastError());
    K_CHECK(hipMemcpy(out, dout, (size_t)batch * 64 * 112 * 4, hipMemcpyDeviceToHost));
  });
}


// ---------------------------------------------------------------------------
// Split-K GEMM that allocates nothing. The float partial sums of the K slices,
// which lc0mi_k_gemm_splitk keeps in a buffer it allocates per call, live in a
// fixed array in device memory. In host code the array's name is only a handle
// for hipGetSymbolAddress: the address kernels and copies use is looked up once
// per device and kept in g_scratch_ptr.
// ---------------------------------------------------------------------------
}  // extern "C"

namespace {
constexpr long long kScratchFloats = 4ll << 20;  // 16 MiB on every device the library runs on
constexpr int kMaxDevices = 64;
static __device__ __align__(256) float scratch[kScratchFloats];
float* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// The device's own copy of the array, with that device current.
float* ScratchOfCurrentDevice() {
  int dev = -1;
  K_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) throw Error("device ordinal beyond the supported range");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    float* ptr = nullptr;
    K_CHECK(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
    if (!ptr) throw Error("hipGetSymbolAddress returned a null scratch address");
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

// C[m][n] = part[0][m][n] + part[1][m][n] + ... in slice order, starting from 0.0f
// like the host loop of lc0mi_k_gemm_splitk, so both give the same bits.
__global__ __launch_bounds__(256) void sum_slices_kernel(const float* __restrict__ part, long long slice_stride,
                                                         int slices, float* __restrict__ C, int M, int N, int ldc) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)M * N) return;
  const int m = (int)(i / N), n = (int)(i - (long long)m * N);
  const long long off = (long long)m * ldc + n;
  float s = 0.0f;
  for (int z = 0; z < slices; z++) s += part[z * slice_stride + off];
  C[off] = s;
}

void RequireDevicePointer(const void* p, const char* what) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess ||
      (attr.type != hipMemoryTypeDevice && attr.type != hipMemoryTypeManaged)) {
    (void)hipGetLastError();
    throw Error(std::string(what) + " is not a device pointer");
  }
}
}  // namespace

extern "C" {

int lc0mi_k_gemm_splitk_noalloc(const uint16_t* dA, int lda, const uint16_t* dW, int ldw, const float* dbias, int M,
                                int N, int K, int split_k, float scale, float* dC, int ldc, void* stream) {
  return Guard([&] {
    RequireDevice();
    if (K < 8 || K % 8 || lda % 8 || ldw % 8) throw Error("K, lda and ldw must be multiples of 8");
    if (M < 1 || N < 1 || split_k < 1 || lda < K || ldw < K || ldc < N) throw Error("bad gemm shape");
    const long long c_elems = (long long)M * ldc;
    if (c_elems * split_k > kScratchFloats)
      throw Error("split-K partial sums need " + std::to_string(c_elems * split_k) + " floats; the fixed scratch array holds " +
                  std::to_string(kScratchFloats));
    if (!dA || !dW || !dC) throw Error("null operand");
    RequireDevicePointer(dA, "A");
    RequireDevicePointer(dW, "W");
    RequireDevicePointer(dC, "C");
    if (dbias) RequireDevicePointer(dbias, "bias");
    if ((reinterpret_cast<uintptr_t>(dA) | reinterpret_cast<uintptr_t>(dW)) & 15) throw Error("A and W must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(dbias) & 15) throw Error("bias must be 16-byte aligned");   // read four floats at a time
    float* part = ScratchOfCurrentDevice();
    hipStream_t st = static_cast<hipStream_t>(stream);
    lc0mi::GemmArgs g;
    g.A = reinterpret_cast<const half_t*>(dA); g.lda = lda;
    g.W = reinterpret_cast<const half_t*>(dW); g.ldw = ldw;
    g.C = part; g.ldc = ldc;
    g.bias = dbias;
    g.M = M; g.N = N; g.K = K; g.scale = scale; g.act = 3; g.out_f32 = true;
    g.split_k = split_k; g.split_stride = c_elems;
    // Every (m < M, n < N) element of every slice is stored by the GEMM, so nothing of the previous call's
    // contents is read and the array needs no clearing.
    lc0mi::LaunchGemm(g, st);
    const long long total = (long long)M * N;
    hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, part, c_elems, split_k,
                       dC, M, N, ldc);
    K_CHECK(hipGetLastError());
  });
}

}  // extern "C"
