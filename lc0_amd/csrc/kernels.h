// Launchers of the gfx950 kernels. Host code sees only these plain functions;
// all of them enqueue work on the given stream and return without waiting.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdint>

namespace lc0mi {

using half_t = _Float16;
using bf16_t = __bf16;
// Element type of a network's activations and weights. The 16-bit launchers below take half_t pointers for either
// 16-bit type (same storage); a `bf16` argument or field says which arithmetic the bits mean.
enum class Dtype { kHalf, kBf16, kFloat };

// C[b][m][n] = act(scale * sum_k A[b][m][k] * W[b][n][k] + bias[n]),  b < batch.
// A and W are K-contiguous (row-major activations, lc0's [out][in] weights).
// Requirements: K % 8 == 0, lda % 8 == 0, ldw % 8 == 0, 16-byte aligned bases
// and batch strides; M, N arbitrary. bias may be null (then no bias; the
// activation is still applied). out_f32 selects float output.
// How a large GEMM writes its output (GemmArgs::out_stores, GemmF8Args::out_stores; only the 256-row tiles of the
// direct-to-LDS kernel know more than ordinary stores). kStoresAuto: ordinary stores, or streaming (non-temporal)
// ones for an output so large that it would push the operands out of L2. kStoresAutoKeep: the same size rule, but
// with stores written through at system scope in place of the streaming ones: they leave L2 alone as well, and the
// kernel that reads the output next finds it in the memory-side cache, which streamed data is not. For outputs
// whose reader is bound by memory (attention, layer norm) as long as a layer's activations fit that cache.
// The last three name a kind of store outright.
enum OutStores { kStoresAuto = 0, kStoresAutoKeep = 1, kStoresCached = 2, kStoresStream = 3, kStoresWriteThrough = 4 };

struct GemmArgs {
  const half_t* A = nullptr; int lda = 0; long long strideA = 0;
  const half_t* W = nullptr; int ldw = 0; long long strideW = 0;
  void* C = nullptr; int ldc = 0; long long strideC = 0;
  const float* bias = nullptr;
  int M = 0, N = 0, K = 0, batch = 1;
  float scale = 1.0f;
  int act = 3;  // Activation enum value (3 = none)
  bool out_f32 = false;
  // A, W and (unless out_f32) C hold bfloat16 instead of half values. Not with the folded layer-norm fields.
  bool bf16 = false;
  int out_stores = kStoresAuto;
  // split_k > 1: the K range is cut into split_k slices computed by different
  // workgroups; slice s stores its partial sums (float, out_f32 required, no
  // activation, bias only in slice 0) at C + s * split_stride. The consumer adds
  // the slices.
  int split_k = 1;
  long long split_stride = 0;
  // Choose the variant with the shortest latency even if it occupies more of the GPU (for a kernel on the
  // critical path; the default favours the variant that leaves room for a concurrent stream).
  bool latency_first = false;

  // Layer norm folded into the GEMMs on either side of it, so that neither the normalised rows nor the sum they
  // are computed from make a round trip of their own through memory. A "producer" GEMM adds the residual and
  // leaves the un-normalised sum u plus per-row partial sums; a "consumer" GEMM multiplies u by weights that
  // already carry gamma and corrects for mean and deviation per output row:
  //   LN(u)[m] . w[n] = rstd[m] * (sum_k u[m][k] gamma[k] w[n][k] - mean[m] * c[n]) + sum_k beta[k] w[n][k]
  // with c[n] = sum_k gamma[k] w[n][k]; the caller passes W = w * gamma, col_c = c and the beta term in bias.
  // Row statistics travel as partial sums: stats[m][part][2] = (sum, sum of squares) over one column tile of u.
  //
  // Consumer (row_stats != nullptr):  C[m][n] = act(rstd[m] * (scale * acc - mean[m] * col_c[n]) + bias[n]),
  //   mean and rstd of row m from the row_parts partial sums over norm_n columns.
  const float* row_stats = nullptr;
  int row_parts = 0;
  const float* col_c = nullptr;
  // Producer (skip != nullptr, no activation, half output):  C[m][n] = scale * acc + bias[n] + s[m][n], where
  //   s = skip (skip_stats == nullptr) or the layer norm of skip's row with skip_gamma / skip_beta and statistics
  //   from skip_stats (skip_parts partial sums per row over norm_n columns). skip may alias C.
  //   stats_out (optional) receives the partial sums of the rows of C as stored (rounded to half):
  //   stats_out[m][tile][2], one part per column tile of the kernel variant (GemmStatsParts()).
  const half_t* skip = nullptr;
  int ldskip = 0;
  const float* skip_stats = nullptr;
  int skip_parts = 0;
  const float* skip_gamma = nullptr;
  const float* skip_beta = nullptr;
  float* stats_out = nullptr;
  int norm_n = 0;        // length of the normalised rows (consumer: K of the real problem; producer: N)
  float norm_eps = 0.0f;
};
void LaunchGemm(const GemmArgs& args, hipStream_t stream);
// Whether LaunchGemm serves the folded layer-norm fields of these arguments (the kernel variant it picks has the
// epilogue), and the number of partial sums per row a producer launch writes to stats_out.
bool GemmSupportsNormFolding(const GemmArgs& args);
int GemmStatsParts(const GemmArgs& args);
// Name of the kernel variant LaunchGemm picks for these arguments (tile shape; "...+rest" when it cuts the product
// along its rows into whole rounds of large tiles and a rest, GemmRowSplit() rows in the first launch).
const char* GemmVariantName(const GemmArgs& args);
int GemmRowSplit(const GemmArgs& args);

// e4m3 (OCP fp8, "fn": max 448, no infinities) GEMM with fp32 accumulation:
//   C[m][n] = act(col_scale[n] * sum_k A[m][k] * W[n][k] + bias[n])
// A, W hold e4m3 bytes, K-contiguous; col_scale[n] = (activation scale) x (scale of weight row n).
// out_f8: C receives e4m3 bytes of C * out_mul (saturating, round to nearest even), else half.
// Requirements: K % 128 == 0, lda % 16 == 0, ldw % 16 == 0, 16-byte aligned bases.
struct GemmF8Args {
  const uint8_t* A = nullptr; int lda = 0;
  const uint8_t* W = nullptr; int ldw = 0;
  void* C = nullptr; int ldc = 0;
  const float* col_scale = nullptr;
  const float* bias = nullptr;
  int M = 0, N = 0, K = 0;
  int act = 3;
  bool out_f8 = false;
  float out_mul = 1.0f;
  int out_stores = kStoresAuto;
};
void LaunchGemmF8(const GemmF8Args& args, hipStream_t stream);
const char* GemmF8VariantName(const GemmF8Args& args);

// *out = max(*out, max_i |x[i]|) (n % 8 == 0; *out must hold a non-negative float).
void LaunchAbsMax(const half_t* x, long long n, float* out, hipStream_t stream);
// y[i] = e4m3(x[i] * mul), saturating; n % 8 == 0.
void LaunchQuantizeF8(const half_t* x, uint8_t* y, long long n, float mul, hipStream_t stream);

// Same contract in float: C = act(scale * A.W^T + bias) with float A, W, C.
// K % 4 == 0, lda % 4 == 0, ldw % 4 == 0.
struct GemmArgsF32 {
  const float* A = nullptr; int lda = 0; long long strideA = 0;
  const float* W = nullptr; int ldw = 0; long long strideW = 0;
  float* C = nullptr; int ldc = 0; long long strideC = 0;
  const float* bias = nullptr;
  int M = 0, N = 0, K = 0, batch = 1;
  float scale = 1.0f;
  int act = 3;
};
void LaunchGemmF32(const GemmArgsF32& args, hipStream_t stream);

// Input planes -> token-major embedding input with the 64 position-encoding
// channels appended: out[b*64+sq][c], c < 112 plane bits * value, 112..175 the
// pos-enc row of sq, then zero padding up to ld. T = half_t or float.
template <typename T>
void LaunchExpandPlanesAttn(const uint64_t* masks, const float* values, const T* pos_enc /*[64][64]*/,
                            T* out, int ld, int batch, hipStream_t stream);
// Same with per-sample extra channels (the dense position encoding): out[b*64+sq][112 + c] =
// extra[b][sq][c], c < n_extra. T = half_t, bf16_t or float (also for the two launchers below and the one above).
template <typename T>
void LaunchExpandPlanesDense(const uint64_t* masks, const float* values, const T* extra, int n_extra, T* out, int ld,
                             int batch, hipStream_t stream);
// First 12 input planes, square-major: out[b][sq * 12 + j] (input of the dense position-encoding layer).
template <typename T>
void LaunchPiecePlanes(const uint64_t* masks, const float* values, T* out, int batch, hipStream_t stream);
// Input gating: x[b][i] = x[b][i] * mult[i] + add[i], i < per_sample (= 64 * channels, square-major).
template <typename T>
void LaunchInputGating(T* x, const float* mult, const float* add, int batch, int per_sample, hipStream_t stream);
// Input planes -> NCHW dense planes out[b][c][sq] (T = half_t or float).
template <typename T>
void LaunchExpandPlanesNchw(const uint64_t* masks, const float* values, T* out, int batch, hipStream_t stream);

// dst[i] = src[i] for n 16-byte vectors (traffic calibration kernel).
void LaunchCopy(const void* src, void* dst, long long n_vec16, hipStream_t stream);
// Sets n floats to zero (a kernel, so that it can be captured into a graph).
void LaunchZero(float* p, long long n, hipStream_t stream);
// Forces LaunchGemm to use one kernel variant (-1 = automatic choice): 0 256x256x64,
// 1 256x192x64, 2 256x128x32 (direct-to-LDS, need K % 64 == 0 and half output),
// 3 128x128x64, 4 64x64x64 (register-staged), 5 128x128x64 direct-to-LDS with 4 waves,
// 6 row-panel 64x32 (K split over the waves), 7 128x64x64 direct-to-LDS with 4 waves. For tests and tuning only.
void SetGemmVariantOverride(int variant);
// Whether LaunchGemm may cut a large product along its rows (GemmRowSplit); on by default.
void SetGemmRowSplit(bool on);

// Layer norm for few, long rows (one workgroup per row): t = act(x) * alpha + skip,
// where x is half (x_f16) or the sum of n_partials float arrays x_f32 + i * partial_stride
// (split-K partial sums); exactly one of x_f32 / x_f16 is non-null. pre_act is an
// Activation enum value applied before the norm. C % 8 == 0, C <= 8192.
// y_f8 (optional): also receives e4m3(y * f8_mul), saturating, taken from the float values.
void LaunchLayerNormRows(const float* x_f32, int n_partials, long long partial_stride, const half_t* x_f16,
                         int pre_act, const half_t* skip, half_t* y, const float* gamma, const float* beta, int rows,
                         int C, float alpha, float eps, hipStream_t stream, bool bf16 = false,
                         uint8_t* y_f8 = nullptr, float f8_mul = 1.0f);

// rows x C layer norm: y = beta + gamma * (t - mean) / sqrt(var + eps) with
// t = x * alpha + skip (skip may be null). x, skip, y may alias. C % 8 == 0, C <= 8192.
// y_f8 (optional): also receives e4m3(y * f8_mul), saturating, the operand of a following fp8 GEMM.
// through: for tensors far larger than L2 inside a pass whose activations fit the memory-side cache: x (not read
// again) comes in with non-temporal loads, y goes out with stores written through at system scope, where the
// kernels that read it next find it (GemmArgs::out_stores has the measurements).
void LaunchLayerNorm(const half_t* x, const half_t* skip, half_t* y, const float* gamma, const float* beta,
                     int rows, int C, float alpha, float eps, hipStream_t stream, uint8_t* y_f8 = nullptr,
                     float f8_mul = 1.0f, bool bf16 = false, bool through = false);
// The same for any element type (half_t, bf16_t, float) and any row length, with an activation applied to x first:
// y = norm(act(x) * alpha + skip). One workgroup per row, scalar accesses.
template <typename T>
void LaunchLayerNormGeneric(const T* x, const T* skip, T* y, const float* gamma, const float* beta, int rows, int C,
                            float alpha, float eps, int pre_act, hipStream_t stream);

// Fused multi-head attention over 64 tokens, head depth 32, 64 or 128 (d_model = heads * depth).
// qkv: [B*64][3*d_model] (q | k | v column blocks), bias: smolgen logits in the
// tile-native layout produced by SmolgenBiasIndex (may be null), out: [B*64][d_model].
void LaunchAttention(const half_t* qkv, const half_t* bias, half_t* out, int batch, int heads,
                     float scale, hipStream_t stream, int depth = 32, bool bf16 = false);
bool AttentionDepthSupported(int depth);
// The same contract (bias in the SmolgenBiasIndex layout, may be null) for any element type and any head depth up to
// 128, on the vector ALUs: the float configuration, and head depths the kernel above does not take.
template <typename T>
void LaunchAttentionGeneric(const T* qkv, const T* bias, T* out, int batch, int heads, int depth, float scale,
                            hipStream_t stream);
bool AttentionGenericDepthSupported(int depth);
// Same with e4m3 output: out[...] = e4m3(result * out_mul), saturating.
void LaunchAttentionF8Out(const half_t* qkv, const half_t* bias, uint8_t* out, float out_mul, int batch, int heads,
                          float scale, hipStream_t stream, int depth = 32);
// Position inside one head's 4096-entry bias block of logit (query q, key k).
__host__ __device__ int SmolgenBiasIndex(int q, int k);

// Smolgen generator layer and attention in one kernel (smolgen_attention.hip): the logits
//   sum_j W[q*64+k][j] * gen[b][h][j]   (W: the shared smolgen_w layer [4096][gen_sz], gen: [B][heads][gen_sz])
// are computed per workgroup and added to scale * Q.K^T without passing through memory. wfrag is W converted to
// halves and reordered with SmolgenFragmentIndex (element (row, col) of W at that position). Head depth 32, at most
// 32 heads, gen_sz 32, 128 or 256 (SmolgenAttentionSupported); qkv and out as for LaunchAttention.
bool SmolgenAttentionSupported(int heads, int depth, int gen_sz);
long long SmolgenFragmentIndex(int row, int col, int gen_sz);
void LaunchSmolgenAttention(const half_t* qkv, const half_t* gen, const half_t* wfrag, half_t* out, int batch,
                            int heads, int depth, int gen_sz, float scale, hipStream_t stream, bool bf16 = false);
void LaunchSmolgenAttentionF8Out(const half_t* qkv, const half_t* gen, const half_t* wfrag, uint8_t* out,
                                 float out_mul, int batch, int heads, int depth, int gen_sz, float scale,
                                 hipStream_t stream);

// Attention policy tail: promotion offsets + gather to 1858 moves.
// logits: [B][64*64] float (already scaled), kq: [B*64][ld_kq] with keys at column
// offset key_off, ppo: [4][pd] float, inv_map: [1858] source index into the
// 4096+192 virtual buffer. out: [B][1858] float.
template <typename T>   // T: element type of kq (half_t, bf16_t, float)
void LaunchAttnPolicyGather(const float* logits, const T* kq, int ld_kq, int key_off, const float* ppo,
                            int pd, const int16_t* inv_map, float* out, int batch, hipStream_t stream);

// Most legal moves one sample may list for LaunchLegalSoftmax (chess positions have at most 218).
constexpr int kMaxLegalMoves = 256;
// Softmax over the listed moves of every sample with lc0's polynomial exponential
// (src/neural/wrapper.cc:135-156, src/utils/fastmath.h:59-86):
//   probs[offsets[b] + i] = FastExp((policy[b][ids[offsets[b] + i]] - max_b) * inv_temperature) / total_b
// policy: [B][1858]; offsets: [B + 1], non-decreasing, at most kMaxLegalMoves apart; ids < 1858.
void LaunchLegalSoftmax(const float* policy, const int* offsets, const uint16_t* ids, float inv_temperature,
                        float* probs, int batch, hipStream_t stream);

}  // namespace lc0mi

// ---------------------------------------------------------------------------
// SE-ResNet tower: winograd F(4x4,3x3) convolution on the 8x8 board.
// Activations are NHWC: x[b][sq][c]. T = half_t or float.
// ---------------------------------------------------------------------------
namespace lc0mi {

// Input planes -> out[b][sq][c], c < 112 (T = half_t or float).
template <typename T>
void LaunchExpandPlanesNhwc(const uint64_t* masks, const float* values, T* out, int batch, hipStream_t stream);

// Host side: filter [cout][cin][3][3] -> U[36][cout][ld_cin] = (G g G^T), with the
// row-scaled G = diag(4,6,6,24,24,1) * G_lavin (integer entries); ld_cin >= cin is the
// zero-padded row length.
void WinogradFilterTransform4x4(const float* filter, int cout, int cin, int ld_cin, float* u);

// V[k][b*4+t][c] = (B^T d B)[k] of the 6x6 input patch of tile t (2x2 tiles of 4x4
// outputs, zero padding), with B^T row-scaled by 1/diag(4,6,6,24,24,1).
// x: [B][64][C], v: [36][B*4][ldv]; columns C..ldv-1 are written as zeros.
template <typename T>
void LaunchWinogradInputTransform(const T* x, T* v, int batch, int C, int ldv, hipStream_t stream);

// Output transform y = A^T m A per tile with the fused tail of a residual block:
//   plain:  out = act(y + bias (+ skip))
//   SE:     pool = mean64(y) + bias; h = act(W1 pool + b1); s = W2 h + b2;
//           gamma = sigmoid(s[0:C]); beta = s[C:2C] + gamma * bias;
//           out = act(gamma * y + skip + beta)
// m: [36][B*4][C] (M_IS_F32 selects float m for T = half_t), out/skip: [B][64][C].
// se_w1: [K][C], se_w2: [K][2C] floats (the transpose of lc0's [2C][K]). C <= 1024, K <= 256.
// v_next (optional, only when WinogradFusedInputTransform(C, sizeof(T), se_k)): the input transform of the next
// convolution is applied to the result in the same kernel and written to v_next[36][B*4][ldv_next];
// out may then be null if nobody else reads the activations.
template <typename T, typename MT>
void LaunchWinogradOutputTransform(const MT* m, const float* bias, const T* skip, const float* se_w1,
                                   const float* se_b1, const float* se_w2, const float* se_b2, int se_k, T* out,
                                   int batch, int C, int act, hipStream_t stream, T* v_next = nullptr,
                                   int ldv_next = 0);
bool WinogradFusedInputTransform(int C, int elem_size, int se_k);

// Gather of the convolutional policy head: out[b][j] = t[b][sq][plane] for
// kConvPolicyMap[plane*64+sq] = j. t: [B][64][ld] (NHWC), inv_map: [1858] holding plane*64+sq.
template <typename T>
void LaunchConvPolicyGather(const T* t, int ld, const int16_t* inv_map, float* out, int batch, hipStream_t stream);

}  // namespace lc0mi
