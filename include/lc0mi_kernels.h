/*
 * Single-kernel entry points of liblc0mi.so, for parity tests and kernel
 * micro-benchmarks. All pointers are HOST pointers; each call stages its
 * operands into HBM, launches exactly one kernel of the forward pass and
 * copies the result back. Halves are passed as raw IEEE binary16 bits.
 * Return value: 0 on success, else lc0mi_last_error() has the message.
 */
#ifndef LC0MI_KERNELS_H_
#define LC0MI_KERNELS_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* C[b][m][n] = act(scale * A[b][m][:] . W[b][n][:] + bias[n]); the kernel behind
 * FullyConnectedLayer::Forward1D (src/neural/backends/blas/fully_connected_layer.cc:49-106).
 * strides in elements between batch entries; out_f32 selects float output.
 * If time_iters > 0, *ms receives the mean HIP-event time of that many extra launches. */
int lc0mi_k_gemm(const uint16_t* A, int lda, long long strideA, const uint16_t* W, int ldw, long long strideW,
                 const float* bias, int M, int N, int K, int batch, float scale, int act, int out_f32, void* C,
                 int ldc, long long strideC, int time_iters, double* ms);
/* Name of the tile shape lc0mi_k_gemm runs a half-precision product of this shape on ("gemm_dma_256x256x64", ...):
 * the launcher's host-side choice, which needs no device. No counterpart in the reference, whose products go to a
 * BLAS library (src/neural/backends/blas/fully_connected_layer.cc:90-101). */
const char* lc0mi_k_gemm_variant_name(int M, int N, int K, int batch, int latency_first);
/* Rows that lc0mi_k_gemm gives to a first launch of whole rounds of large tiles when it cuts a half-precision product
 * of this shape along its rows (0: one launch). Host-side choice, no device needed; no counterpart in the reference. */
int lc0mi_k_gemm_row_split(int M, int N, int K);
/* Switches that cut off (0) or on (1, the default), for measurements and tests; process-wide, like lc0mi_k_set_gemm_variant. */
void lc0mi_k_set_gemm_row_split(int on);
/* Split-K form: K is cut into split_k slices whose float partial sums are added in
 * slice order (bias added once, no activation). C is float [M][N]. */
int lc0mi_k_gemm_splitk(const uint16_t* A, int lda, const uint16_t* W, int ldw, const float* bias, int M, int N,
                        int K, int split_k, float scale, float* C, int ldc);
/* The two GEMMs around a layer norm with the norm folded into them, so that neither the normalised rows nor the
 * sum they are computed from travel through memory on their own (LayerNorm2DWithSkipConnection between the dense
 * layers of an encoder block, src/neural/backends/blas/network_blas.cc:441-470 with encoder.h:29-66).
 * Producer: U[m][n] = scale * A[m][:] . W[n][:] + bias[n] + s[m][n] as halves, where s = skip, or, when skip_stats
 * is given, the layer norm of skip's rows with skip_gamma / skip_beta and the statistics in skip_stats
 * ([M][skip_parts][2] partial (sum, sum of squares) per row). skip is [M][N]. stats_out receives [M][*parts_out][2]
 * partial sums of the stored U per column tile (at most stats_cap floats). */
int lc0mi_k_gemm_norm_producer(const uint16_t* A, int lda, const uint16_t* W, int ldw, const float* bias, int M, int N,
                               int K, float scale, const uint16_t* skip, const float* skip_stats, int skip_parts,
                               const float* skip_gamma, const float* skip_beta, float eps, uint16_t* U,
                               float* stats_out, int stats_cap, int* parts_out, int time_iters, double* ms);
/* Consumer: C[m][n] = act(rstd[m] * (U[m][:] . W[n][:] - mean[m] * col_c[n]) + bias[n]), mean and rstd of row m of
 * U (K columns) from stats [M][parts][2]. With W = w * gamma, col_c[n] = sum_k W[n][k] and bias[n] = b[n] +
 * sum_k beta[k] w[n][k] this equals act(LN(U) . w^T + b). */
int lc0mi_k_gemm_norm_consumer(const uint16_t* U, int ldu, const uint16_t* W, int ldw, const float* col_c,
                               const float* bias, int M, int N, int K, const float* stats, int parts, float eps,
                               int act, int latency_first, uint16_t* C, int ldc, int time_iters, double* ms);
/* Forces the GEMM tile variant of subsequent calls (-1 automatic; 0 256x256x64,
 * 1 256x192x64, 2 256x128x32 direct-to-LDS kernels, 3 128x128x64, 4 64x64x64, 5 direct-to-LDS 128x128x64,
 * 6 row panels of 16x16 to 64x32 outputs, 7 direct-to-LDS 128x64x64, 8 unused (automatic choice), 9 direct-to-LDS
 * 128x32x64, 10 direct-to-LDS 64x64x64). */
int lc0mi_k_set_gemm_variant(int variant);
/* Test hook, process-wide: from now on the 16-bit buffers of lc0mi_k_gemm, lc0mi_k_layer_norm, lc0mi_k_layer_norm_rows,
 * lc0mi_k_attention and lc0mi_k_smolgen_attention (half output) hold bfloat16 values and the kernels run their bf16
 * instances (precision=bf16 of the network; the reference's type: src/utils/bf16_utils.h). 0 switches back to half. */
int lc0mi_k_set_bf16(int on);
/* Test hook, process-wide: the kind of output stores of lc0mi_k_gemm and lc0mi_k_gemm_f8 (256-row tiles of the
 * direct-to-LDS kernel; others always store ordinarily) and of lc0mi_k_layer_norm: 0 by output size (ordinary or
 * streaming), 1 by output size (ordinary or written through), 2 ordinary, 3 streaming (non-temporal), 4 written
 * through at system scope (the layer norm then also reads x with non-temporal loads). The network picks 1 and the
 * written-through layer norm for the big tensors of an encoder layer while a layer's activations fit the memory-side
 * cache. No counterpart in the reference. */
int lc0mi_k_set_out_stores(int kind);
/* Profiling hook, process-wide: with mib > 0 every timed launch (time_iters of the entry points here) is preceded by
 * an untimed copy of mib MiB, so that the kernel finds its operands in memory rather than in L2 or the memory-side
 * cache, as it does between other kernels inside a forward pass; the timed launches are then timed one by one.
 * 0 switches back to back-to-back launches. No counterpart in the reference. */
int lc0mi_k_set_cold_cache(int mib);
/* The general attention and layer norm kernels (any element type, head depth up to 128, any row length): dtype 0 half,
 * 1 bfloat16, 2 float for qkv / bias / out and x / skip / y. Same contracts as lc0mi_k_attention (bias [b][h][q][k])
 * and lc0mi_k_layer_norm, with an activation (lc0's numbering) applied to x first. Counterparts in the reference:
 * src/neural/backends/blas/network_blas.cc:352-439, src/neural/backends/blas/encoder.h:29-66. */
int lc0mi_k_attention_generic(int dtype, const void* qkv, const void* bias, int batch, int heads, int depth, float scale,
                              void* out);
int lc0mi_k_layer_norm_generic(int dtype, const void* x, const void* skip, const float* gamma, const float* beta, int rows,
                               int C, float alpha, float eps, int pre_act, void* y);
/* float variant (fp32 configuration). */
int lc0mi_k_gemm_f32(const float* A, int lda, const float* W, int ldw, const float* bias, int M, int N, int K,
                     float scale, int act, float* C, int ldc);
/* y = LN(x * alpha + skip) * gamma + beta, rows of C halves; skip may be NULL.
 * (LayerNorm2DWithSkipConnection, src/neural/backends/blas/encoder.h:29-66) */
int lc0mi_k_layer_norm(const uint16_t* x, const uint16_t* skip, const float* gamma, const float* beta, int rows,
                       int C, float alpha, float eps, uint16_t* y, int time_iters, double* ms);
/* One-workgroup-per-row layer norm with an activation applied first:
 * y = LN(act(x) * alpha + skip); x is float (x_f32) or half (x_f16), one of them NULL. */
int lc0mi_k_layer_norm_rows(const float* x_f32, const uint16_t* x_f16, int pre_act, const uint16_t* skip,
                            const float* gamma, const float* beta, int rows, int C, float alpha, float eps,
                            uint16_t* y);
/* Fused attention, head depth 32, 64 or 128: qkv [B*64][3*heads*depth] halves, bias [B][heads][64 q][64 k]
 * halves in natural order (may be NULL), out [B*64][heads*depth]
 * (src/neural/backends/blas/network_blas.cc:352-439). */
int lc0mi_k_attention(const uint16_t* qkv, const uint16_t* bias, int batch, int heads, int depth, float scale,
                      uint16_t* out, int time_iters, double* ms);
/* Input planes -> [B*64][ld] halves with position encoding appended
 * (src/neural/backends/blas/network_blas.cc:973-981, 630-652). */
int lc0mi_k_expand_planes_attn(const uint64_t* masks, const float* values, int batch, int ld, uint16_t* out,
                               int time_iters, double* ms);
/* Input planes -> [B][112][64] floats (EncodePlanes, network_blas.cc:973-981). */
int lc0mi_k_expand_planes_nchw(const uint64_t* masks, const float* values, int batch, float* out);
/* Attention-policy tail: logits [B][4096] floats, keys [B*64][pd] halves,
 * ppo [4][pd] floats -> policy [B][1858] (network_blas.cc:873-914). */
int lc0mi_k_attn_policy_gather(const float* logits, const uint16_t* keys, const float* ppo, int pd, int batch,
                               float* out);

/* Softmax over listed moves with lc0's FastExp (NetworkAsBackendComputation::SoftmaxPolicy,
 * src/neural/wrapper.cc:135-156; src/utils/fastmath.h:59-86): policy [batch][1858]; sample b lists
 * ids[offsets[b] .. offsets[b + 1]) (at most 256); probs is laid out like ids. */
int lc0mi_k_legal_softmax(const float* policy, const int* offsets, const uint16_t* ids, float inv_temperature,
                          int batch, float* probs);

/* One 3x3 convolution of the residual tower through the winograd F(4x4,3x3) path
 * (input transform, 36 batched GEMMs, output transform with the fused tail):
 *   out = act(conv(x) + bias (+ skip))                      when se_k == 0
 *   out = ApplySEUnit(conv(x), bias, skip, w1,b1,w2,b2)     when se_k > 0
 * (WinogradConvolution3::Forward + BiasActivate / BiasResidual / ApplySEUnit,
 *  src/neural/backends/blas/winograd_convolution3.cc:47-324, se_unit.cc:31-91).
 * x, skip, out: [B][64][C] floats (NHWC); filter: [cout][cin][3][3]; use_fp16 selects
 * the half-precision kernels (operands rounded to fp16 on the way in).
 * v_fused / v_separate (both or neither, [36][B*4][cout]): the transformed input of a following
 * convolution, from the output transform kernel that fuses it and from the stand-alone input
 * transform applied to `out`. */
int lc0mi_k_winograd_conv(const float* x, const float* filter, const float* bias, const float* skip,
                          const float* se_w1, const float* se_b1, const float* se_w2, const float* se_b2, int se_k,
                          int batch, int cin, int cout, int act, int use_fp16, float* out, float* v_fused,
                          float* v_separate);
/* e4m3 GEMM: C = act(col_scale[n] * A.W^T + bias[n]); A [M][lda], W [N][ldw] e4m3 bytes, K % 128 == 0.
 * out_f8 != 0: C receives e4m3(C * out_mul) bytes, else halves. Counterpart of FullyConnectedLayer::Forward1D
 * (src/neural/backends/blas/fully_connected_layer.cc:66-106) on quantised operands. */
int lc0mi_k_gemm_f8(const uint8_t* A, int lda, const uint8_t* W, int ldw, const float* col_scale, const float* bias,
                    int M, int N, int K, int act, int out_f8, float out_mul, void* C, int ldc, int time_iters,
                    double* ms);
/* y[i] = e4m3(x[i] * mul): round to nearest even, saturating at +-448 (FP32toFP8E4M3FN,
 * src/utils/fp8_utils.h:111-138, applied to half inputs). n % 8 == 0. */
int lc0mi_k_quantize_f8(const uint16_t* x, long long n, float mul, uint8_t* y);
/* lc0mi_k_layer_norm with a second, e4m3 output y_f8 = e4m3(y * f8_mul). */
int lc0mi_k_layer_norm_f8(const uint16_t* x, const uint16_t* skip, const float* gamma, const float* beta, int rows,
                          int C, float alpha, float eps, float f8_mul, uint16_t* y, uint8_t* y_f8);
/* The shared smolgen generator layer and the attention in one kernel (network_blas.cc:332-347 followed by :352-439):
 * logits[b][h][q][k] = scale * Q.K^T + sum_j w[q*64+k][j] * gen[b][h][j], out = softmax_k(logits) . V.
 * qkv [B*64][3*heads*32] halves, gen [B][heads][gen_sz] halves, w [4096][gen_sz] halves (row q*64+k); head depth 32,
 * heads <= 32, gen_sz 32, 128 or 256. out [B*64][heads*32]: halves, or e4m3(out * out_mul) bytes when f8_out. */
int lc0mi_k_smolgen_attention(const uint16_t* qkv, const uint16_t* gen, const uint16_t* w, int batch, int heads,
                              int gen_sz, float scale, int f8_out, float out_mul, void* out, int time_iters,
                              double* ms);
/* lc0mi_k_attention with e4m3 output e4m3(out * out_mul). */
int lc0mi_k_attention_f8(const uint16_t* qkv, const uint16_t* bias, int batch, int heads, float scale, float out_mul,
                         uint8_t* out);
/* Plain device-to-device copy of `bytes` bytes (16-byte vectors), launched `iters`
 * times: the known-traffic kernel used to calibrate HBM byte counters. *ms receives
 * the mean HIP-event time per launch. */
int lc0mi_k_copy(long long bytes, int iters, double* ms);
/* Input planes -> [B][64][112] floats (NHWC form of EncodePlanes). */
int lc0mi_k_expand_planes_nhwc(const uint64_t* masks, const float* values, int batch, float* out);

/* lc0mi_k_gemm_splitk for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. dA, dW, dbias (may be
 * NULL) and dC are DEVICE pointers (device or managed memory; dA, dW and dbias 16-byte aligned); the work is enqueued on `stream` (a hipStream_t, NULL =
 * the default stream) and the call returns without waiting. The partial sums of the K slices go to a fixed 16 MiB
 * array inside the library (one per GPU, held until the process ends): M * ldc * split_k may be at most 4194304
 * floats, larger requests fail with an error. The call uses no hipMalloc / hipFree. All calls on one GPU share that
 * array, so two calls that overlap in time on one GPU (different streams or threads) race; calls on one stream do
 * not. The first call on a device looks up the array's address and should be made outside graph capture. The kernel
 * variant is the automatic choice unless lc0mi_k_set_gemm_variant, a process-wide test hook, has forced another:
 * do not change that setting while calls are in flight. */
int lc0mi_k_gemm_splitk_noalloc(const uint16_t* dA, int lda, const uint16_t* dW, int ldw, const float* dbias, int M,
                                int N, int K, int split_k, float scale, float* dC, int ldc, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LC0MI_KERNELS_H_ */
