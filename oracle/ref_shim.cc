// TEST INFRASTRUCTURE.  extern "C" callers for the self-contained translation
// units of the reference (compiled where they lie under /root/reference by
// `make -C oracle ref` into oracle/_ref/libref_pieces.so).  Used only to
// validate the numpy/C restatement in oracle/; never shipped, never built on
// a machine that has no reference tree.
#include <cstdint>
#include <cstring>
#include <vector>

#include "neural/backends/blas/encoder.h"
#include "neural/backends/shared/activation.h"
#include "neural/backends/shared/winograd_filter.h"
#include "neural/tables/attention_policy_map.h"
#include "neural/tables/policy_map.h"
#include "utils/bf16_utils.h"
#include "utils/bititer.h"
#include "utils/fastmath.h"
#include "utils/fp16_utils.h"
#include "utils/fp8_utils.h"

using namespace lczero;

extern "C" {

float ref_activate(float v, int act) { return Activate(v, static_cast<ActivationFunction>(act)); }
void ref_softmax(size_t n, const float* in, float* out) { SoftmaxActivation(n, in, out); }
void ref_bias_activate(size_t batch, size_t channels, float* data, const float* biases, int act) {
  BiasActivate(batch, channels, data, biases, static_cast<ActivationFunction>(act));
}
void ref_bias_residual(size_t batch, size_t channels, float* data, const float* biases,
                       const float* eltwise, int act) {
  BiasResidual(batch, channels, data, biases, eltwise, static_cast<ActivationFunction>(act));
}
void ref_activate_vec(size_t len, const float* data, const float* bias, float* out, int act) {
  Activate(len, data, bias, out, static_cast<ActivationFunction>(act));
}
void ref_activate_se(size_t len, float gamma, const float* data, const float* bias, float beta,
                     float* out, int act) {
  Activate(len, gamma, data, bias, beta, out, static_cast<ActivationFunction>(act));
}
void ref_layernorm_skip(size_t batch, size_t channels, float* data, float alpha, const float* skip,
                        const float* gammas, const float* betas, float eps) {
  LayerNorm2DWithSkipConnection(batch, channels, data, alpha, skip, gammas, betas, eps);
}
void ref_winograd_filter_transform(const float* f, size_t outputs, size_t channels, float* out) {
  std::vector<float> in(f, f + outputs * channels * 9);
  std::vector<float> u = WinogradFilterTransformF(in, outputs, channels);
  std::memcpy(out, u.data(), u.size() * sizeof(float));
}
uint16_t ref_fp32_to_fp16(float f) { return FP32toFP16(f); }
float ref_fp16_to_fp32(uint16_t h) { return FP16toFP32(h); }
uint16_t ref_fp32_to_bf16(float f) { return FP32toBF16(f); }
float ref_bf16_to_fp32(uint16_t h) { return BF16toFP32(h); }
uint8_t ref_fp32_to_fp8e4m3(float f) { return FP32toFP8E4M3FN(f); }
float ref_fp8e4m3_to_fp32(uint8_t b) { return FP8E4M3FNtoFP32(b); }
float ref_fast_exp(float a) { return FastExp(a); }
uint64_t ref_reverse_bits_in_bytes(uint64_t v) { return ReverseBitsInBytes(v); }
uint64_t ref_reverse_bytes_in_bytes(uint64_t v) { return ReverseBytesInBytes(v); }
uint64_t ref_transpose_bits_in_bytes(uint64_t v) { return TransposeBitsInBytes(v); }
const short* ref_attn_policy_map() { return kAttnPolicyMap; }
int ref_attn_policy_map_size() { return sizeof(kAttnPolicyMap) / sizeof(short); }
const short* ref_conv_policy_map() { return kConvPolicyMap; }
int ref_conv_policy_map_size() { return sizeof(kConvPolicyMap) / sizeof(short); }
const float* ref_pos_encoding() { return &kPosEncoding[0][0]; }
}
