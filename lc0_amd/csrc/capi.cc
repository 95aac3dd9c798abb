// extern "C" boundary of the backend: translates lc0mi::Error into return
// codes plus a thread-local message and owns the opaque handles.
#include "../../include/lc0mi.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <limits>
#include <memory>
#include <string>

#include "network.h"
#include "tables.h"
#include "weights.h"

struct lc0mi_net {
  std::unique_ptr<lc0mi::Network> impl;
};
struct lc0mi_comp {
  std::unique_ptr<lc0mi::NetworkComputation> impl;
};

namespace {
thread_local std::string g_last_error;
}  // namespace

namespace lc0mi {
void SetLastError(const std::string& msg) { g_last_error = msg; }
}  // namespace lc0mi

namespace {

template <typename F>
int Guard(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_last_error = e.what();
    return 1;
  } catch (...) {
    g_last_error = "unknown error";
    return 1;
  }
}

int CreateNet(lc0mi::WeightsFile&& file, const char* opts_kv, lc0mi_net** out) {
  lc0mi::Options options(opts_kv ? opts_kv : "");
  auto net = std::make_unique<lc0mi_net>();
  net->impl = lc0mi::MakeMi355xNetwork(file, options);
  *out = net.release();
  return 0;
}
}  // namespace

extern "C" {

int lc0mi_net_create_from_buffer(const void* data, size_t len, const char* opts_kv, lc0mi_net** out) {
  return Guard([&] {
    if (!data || !out) throw lc0mi::Error("null argument");
    std::string raw = lc0mi::MaybeGunzip(data, len);
    CreateNet(lc0mi::ParseWeightsProto(raw.data(), raw.size()), opts_kv, out);
  });
}

int lc0mi_net_create_from_file(const char* path, const char* opts_kv, lc0mi_net** out) {
  return Guard([&] {
    if (!path || !out) throw lc0mi::Error("null argument");
    CreateNet(lc0mi::LoadWeightsFromFile(path), opts_kv, out);
  });
}

void lc0mi_net_destroy(lc0mi_net* net) { delete net; }

int lc0mi_net_caps(const lc0mi_net* net, int* input_format, int* output_format, int* moves_left_format) {
  return Guard([&] {
    if (!net) throw lc0mi::Error("null network");
    const auto& c = net->impl->GetCapabilities();
    if (input_format) *input_format = c.input_format;
    if (output_format) *output_format = c.output_format;
    if (moves_left_format) *moves_left_format = c.moves_left;
  });
}

int lc0mi_net_hints(const lc0mi_net* net, int* minibatch, int* batch_step, int* max_batch, int* threads,
                    int* is_cpu) {
  return Guard([&] {
    if (!net) throw lc0mi::Error("null network");
    if (minibatch) *minibatch = net->impl->GetMiniBatchSize();
    if (batch_step) *batch_step = net->impl->GetPreferredBatchStep();
    if (max_batch) *max_batch = net->impl->GetMaxBatchSize();
    if (threads) *threads = net->impl->GetThreads();
    if (is_cpu) *is_cpu = net->impl->IsCpu() ? 1 : 0;
  });
}

int lc0mi_comp_create(lc0mi_net* net, lc0mi_comp** out) {
  return Guard([&] {
    if (!net || !out) throw lc0mi::Error("null argument");
    auto c = std::make_unique<lc0mi_comp>();
    c->impl = net->impl->NewComputation();
    *out = c.release();
  });
}

void lc0mi_comp_destroy(lc0mi_comp* comp) { delete comp; }

int lc0mi_comp_add_input(lc0mi_comp* comp, const uint64_t masks[112], const float values[112]) {
  return Guard([&] {
    if (!comp || !masks || !values) throw lc0mi::Error("null argument");
    comp->impl->AddInputs(1, masks, values);
  });
}

int lc0mi_comp_add_inputs(lc0mi_comp* comp, int n, const uint64_t* masks, const float* values) {
  return Guard([&] {
    if (!comp || (n > 0 && (!masks || !values))) throw lc0mi::Error("null argument");
    comp->impl->AddInputs(n, masks, values);
  });
}

int lc0mi_comp_compute_blocking(lc0mi_comp* comp) {
  return Guard([&] {
    if (!comp) throw lc0mi::Error("null computation");
    comp->impl->ComputeBlocking();
  });
}

int lc0mi_comp_batch_size(const lc0mi_comp* comp) { return comp ? comp->impl->GetBatchSize() : 0; }

#define LC0MI_GETTER(expr)                                   \
  float result = std::numeric_limits<float>::quiet_NaN();    \
  Guard([&] {                                                \
    if (!comp) throw lc0mi::Error("null computation");       \
    result = (expr);                                         \
  });                                                        \
  return result;

float lc0mi_comp_q(const lc0mi_comp* comp, int sample) { LC0MI_GETTER(comp->impl->GetQVal(sample)) }
float lc0mi_comp_d(const lc0mi_comp* comp, int sample) { LC0MI_GETTER(comp->impl->GetDVal(sample)) }
float lc0mi_comp_m(const lc0mi_comp* comp, int sample) { LC0MI_GETTER(comp->impl->GetMVal(sample)) }
float lc0mi_comp_p(const lc0mi_comp* comp, int sample, int move_id) {
  float result = std::numeric_limits<float>::quiet_NaN();
  Guard([&] {
    if (!comp) throw lc0mi::Error("null computation");
    if (move_id < 0 || move_id >= lc0mi::kPolicyOutputs) throw lc0mi::Error("move id out of range");
    result = comp->impl->GetPVal(sample, move_id);
  });
  return result;
}

const float* lc0mi_comp_policy_row(const lc0mi_comp* comp, int sample) {
  const float* row = nullptr;
  Guard([&] {
    if (!comp) throw lc0mi::Error("null computation");
    row = comp->impl->GetPolicyRow(sample);
  });
  return row;
}

int lc0mi_comp_add_legal_moves(lc0mi_comp* comp, int n, const uint16_t* move_ids) {
  return Guard([&] {
    if (!comp) throw lc0mi::Error("null computation");
    comp->impl->AddLegalMoves(n, move_ids);
  });
}

int lc0mi_comp_set_policy_softmax_temperature(lc0mi_comp* comp, float temperature) {
  return Guard([&] {
    if (!comp) throw lc0mi::Error("null computation");
    comp->impl->SetPolicySoftmaxTemperature(temperature);
  });
}

const float* lc0mi_comp_legal_policy(const lc0mi_comp* comp, int sample, int* n) {
  const float* probs = nullptr;
  Guard([&] {
    if (!comp) throw lc0mi::Error("null computation");
    probs = comp->impl->GetLegalPolicy(sample, n);
  });
  return probs;
}

const char* lc0mi_last_error(void) { return g_last_error.c_str(); }

int lc0mi_net_set_profiling(lc0mi_net* net, int on) {
  return Guard([&] {
    if (!net) throw lc0mi::Error("null network");
    net->impl->SetProfiling(on != 0);
  });
}

int lc0mi_net_take_profile(lc0mi_net* net, char* buf, int cap) {
  int needed = 0;
  Guard([&] {
    if (!net) throw lc0mi::Error("null network");
    std::string text;
    char line[256];
    for (const auto& k : net->impl->TakeProfile()) {
      std::snprintf(line, sizeof(line), "%s %.6f %d %.6e %.6e\n", k.name.c_str(), k.ms, k.launches, k.flops,
                    k.bytes);
      text += line;
    }
    needed = static_cast<int>(text.size()) + 1;
    if (buf && cap > 0) {
      size_t n = std::min<size_t>(text.size(), static_cast<size_t>(cap) - 1);
      std::memcpy(buf, text.data(), n);
      buf[n] = 0;
    }
  });
  return needed;
}

int lc0mi_net_time_resident_forward(lc0mi_net* net, int batch, int iters, double* ms_per_pass) {
  return Guard([&] {
    if (!net || !ms_per_pass) throw lc0mi::Error("null argument");
    *ms_per_pass = net->impl->TimeResidentForward(batch, iters);
  });
}

int lc0mi_net_calibrate_fp8(lc0mi_net* net, int n, const uint64_t* masks, const float* values) {
  return Guard([&] {
    if (!net) throw lc0mi::Error("null network");
    net->impl->CalibrateFp8(n, masks, values);
  });
}

int lc0mi_net_fp8_scales(const lc0mi_net* net, float* out, int cap) {
  int needed = -1;
  Guard([&] {
    if (!net) throw lc0mi::Error("null network");
    const std::vector<float> v = net->impl->Fp8Scales();
    if (out != nullptr && cap > 0) std::memcpy(out, v.data(), sizeof(float) * std::min<size_t>(v.size(), static_cast<size_t>(cap)));
    needed = static_cast<int>(v.size());
  });
  return needed;
}

}  // extern "C"

// ---- decoded weights, for checking the loader without a GPU ----
namespace {
template <typename F>
void VisitConv(const std::string& name, const lc0mi::ConvBlock& c, F&& f) {
  f(name + ".weights", c.weights);
  f(name + ".biases", c.biases);
}
template <typename F>
void VisitEncoder(const std::string& name, const lc0mi::EncoderLayer& l, F&& f) {
  f(name + ".mha.q_w", l.mha.q_w); f(name + ".mha.q_b", l.mha.q_b);
  f(name + ".mha.k_w", l.mha.k_w); f(name + ".mha.k_b", l.mha.k_b);
  f(name + ".mha.v_w", l.mha.v_w); f(name + ".mha.v_b", l.mha.v_b);
  f(name + ".mha.dense_w", l.mha.dense_w); f(name + ".mha.dense_b", l.mha.dense_b);
  if (l.mha.has_smolgen) {
    const auto& s = l.mha.smolgen;
    f(name + ".mha.smolgen.compress", s.compress);
    f(name + ".mha.smolgen.dense1_w", s.dense1_w); f(name + ".mha.smolgen.dense1_b", s.dense1_b);
    f(name + ".mha.smolgen.ln1_gammas", s.ln1_gammas); f(name + ".mha.smolgen.ln1_betas", s.ln1_betas);
    f(name + ".mha.smolgen.dense2_w", s.dense2_w); f(name + ".mha.smolgen.dense2_b", s.dense2_b);
    f(name + ".mha.smolgen.ln2_gammas", s.ln2_gammas); f(name + ".mha.smolgen.ln2_betas", s.ln2_betas);
  }
  f(name + ".ln1_gammas", l.ln1_gammas); f(name + ".ln1_betas", l.ln1_betas);
  f(name + ".ffn.dense1_w", l.ffn.dense1_w); f(name + ".ffn.dense1_b", l.ffn.dense1_b);
  f(name + ".ffn.dense2_w", l.ffn.dense2_w); f(name + ".ffn.dense2_b", l.ffn.dense2_b);
  f(name + ".ln2_gammas", l.ln2_gammas); f(name + ".ln2_betas", l.ln2_betas);
}
// Calls f(name, tensor) for every tensor of the file, heads resolved and batch norm folded.
template <typename F>
void VisitTensors(const lc0mi::NetWeights& w, F&& f) {
  VisitConv("input", w.input, f);
  for (size_t i = 0; i < w.residual.size(); i++) {
    const std::string n = "residual." + std::to_string(i);
    VisitConv(n + ".conv1", w.residual[i].conv1, f);
    VisitConv(n + ".conv2", w.residual[i].conv2, f);
    if (w.residual[i].has_se) {
      f(n + ".se.w1", w.residual[i].se.w1); f(n + ".se.b1", w.residual[i].se.b1);
      f(n + ".se.w2", w.residual[i].se.w2); f(n + ".se.b2", w.residual[i].se.b2);
    }
  }
  f("ip_emb_preproc_w", w.ip_emb_preproc_w); f("ip_emb_preproc_b", w.ip_emb_preproc_b);
  f("ip_emb_w", w.ip_emb_w); f("ip_emb_b", w.ip_emb_b);
  f("ip_emb_ln_gammas", w.ip_emb_ln_gammas); f("ip_emb_ln_betas", w.ip_emb_ln_betas);
  f("ip_mult_gate", w.ip_mult_gate); f("ip_add_gate", w.ip_add_gate);
  f("ip_emb_ffn.dense1_w", w.ip_emb_ffn.dense1_w); f("ip_emb_ffn.dense1_b", w.ip_emb_ffn.dense1_b);
  f("ip_emb_ffn.dense2_w", w.ip_emb_ffn.dense2_w); f("ip_emb_ffn.dense2_b", w.ip_emb_ffn.dense2_b);
  f("ip_emb_ffn_ln_gammas", w.ip_emb_ffn_ln_gammas); f("ip_emb_ffn_ln_betas", w.ip_emb_ffn_ln_betas);
  for (size_t i = 0; i < w.encoder.size(); i++) VisitEncoder("encoder." + std::to_string(i), w.encoder[i], f);
  VisitConv("moves_left", w.moves_left, f);
  f("ip_mov_w", w.ip_mov_w); f("ip_mov_b", w.ip_mov_b);
  f("ip1_mov_w", w.ip1_mov_w); f("ip1_mov_b", w.ip1_mov_b);
  f("ip2_mov_w", w.ip2_mov_w); f("ip2_mov_b", w.ip2_mov_b);
  f("smolgen_w", w.smolgen_w);
  for (const auto& kv : w.policy_heads) {
    const std::string n = "policy_heads." + kv.first;
    const auto& h = kv.second;
    f(n + ".ip_pol_w", h.ip_pol_w); f(n + ".ip_pol_b", h.ip_pol_b);
    VisitConv(n + ".policy1", h.policy1, f);
    VisitConv(n + ".policy", h.policy, f);
    f(n + ".ip2_pol_w", h.ip2_pol_w); f(n + ".ip2_pol_b", h.ip2_pol_b);
    f(n + ".ip3_pol_w", h.ip3_pol_w); f(n + ".ip3_pol_b", h.ip3_pol_b);
    f(n + ".ip4_pol_w", h.ip4_pol_w);
    for (size_t i = 0; i < h.pol_encoder.size(); i++) VisitEncoder(n + ".pol_encoder." + std::to_string(i), h.pol_encoder[i], f);
  }
  for (const auto& kv : w.value_heads) {
    const std::string n = "value_heads." + kv.first;
    const auto& h = kv.second;
    VisitConv(n + ".value", h.value, f);
    f(n + ".ip_val_w", h.ip_val_w); f(n + ".ip_val_b", h.ip_val_b);
    f(n + ".ip1_val_w", h.ip1_val_w); f(n + ".ip1_val_b", h.ip1_val_b);
    f(n + ".ip2_val_w", h.ip2_val_w); f(n + ".ip2_val_b", h.ip2_val_b);
  }
}
}  // namespace

extern "C" {

int lc0mi_weights_list(const void* data, size_t len, char* buf, int cap) {
  int needed = -1;
  const int rc = Guard([&] {
    if (!data) throw lc0mi::Error("null argument");
    std::string raw = lc0mi::MaybeGunzip(data, len);
    const lc0mi::WeightsFile file = lc0mi::ParseWeightsProto(raw.data(), raw.size());
    const auto& nf = file.format;
    std::string text = "format input=" + std::to_string(nf.input) + " output=" + std::to_string(nf.output) +
                       " network=" + std::to_string(nf.network) + " policy=" + std::to_string(nf.policy) +
                       " value=" + std::to_string(nf.value) + " moves_left=" + std::to_string(nf.moves_left) +
                       " default_activation=" + std::to_string(nf.default_activation) +
                       " smolgen_activation=" + std::to_string(nf.smolgen_activation) +
                       " ffn_activation=" + std::to_string(nf.ffn_activation) +
                       " input_embedding=" + std::to_string(nf.input_embedding) +
                       " headcount=" + std::to_string(file.weights.encoder_head_count) + "\n";
    VisitTensors(file.weights, [&](const std::string& name, const lc0mi::Vec& v) {
      if (!v.empty()) text += name + " " + std::to_string(v.size()) + "\n";
    });
    needed = static_cast<int>(text.size()) + 1;
    if (buf && cap > 0) {
      const size_t n = std::min<size_t>(text.size(), static_cast<size_t>(cap) - 1);
      std::memcpy(buf, text.data(), n);
      buf[n] = 0;
    }
  });
  return rc ? -1 : needed;
}

long long lc0mi_weights_tensor(const void* data, size_t len, const char* name, float* out, long long cap) {
  long long count = -1;
  const int rc = Guard([&] {
    if (!data || !name) throw lc0mi::Error("null argument");
    std::string raw = lc0mi::MaybeGunzip(data, len);
    const lc0mi::WeightsFile file = lc0mi::ParseWeightsProto(raw.data(), raw.size());
    VisitTensors(file.weights, [&](const std::string& n, const lc0mi::Vec& v) {
      if (n != name) return;
      count = static_cast<long long>(v.size());
      if (out) std::memcpy(out, v.data(), sizeof(float) * static_cast<size_t>(std::min<long long>(count, cap)));
    });
    if (count < 0) throw lc0mi::Error(std::string("no tensor named ") + name);
  });
  return rc ? -1 : count;
}

const int16_t* lc0mi_attn_policy_map(int* count) {
  const auto& m = lc0mi::AttnPolicyMap();
  if (count) *count = static_cast<int>(m.size());
  return m.data();
}
const int16_t* lc0mi_conv_policy_map(int* count) {
  const auto& m = lc0mi::ConvPolicyMap();
  if (count) *count = static_cast<int>(m.size());
  return m.data();
}
const float* lc0mi_pos_encoding(int* count) {
  const auto& m = lc0mi::PosEncoding();
  if (count) *count = static_cast<int>(m.size());
  return m.data();
}

}  // extern "C"
