// extern "C" boundary of the backend: translates lc0mi::Error into return
// codes plus a thread-local message and owns the opaque handles.
#include "../../include/lc0mi.h"

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
