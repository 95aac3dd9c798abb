// lc0-side adapter, second form: the MI355X library behind lc0's Backend interface
// (src/neural/backend.h:75-125) instead of the older Network interface.
//
// network_mi355x.cc registers a Network; lc0 then wraps it in NetworkAsBackend
// (src/neural/wrapper.cc:48-160), which downloads all 1858 logits of every position and
// runs the legal-move softmax on the host. A Backend receives the legal moves together
// with the position (EvalPosition, src/neural/backend.h:69-72), so this adapter hands their
// policy indices to the library: the softmax of wrapper.cc:135-156 then runs on the GPU
// with the same float arithmetic and only the probabilities of the legal moves are copied
// back, straight into the spans the search gave us.
//
// Drop into an lc0 tree as src/neural/backends/mi355x/backend_mi355x.cc next to
// network_mi355x.cc (register only one of the two under a given name) and link against
// liblc0mi.so. It is not compiled as part of liblc0mi.so: it needs lc0's headers.
#include <algorithm>
#include <memory>
#include <optional>
#include <string>
#include <vector>

#include "lc0mi.h"
#include "neural/backend.h"
#include "neural/encoder.h"
#include "neural/loader.h"
#include "neural/network.h"
#include "neural/register.h"
#include "neural/shared_params.h"
#include "utils/exception.h"
#include "utils/optionsdict.h"

namespace lczero {
namespace {

void Check(int rc) {
  if (rc != 0) throw Exception(std::string("mi355x: ") + lc0mi_last_error());
}

FillEmptyHistory HistoryFillFromString(const std::string& s) {
  if (s == "fen_only") return FillEmptyHistory::FEN_ONLY;
  if (s == "always") return FillEmptyHistory::ALWAYS;
  return FillEmptyHistory::NO;
}

class Mi355xBackend;

class Mi355xBackendComputation : public BackendComputation {
 public:
  explicit Mi355xBackendComputation(Mi355xBackend* backend);
  ~Mi355xBackendComputation() override { lc0mi_comp_destroy(comp_); }

  size_t UsedBatchSize() const override { return results_.size(); }

  AddInputResult AddInput(const EvalPosition& pos, EvalResultPtr result) override;

  void ComputeBlocking() override {
    if (results_.empty()) return;
    Check(lc0mi_comp_compute_blocking(comp_));
    for (size_t i = 0; i < results_.size(); ++i) {
      const EvalResultPtr& r = results_[i];
      const int s = static_cast<int>(i);
      if (r.q) *r.q = lc0mi_comp_q(comp_, s);
      if (r.d) *r.d = lc0mi_comp_d(comp_, s);
      if (r.m) *r.m = lc0mi_comp_m(comp_, s);
      if (!r.p.empty()) {
        int n = 0;
        const float* p = lc0mi_comp_legal_policy(comp_, s, &n);
        if (!p || static_cast<size_t>(n) != r.p.size()) {
          throw Exception(std::string("mi355x: ") + (p ? "policy size mismatch" : lc0mi_last_error()));
        }
        std::copy(p, p + n, r.p.begin());
      }
    }
  }

 private:
  Mi355xBackend* backend_;
  lc0mi_comp* comp_ = nullptr;
  std::vector<EvalResultPtr> results_;
  std::vector<uint16_t> ids_;
};

class Mi355xBackend : public Backend {
 public:
  explicit Mi355xBackend(const OptionsDict& options)
      : backend_opts_(options.Get<std::string>(SharedBackendParams::kBackendOptionsId)),
        weights_path_(options.Get<std::string>(SharedBackendParams::kWeightsId)) {
    // --backend-opts of this backend are passed through as they are ("gpu=0,precision=fp8,...");
    // the library reports keys it does not know.
    std::optional<WeightsFile> weights = LoadWeights(weights_path_);
    if (!weights) throw Exception("The mi355x backend requires a network file.");
    const std::string raw = weights->OutputAsString();
    Check(lc0mi_net_create_from_buffer(raw.data(), raw.size(), backend_opts_.c_str(), &net_));
    int in = 0, out = 0, mlh = 0;
    Check(lc0mi_net_caps(net_, &in, &out, &mlh));
    input_format_ = static_cast<pblczero::NetworkFormat::InputFormat>(in);
    int minibatch = 256, max_batch = 1024, threads = 1;
    Check(lc0mi_net_hints(net_, &minibatch, nullptr, &max_batch, &threads, nullptr));
    attrs_.has_mlh = mlh != pblczero::NetworkFormat::MOVES_LEFT_NONE;
    attrs_.has_wdl = out == pblczero::NetworkFormat::OUTPUT_WDL;
    attrs_.runs_on_cpu = false;
    attrs_.suggested_num_search_threads = threads;
    attrs_.recommended_batch_size = minibatch;
    attrs_.maximum_batch_size = max_batch;
    UpdateConfiguration(options);
  }
  ~Mi355xBackend() override { lc0mi_net_destroy(net_); }

  BackendAttributes GetAttributes() const override { return attrs_; }
  std::unique_ptr<BackendComputation> CreateComputation() override {
    return std::make_unique<Mi355xBackendComputation>(this);
  }
  UpdateConfigurationResult UpdateConfiguration(const OptionsDict& options) override {
    Backend::UpdateConfiguration(options);
    if (backend_opts_ != options.Get<std::string>(SharedBackendParams::kBackendOptionsId) ||
        weights_path_ != options.Get<std::string>(SharedBackendParams::kWeightsId)) {
      return NEED_RESTART;
    }
    policy_temperature_ = options.Get<float>(SharedBackendParams::kPolicySoftmaxTemp);
    fill_empty_history_ = HistoryFillFromString(options.Get<std::string>(SharedBackendParams::kHistoryFill));
    return UPDATE_OK;
  }

 private:
  friend class Mi355xBackendComputation;
  const std::string backend_opts_;
  const std::string weights_path_;
  lc0mi_net* net_ = nullptr;
  BackendAttributes attrs_;
  pblczero::NetworkFormat::InputFormat input_format_;
  float policy_temperature_ = 1.359f;
  FillEmptyHistory fill_empty_history_ = FillEmptyHistory::FEN_ONLY;
};

Mi355xBackendComputation::Mi355xBackendComputation(Mi355xBackend* backend) : backend_(backend) {
  Check(lc0mi_comp_create(backend->net_, &comp_));
  // The library forms 1 / temperature in float as wrapper.cc:81-82 does.
  Check(lc0mi_comp_set_policy_softmax_temperature(comp_, backend->policy_temperature_));
  results_.reserve(backend->attrs_.maximum_batch_size);
}

BackendComputation::AddInputResult Mi355xBackendComputation::AddInput(const EvalPosition& pos,
                                                                       EvalResultPtr result) {
  int transform = 0;
  const InputPlanes planes =
      EncodePositionForNN(backend_->input_format_, pos.pos, 8, backend_->fill_empty_history_, &transform);
  uint64_t masks[kInputPlanes];
  float values[kInputPlanes];
  for (int i = 0; i < kInputPlanes; ++i) {
    masks[i] = planes[i].mask;
    values[i] = planes[i].value;
  }
  Check(lc0mi_comp_add_input(comp_, masks, values));
  // Same order as the legal-move span: the probabilities come back in that order.
  ids_.clear();
  for (const Move& move : pos.legal_moves) ids_.push_back(MoveToNNIndex(move, transform));
  Check(lc0mi_comp_add_legal_moves(comp_, static_cast<int>(ids_.size()), ids_.data()));
  results_.push_back(result);
  return ENQUEUED_FOR_EVAL;
}

class Mi355xBackendFactory : public BackendFactory {
 public:
  // Same opt-in priority as the Network form (network_mi355x.cc).
  int GetPriority() const override { return 90; }
  std::string_view GetName() const override { return "mi355x-direct"; }
  std::unique_ptr<Backend> Create(const OptionsDict& options) override {
    return std::make_unique<Mi355xBackend>(options);
  }
};

[[maybe_unused]] static BackendManager::Register reg_mi355x_direct(std::make_unique<Mi355xBackendFactory>());

}  // namespace
}  // namespace lczero
