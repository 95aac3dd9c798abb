// lc0-side adapter: registers the MI355X backend with lc0's network factory.
//
// This file is meant to be dropped into an lc0 source tree as
// src/neural/backends/mi355x/network_mi355x.cc and linked against liblc0mi.so
// (include/lc0mi.h). It forwards lc0's Network / NetworkComputation virtuals
// (src/neural/network.h:56-71,116-126) to the C ABI one to one and turns error
// codes back into lczero::Exception, which is what lc0 expects from a backend
// (src/neural/backends/blas/network_blas.cc:1118-1180 throws the same way).
//
// It is not compiled as part of liblc0mi.so: it needs lc0's headers.
#include <memory>
#include <optional>
#include <random>
#include <string>
#include <vector>

#include "chess/position.h"
#include "lc0mi.h"
#include "neural/encoder.h"
#include "neural/factory.h"
#include "neural/network.h"
#include "utils/exception.h"
#include "utils/optionsdict.h"

namespace lczero {
namespace {

void Check(int rc) {
  if (rc != 0) throw Exception(std::string("mi355x: ") + lc0mi_last_error());
}

class Mi355xComputation : public NetworkComputation {
 public:
  explicit Mi355xComputation(lc0mi_net* net) { Check(lc0mi_comp_create(net, &comp_)); }
  ~Mi355xComputation() override { lc0mi_comp_destroy(comp_); }

  void AddInput(InputPlanes&& input) override {
    if (input.size() != static_cast<size_t>(kInputPlanes)) {
      throw Exception("mi355x: AddInput expects 112 planes");
    }
    uint64_t masks[kInputPlanes];
    float values[kInputPlanes];
    for (int i = 0; i < kInputPlanes; ++i) {
      masks[i] = input[i].mask;
      values[i] = input[i].value;
    }
    Check(lc0mi_comp_add_input(comp_, masks, values));
  }
  void ComputeBlocking() override { Check(lc0mi_comp_compute_blocking(comp_)); }
  int GetBatchSize() const override { return lc0mi_comp_batch_size(comp_); }
  float GetQVal(int sample) const override { return lc0mi_comp_q(comp_, sample); }
  float GetDVal(int sample) const override { return lc0mi_comp_d(comp_, sample); }
  float GetMVal(int sample) const override { return lc0mi_comp_m(comp_, sample); }
  float GetPVal(int sample, int move_id) const override {
    // One pointer fetch per sample, then plain array reads: the caller asks
    // for every legal move of the sample in a row (src/neural/wrapper.cc:135-156).
    if (sample != cached_sample_) {
      cached_row_ = lc0mi_comp_policy_row(comp_, sample);
      if (!cached_row_) throw Exception(std::string("mi355x: ") + lc0mi_last_error());
      cached_sample_ = sample;
    }
    return cached_row_[move_id];
  }

 private:
  lc0mi_comp* comp_ = nullptr;
  mutable int cached_sample_ = -1;
  mutable const float* cached_row_ = nullptr;
};

class Mi355xNetwork : public Network {
 public:
  Mi355xNetwork(const WeightsFile& file, const OptionsDict& options) {
    // Options understood by the backend (unknown keys are reported by lc0 itself
    // through OptionsDict::CheckAllOptionsRead, src/neural/wrapper.cc:194).
    std::string kv;
    auto add = [&kv](const std::string& k, const std::string& v) {
      if (!kv.empty()) kv += ',';
      kv += k + '=' + v;
    };
    add("gpu", std::to_string(options.GetOrDefault<int>("gpu", 0)));
    add("max_batch", std::to_string(options.GetOrDefault<int>("max_batch", 1024)));
    add("lanes", std::to_string(options.GetOrDefault<int>("lanes", 4)));
    add("graphs", options.GetOrDefault<bool>("graphs", true) ? "true" : "false");
    add("overlap_min_batch", std::to_string(options.GetOrDefault<int>("overlap_min_batch", -1)));
    add("heads_overlap_min_batch", std::to_string(options.GetOrDefault<int>("heads_overlap_min_batch", -1)));
    add("fused_smolgen_attention", options.GetOrDefault<bool>("fused_smolgen_attention", true) ? "true" : "false");
    add("fused_smolgen_min_batch", std::to_string(options.GetOrDefault<int>("fused_smolgen_min_batch", 72)));
    add("dense1_split_min_batch", std::to_string(options.GetOrDefault<int>("dense1_split_min_batch", 112)));
    add("chain_latency_max_batch", std::to_string(options.GetOrDefault<int>("chain_latency_max_batch", 128)));
    add("fold_layer_norm", options.GetOrDefault<bool>("fold_layer_norm", false) ? "true" : "false");
    const std::string precision = options.GetOrDefault<std::string>("precision", "fp16");
    add("precision", precision);
    if (precision == "fp8") {
      add("fp8_gemms", options.GetOrDefault<std::string>("fp8_gemms", "auto"));
      add("fp8_fp16_layers", std::to_string(options.GetOrDefault<int>("fp8_fp16_layers", 0)));
    }
    add("qkv_first", options.GetOrDefault<bool>("qkv_first", true) ? "true" : "false");
    add("write_through", options.GetOrDefault<bool>("write_through", true) ? "true" : "false");
    add("policy_head", options.GetOrDefault<std::string>("policy_head", "vanilla"));
    add("value_head", options.GetOrDefault<std::string>("value_head", "winner"));
    add("mlh", options.GetOrDefault<bool>("mlh", true) ? "true" : "false");
    const std::string raw = file.OutputAsString();
    Check(lc0mi_net_create_from_buffer(raw.data(), raw.size(), kv.c_str(), &net_));
    int in = 0, out = 0, mlh = 0;
    Check(lc0mi_net_caps(net_, &in, &out, &mlh));
    capabilities_ = {static_cast<pblczero::NetworkFormat::InputFormat>(in),
                     static_cast<pblczero::NetworkFormat::OutputFormat>(out),
                     static_cast<pblczero::NetworkFormat::MovesLeftFormat>(mlh)};
    Check(lc0mi_net_hints(net_, &minibatch_, &batch_step_, nullptr, &threads_, nullptr));
    if (precision == "fp8") CalibrateFp8(capabilities_.input_format);
  }
  ~Mi355xNetwork() override { lc0mi_net_destroy(net_); }

  // The library calibrates its fp8 activation scales on built-in pseudo-positions; here
  // lc0's own move generator and encoder are at hand, so it gets real ones instead:
  // positions reached by seeded uniform-random legal playouts from the start position.
  void CalibrateFp8(pblczero::NetworkFormat::InputFormat input_format) {
    constexpr int kPositions = 256;
    std::vector<uint64_t> masks(static_cast<size_t>(kPositions) * kInputPlanes);
    std::vector<float> values(masks.size());
    std::mt19937 rng(20240);
    int filled = 0;
    while (filled < kPositions) {
      PositionHistory history;
      history.Reset(ChessBoard::kStartposBoard, 0, 1);
      const int plies = 10 + static_cast<int>(rng() % 71);
      for (int ply = 0; ply < plies; ++ply) {
        const MoveList moves = history.Last().GetBoard().GenerateLegalMoves();
        if (moves.empty() || history.ComputeGameResult() != GameResult::UNDECIDED) break;
        history.Append(moves[rng() % moves.size()]);
      }
      const InputPlanes planes =
          EncodePositionForNN(input_format, history, 8, FillEmptyHistory::FEN_ONLY, nullptr);
      for (int i = 0; i < kInputPlanes; ++i) {
        masks[static_cast<size_t>(filled) * kInputPlanes + i] = planes[i].mask;
        values[static_cast<size_t>(filled) * kInputPlanes + i] = planes[i].value;
      }
      ++filled;
    }
    Check(lc0mi_net_calibrate_fp8(net_, kPositions, masks.data(), values.data()));
  }

  const NetworkCapabilities& GetCapabilities() const override { return capabilities_; }
  std::unique_ptr<NetworkComputation> NewComputation() override {
    return std::make_unique<Mi355xComputation>(net_);
  }
  int GetThreads() const override { return threads_; }
  bool IsCpu() const override { return false; }
  int GetMiniBatchSize() const override { return minibatch_; }
  int GetPreferredBatchStep() const override { return batch_step_; }

 private:
  lc0mi_net* net_ = nullptr;
  NetworkCapabilities capabilities_;
  int minibatch_ = 256, batch_step_ = 1, threads_ = 1;
};

std::unique_ptr<Network> MakeMi355xNetwork(const std::optional<WeightsFile>& w, const OptionsDict& options) {
  if (!w) throw Exception("The mi355x backend requires a network file.");
  return std::make_unique<Mi355xNetwork>(*w, options);
}

// Above cuda-auto (104) and below sycl-auto (132) would make it the default on
// a machine that has it; 90 keeps it opt-in next to the vendor backends.
REGISTER_NETWORK("mi355x", MakeMi355xNetwork, 90)

}  // namespace
}  // namespace lczero
