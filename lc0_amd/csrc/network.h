// C++ host interface of the MI355X backend. The class and method names mirror
// lc0's backend interface (src/neural/network.h:43-126) so that the lc0
// adapter (network_mi355x.cc) is a one-to-one forwarding layer.
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "weights.h"

namespace lc0mi {

constexpr int kInputPlanes = 112;      // src/neural/network.h:38
constexpr int kPolicyOutputs = 1858;

// src/neural/network.h:43-52
struct InputPlane {
  uint64_t mask = 0;
  float value = 1.0f;
};
using InputPlanes = std::vector<InputPlane>;

// src/neural/network.h:56-71
class NetworkComputation {
 public:
  virtual ~NetworkComputation() = default;
  virtual void AddInput(InputPlanes&& input) = 0;
  // Bulk variant of AddInput: n positions, 112 masks and 112 values each.
  virtual void AddInputs(int n, const uint64_t* masks, const float* values) = 0;
  virtual void ComputeBlocking() = 0;
  virtual int GetBatchSize() const = 0;
  virtual float GetQVal(int sample) const = 0;
  virtual float GetDVal(int sample) const = 0;
  virtual float GetPVal(int sample, int move_id) const = 0;
  virtual float GetMVal(int sample) const = 0;
  // 1858 raw policy logits of one sample (host memory owned by the computation).
  virtual const float* GetPolicyRow(int sample) const = 0;

  // Legal-move policy: the softmax that lc0's search wrapper applies to the logits of the legal moves
  // (NetworkAsBackendComputation::SoftmaxPolicy, src/neural/wrapper.cc:135-156) runs on the device and only
  // those probabilities are downloaded. AddLegalMoves lists the policy indices (MoveToNNIndex,
  // src/neural/encoder.cc:339-619) of the legal moves of the input added last; it must then be called for
  // every input of the computation, and the raw logits (GetPVal, GetPolicyRow) are not available.
  virtual void AddLegalMoves(int n, const uint16_t* move_ids) = 0;
  // Policy softmax temperature (lc0's PolicyTemperature, default 1.359, src/neural/shared_params.cc:69).
  virtual void SetPolicySoftmaxTemperature(float temperature) = 0;
  // Probabilities of the listed moves of one sample, in the order they were listed.
  virtual const float* GetLegalPolicy(int sample, int* n) const = 0;
};

// src/neural/network.h:85-114
struct NetworkCapabilities {
  int input_format = 0;
  int output_format = 0;
  int moves_left = 0;
};

// Backend options, "key=value,key=value" as in lc0's --backend-opts
// (src/utils/optionsdict.cc:81-325, flat subset). Every key must be consumed.
class Options {
 public:
  Options() = default;
  explicit Options(const std::string& kv);
  int GetInt(const std::string& key, int def);
  bool GetBool(const std::string& key, bool def);
  std::string GetString(const std::string& key, const std::string& def);
  // Throws Error naming the first key nobody read (src/utils/optionsdict.cc:330-341).
  void CheckAllOptionsRead(const std::string& backend_name) const;

 private:
  std::map<std::string, std::string> kv_;
  mutable std::map<std::string, bool> read_;
};

// One timed kernel label of a profiled ComputeBlocking.
struct KernelTime {
  std::string name;
  double ms = 0.0;       // summed HIP-event time of all launches with this label
  int launches = 0;
  double flops = 0.0;    // algorithmic flops of those launches
  double bytes = 0.0;    // algorithmic bytes moved by those launches
};

// src/neural/network.h:116-126
class Network {
 public:
  virtual ~Network() = default;
  virtual const NetworkCapabilities& GetCapabilities() const = 0;
  virtual std::unique_ptr<NetworkComputation> NewComputation() = 0;
  virtual int GetThreads() const { return 1; }
  virtual void InitThread(int /*id*/) {}
  virtual bool IsCpu() const { return false; }
  virtual int GetMiniBatchSize() const { return 256; }
  virtual int GetPreferredBatchStep() const { return 1; }
  virtual int GetMaxBatchSize() const = 0;
  // When on, every kernel launch of the next ComputeBlocking calls is bracketed
  // by HIP events on the compute stream; TakeProfile returns and clears them.
  virtual void SetProfiling(bool on) = 0;
  virtual std::vector<KernelTime> TakeProfile() = 0;
  // Runs the device part of the last batch again `iters` times (inputs already
  // resident in HBM) and returns the mean milliseconds per pass measured with
  // HIP events on the compute stream.
  virtual double TimeResidentForward(int batch, int iters) = 0;
  // precision=fp8 only: re-derives the per-tensor activation scales from the maxima
  // that these n positions (packed planes as for AddInputs) produce in an fp16 pass.
  virtual void CalibrateFp8(int n, const uint64_t* masks, const float* values) = 0;
  // precision=fp8 only: the activation scales in use (value = code x scale), seven per encoder layer: the operands of
  // Q/K/V, attention output, FFN1 and FFN2, then of smolgen's first dense layer, second dense layer and generator
  // (1 where that operand stays in fp16).
  virtual std::vector<float> Fp8Scales() const = 0;
};

// Factory: the counterpart of MakeBlasNetwork (src/neural/backends/blas/network_blas.cc:1115-1182).
std::unique_ptr<Network> MakeMi355xNetwork(const WeightsFile& weights, Options& options);

}  // namespace lc0mi
