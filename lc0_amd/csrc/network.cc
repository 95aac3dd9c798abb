// MI355X network backend: weight preparation, buffer management and the
// launch sequence of the forward pass.
//
// Forward pass semantics follow lc0's blas backend (reference file:line):
//   format validation / options        blas/network_blas.cc:983-1072,1115-1182
//   attention body prologue            blas/network_blas.cc:603-721
//   encoder layer                      blas/network_blas.cc:271-471
//   value / moves-left / policy heads  blas/network_blas.cc:725-968
//   WDL softmax, q = w - l             blas/network_blas.cc:86-111,747-762
#include "network.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <condition_variable>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>

#include "kernels.h"
#include "tables.h"

namespace lc0mi {

#define HIP_CHECK(expr)                                                                      \
  do {                                                                                       \
    hipError_t err__ = (expr);                                                               \
    if (err__ != hipSuccess) {                                                               \
      throw Error(std::string("HIP error: ") + hipGetErrorString(err__) + " (" #expr ") at " \
                  __FILE__ ":" + std::to_string(__LINE__));                                  \
    }                                                                                        \
  } while (0)

// ------------------------------------------------------------------ options --
Options::Options(const std::string& kv) {
  std::string item;
  std::stringstream ss(kv);
  while (std::getline(ss, item, ',')) {
    size_t b = item.find_first_not_of(" \t");
    if (b == std::string::npos) continue;
    size_t e = item.find_last_not_of(" \t");
    item = item.substr(b, e - b + 1);
    size_t eq = item.find('=');
    if (eq == std::string::npos) {
      kv_[item] = "true";
    } else {
      kv_[item.substr(0, eq)] = item.substr(eq + 1);
    }
  }
}
int Options::GetInt(const std::string& key, int def) {
  auto it = kv_.find(key);
  if (it == kv_.end()) return def;
  read_[key] = true;
  try {
    size_t pos = 0;
    int v = std::stoi(it->second, &pos);
    if (pos != it->second.size()) throw std::invalid_argument("trailing");
    return v;
  } catch (const std::exception&) {
    throw Error("Option '" + key + "' expects an integer, got '" + it->second + "'.");
  }
}
bool Options::GetBool(const std::string& key, bool def) {
  auto it = kv_.find(key);
  if (it == kv_.end()) return def;
  read_[key] = true;
  if (it->second == "true" || it->second == "1") return true;
  if (it->second == "false" || it->second == "0") return false;
  throw Error("Option '" + key + "' expects true/false, got '" + it->second + "'.");
}
std::string Options::GetString(const std::string& key, const std::string& def) {
  auto it = kv_.find(key);
  if (it == kv_.end()) return def;
  read_[key] = true;
  return it->second;
}
void Options::CheckAllOptionsRead(const std::string& backend_name) const {
  for (const auto& kv : kv_) {
    if (!read_.count(kv.first)) {
      throw Error("Unknown option '" + kv.first + "' for backend " + backend_name + ".");
    }
  }
}

namespace {

// -------------------------------------------------------------- device memory --
class DeviceArena {
 public:
  ~DeviceArena() {
    for (void* p : ptrs_) (void)hipFree(p);
  }
  void* Alloc(size_t bytes) {
    void* p = nullptr;
    HIP_CHECK(hipMalloc(&p, std::max<size_t>(bytes, 256)));
    ptrs_.push_back(p);
    total_ += bytes;
    return p;
  }
  template <typename T>
  T* Upload(const std::vector<T>& host) {
    T* d = static_cast<T*>(Alloc(host.size() * sizeof(T)));
    if (!host.empty()) HIP_CHECK(hipMemcpy(d, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
  }
  size_t total() const { return total_; }

 private:
  std::vector<void*> ptrs_;
  size_t total_ = 0;
};

// (Weights and activations of an attention body are typed half_t* whatever the network's element type is: the same
// storage holds bfloat16 bits with precision=bf16, and twice as many bytes holding floats with precision=fp32. The
// launch helpers of Mi355xNetwork pick the kernels by dtype_; nothing else dereferences these pointers.)
struct Linear {
  half_t* w = nullptr;   // [out][ld] elements, K zero-padded to ld
  float* b = nullptr;    // [out] or null
  int out = 0, in = 0, ld = 0;
  float* c = nullptr;    // [out] row sums of w, for a layer whose input layer norm is folded into it (GemmArgs::col_c)
};

// The layer-norm side of one GEMM launch (see GemmArgs in kernels.h): the statistics of the rows the GEMM reads
// (consumer), or the residual it adds and the statistics it leaves (producer).
struct NormFold {
  const float* row_stats = nullptr;
  int row_parts = 0;
  const half_t* skip = nullptr;
  int ldskip = 0;
  const float* skip_stats = nullptr;
  int skip_parts = 0;
  const float* skip_gamma = nullptr;
  const float* skip_beta = nullptr;
  float* stats_out = nullptr;
  int* parts_out = nullptr;      // receives the number of partial sums per row written to stats_out
  const float* bias = nullptr;   // replaces the layer's bias (producer: bias x scale)
  float scale = 1.0f;
  int norm_n = 0;
  float eps = 0.0f;
};

int RoundUp(int v, int m) { return (v + m - 1) / m * m; }

// Residual-tower device weights (element type chosen by the precision option).
struct ConvDev {
  void* u = nullptr;      // [36][cout][ld] winograd-domain filter
  float* bias = nullptr;  // [cout]
  int cin = 0, cout = 0, ld = 0;
};
struct SeDev {
  float *w1 = nullptr, *b1 = nullptr, *w2 = nullptr, *b2 = nullptr;
  int k = 0;
};
struct ResBlockDev {
  ConvDev conv1, conv2;
  bool has_se = false;
  SeDev se;
};
struct LinearT {
  void* w = nullptr;      // [out][ld]
  float* b = nullptr;
  int out = 0, in = 0, ld = 0;
};

// e4m3 copy of a dense layer: one scale per output row (absmax / 448).
struct LinearF8 {
  uint8_t* w = nullptr;        // [out][in] e4m3 codes
  std::vector<float> wscale;   // [out], host copy
  float* col_scale = nullptr;  // [out] device: activation scale x wscale (set by calibration)
};

struct EncoderDev {
  Linear qkv, dense, ffn1, ffn2;
  LinearF8 qkv8, dense8, ffn18, ffn28;
  // Per-tensor activation scales (value = code x scale) of the four fp8 operands.
  float s_x = 1.0f, s_att = 1.0f, s_x1 = 1.0f, s_ffn = 1.0f;
  float *ln1_g = nullptr, *ln1_b = nullptr, *ln2_g = nullptr, *ln2_b = nullptr;
  bool has_smolgen = false;
  Linear sg_compress, sg_dense1, sg_dense2;
  // Option fp8_gemms=...+smolgen: e4m3 copies of the chain's layers (sg_global8: the shared generator weights with
  // this layer's activation scale) and the scales of their three operands besides x.
  LinearF8 sg_compress8, sg_dense18, sg_dense28, sg_global8;
  float s_sg1 = 1.0f, s_sg2 = 1.0f, s_sg3 = 1.0f;
  float *sg_ln1_g = nullptr, *sg_ln1_b = nullptr, *sg_ln2_g = nullptr, *sg_ln2_b = nullptr;
  // Folded layer norms: the three layers that read normalised rows, with the gamma / beta of the norm before them
  // multiplied in (qkv and sg_compress: the second norm of the previous encoder layer, absent in the first layer;
  // ffn1: this layer's first norm), and the biases of the two layers before a norm times the DeepNorm alpha.
  Linear qkv_n, sg_compress_n, ffn1_n;
  float *dense_ab = nullptr, *ffn2_ab = nullptr;
};

// Pinned host staging of one batch (inputs and outputs).
struct HostSlot {
  uint64_t* masks = nullptr;
  float* values = nullptr;
  float* policy = nullptr;
  float* wdl = nullptr;   // raw value-head outputs, 3 (WDL) or 1 per sample
  float* mlh = nullptr;
  int capacity = 0;
  // Legal-move lists (allocated when a computation first gives one): legal_off[i] .. legal_off[i + 1] index the
  // ids and the probabilities of sample i; legal_samples counts the samples that have a list.
  int* legal_off = nullptr;        // [capacity + 1]
  uint16_t* legal_ids = nullptr;   // [capacity * kMaxLegalMoves]
  float* legal_probs = nullptr;    // [capacity * kMaxLegalMoves]
  int legal_samples = 0;
  float inv_temperature = 1.0f;
  ~HostSlot() {
    if (legal_off) (void)hipHostFree(legal_off);
    if (legal_ids) (void)hipHostFree(legal_ids);
    if (legal_probs) (void)hipHostFree(legal_probs);
    if (masks) (void)hipHostFree(masks);
    if (values) (void)hipHostFree(values);
    if (policy) (void)hipHostFree(policy);
    if (wdl) (void)hipHostFree(wdl);
    if (mlh) (void)hipHostFree(mlh);
  }
};

class Mi355xNetwork;

// Free list of pinned staging slots. Shared by the network and its computations
// so that a computation destroyed after its network still has a valid place to
// return its slots to.
struct SlotPool {
  std::mutex mutex;
  std::vector<std::unique_ptr<HostSlot>> free_slots;
  bool network_alive = true;
};

class Mi355xComputation : public NetworkComputation {
 public:
  Mi355xComputation(Mi355xNetwork* net, std::shared_ptr<SlotPool> pool) : net_(net), pool_(std::move(pool)) {}
  ~Mi355xComputation() override;
  void AddInput(InputPlanes&& input) override;
  void AddInputs(int n, const uint64_t* masks, const float* values) override;
  void ComputeBlocking() override;
  int GetBatchSize() const override { return batch_; }
  float GetQVal(int sample) const override;
  float GetDVal(int sample) const override;
  float GetPVal(int sample, int move_id) const override { return GetPolicyRow(sample)[move_id]; }
  float GetMVal(int sample) const override;
  const float* GetPolicyRow(int sample) const override;
  void AddLegalMoves(int n, const uint16_t* move_ids) override;
  void SetPolicySoftmaxTemperature(float temperature) override;
  const float* GetLegalPolicy(int sample, int* n) const override;

 private:
  void CheckSample(int sample) const {
    if (sample < 0 || sample >= batch_) throw Error("sample index out of range");
    if (!computed_) throw Error("ComputeBlocking() has not been called");
  }
  HostSlot* SlotFor(int index);
  Mi355xNetwork* Net() const {
    if (!pool_->network_alive) throw Error("the network of this computation has been destroyed");
    return net_;
  }
  Mi355xNetwork* net_;
  std::shared_ptr<SlotPool> pool_;
  int max_batch_ = 0;
  bool wdl_ = false, moves_left_ = false;
  std::vector<std::unique_ptr<HostSlot>> slots_;
  int batch_ = 0;
  bool computed_ = false;
  bool legal_mode_ = false;           // legal-move lists were given: probabilities instead of raw logits
  float temperature_ = 1.359f;        // src/neural/shared_params.cc:69
};

// Everything that describes the loaded network and is the same for every lane: options,
// dimensions and device weights (pointers into the arena of the network that loaded them).
struct ModelState {
  NetworkCapabilities caps_;
  int device_ = 0;
  int max_batch_ = 1024;
  bool wdl_ = false, moves_left_ = false, attn_body_ = false, attn_policy_ = false, conv_policy_ = false;
  int default_act_ = kActRelu, smolgen_act_ = kActNone, ffn_act_ = kActNone;
  std::string policy_head_, value_head_;
  bool use_graphs_ = true;
  int overlap_min_batch_ = 0;   // smallest batch whose smolgen chain runs on the side stream
  int heads_overlap_min_batch_ = -1;   // smallest batch whose value and moves-left heads run beside the policy head (-1: automatic)

  // Attention body dimensions.
  int emb_ = 0, d_model_ = 0, heads_ = 0, dff_ = 0, in_ld_ = 192;
  int sg_hc_ = 0, sg_hs_ = 0, sg_gen_ = 0;
  int pol_emb_ = 0, pol_d_ = 0, val_ch_ = 0, val_fc_ = 0, val_out_ = 0, mov_ch_ = 0, mov_fc_ = 0;
  float alpha_ = 1.0f, eps_ = 1e-6f;
  bool fold_layer_norm_ = false;
  bool fused_smolgen_attention_ = true;
  int fused_smolgen_min_batch_ = 72;
  int dense1_split_min_batch_ = 112;   // smallest batch whose smolgen dense1 splits K between workgroups
  bool qkv_first_ = true;
  bool write_through_ = true;   // big activations go to the memory-side cache while a layer's worth fits it
  int chain_latency_max_batch_ = 128;   // largest fp16 batch whose smolgen chain takes the shortest-latency GEMM variants
  half_t* smolgen_wfrag_ = nullptr;   // smolgen_w in the fragment order of smolgen_attention_kernel (null: not fused)
  bool any_smolgen_ = false;
  // Dense position encoding (PE_DENSE nets): preprocessing layer, embedding layer norm and
  // embedding FFN; optional input gating.
  bool pe_dense_ = false, gating_ = false;
  int enc_ch_ = 0, emb_dff_ = 0;
  Linear preproc_lin_, emb_ffn1_, emb_ffn2_;
  float *emb_ln_g_ = nullptr, *emb_ln_b_ = nullptr, *emb_ffn_ln_g_ = nullptr, *emb_ffn_ln_b_ = nullptr;
  float *gate_mult_ = nullptr, *gate_add_ = nullptr;   // [64][emb]

  // Device weights.
  Linear emb_lin_, smolgen_w_, pol_emb_lin_, pol_qk_lin_, val_emb_lin_, val_fc1_, val_fc2_, mov_emb_lin_, mov_fc1_,
      mov_fc2_;
  std::vector<EncoderDev> encoders_;
  int depth_ = 32;   // attention head depth of the body
  // Policy-head encoder layers (network_blas.cc:836-842): post-LN layers without smolgen on the policy embedding.
  std::vector<EncoderDev> pol_encoders_;
  int pe_heads_ = 0, pe_dmodel_ = 0, pe_dff_ = 0, pe_depth_ = 32, pe_ffn_act_ = kActNone, pol_emb_act_ = kActNone;
  bool pe_smolgen_ = false;                      // policy encoder layers with smolgen (network_blas.cc:836-842)
  int pe_sg_hc_ = 0, pe_sg_hs_ = 0, pe_sg_gen_ = 0;
  half_t* pos_enc_ = nullptr;
  float* ppo_ = nullptr;
  int16_t* inv_map_ = nullptr;

  // fp8 configuration: the four large GEMMs of every encoder layer run on e4m3 operands.
  bool fp8_ = false;
  bool q_qkv_ = true, q_dense_ = true, q_ffn1_ = true, q_ffn2_ = true;   // option fp8_gemms
  bool q_smolgen_ = false;   // ... +smolgen: the four layers of the smolgen chain as well
  bool q_smolgen_auto_ = false;   // fp8_gemms=auto: the chain too, if its widths are multiples of 128
  uint8_t* smolgen_w8_ = nullptr;        // e4m3 codes of the shared generator layer (rows in SmolgenBiasIndex order)
  std::vector<float> smolgen_w8_scale_;  // their per-row scales
  int fp8_fp16_layers_ = 0;   // option fp8_fp16_layers: the last that many encoder layers keep fp16 operands

  // Element type of activations and weights (option precision: fp16, bf16, fp32; fp8 is fp16 with e4m3 operands in
  // the large GEMMs) and its size in bytes.
  Dtype dtype_ = Dtype::kHalf;
  size_t es_ = 2;

  // Residual tower.
  bool fp32_ = false;
  int filters_ = 0;
  bool classical_value_ = false;
  ConvDev res_input_, res_policy1_, res_policy_conv_;
  std::vector<ResBlockDev> res_blocks_;
  LinearT res_pol_conv1x1_, res_pol_fc_, res_val_conv_, res_val_fc1_, res_val_fc2_, res_mov_conv_, res_mov_fc1_,
      res_mov_fc2_;
  int16_t* conv_inv_map_ = nullptr;
  size_t res_max_fc_ = 0, res_cmax_ = 0;
};

class Mi355xNetwork : public Network, protected ModelState {
 public:
  struct LaneTag {};
  Mi355xNetwork(const WeightsFile& file, Options& options);
  Mi355xNetwork(const Mi355xNetwork& parent, LaneTag);   // one more lane on the parent's weights
  ~Mi355xNetwork() override;

  const NetworkCapabilities& GetCapabilities() const override { return caps_; }
  std::unique_ptr<NetworkComputation> NewComputation() override {
    return std::make_unique<Mi355xComputation>(this, pool_);
  }
  int GetMiniBatchSize() const override { return 256; }
  int GetMaxBatchSize() const override { return max_batch_; }
  void SetProfiling(bool on) override {
    std::lock_guard<std::mutex> lock(eval_mutex_);
    profiling_ = on;
  }
  std::vector<KernelTime> TakeProfile() override;
  double TimeResidentForward(int batch, int iters) override;
  void CalibrateFp8(int n, const uint64_t* masks, const float* values) override;
  std::vector<float> Fp8Scales() const override;

  // Used by the computation.
  std::unique_ptr<HostSlot> GetSlot();
  void ReleaseSlot(std::unique_ptr<HostSlot> slot);
  void Evaluate(HostSlot* slot, int batch);
  bool wdl() const { return wdl_; }
  bool moves_left() const { return moves_left_; }

 private:
  void BuildAttentionBody(const WeightsFile& file);
  template <typename T>
  void BuildResnet(const WeightsFile& file);
  void ForwardDevice(int batch);
  void ForwardAttentionBody(int B);
  void BuildAttentionPolicy(const NetWeights& w, const PolicyHead& ph, int in_channels);
  void ForwardAttentionPolicy(const half_t* x, int ld_x, int B);
  EncoderDev MakeEncoderLayer(const EncoderLayer& l, int emb, int d_model, int dff);
  // Smolgen weights of one encoder layer; hc / hs / gen receive (or are checked against) the chain's widths.
  void LoadSmolgen(const Smolgen& s, int emb, int heads, EncoderDev* e, int* hc, int* hs, int* gen, bool* any);
  // The shared generator layer smolgen_w (4096 x g), rows in the order the attention kernels read the logits.
  void EnsureSmolgenGlobal(const NetWeights& w, int g);
  template <typename T>
  void ForwardResnet(int B);
  template <typename T>
  bool WinogradConv(const char* name, const struct ConvDev& conv, const void* x, const void* skip, const struct SeDev* se,
                    int act, void* out, int B, bool have_v = false, const struct ConvDev* next = nullptr);
  template <typename T>
  void GemmT(const char* name, const void* A, int lda, long long strideA, const void* W, int ldw, long long strideW,
             void* C, int ldc, long long strideC, const float* bias, int M, int N, int K, int batch, int act,
             bool out_f32);
  template <typename T>
  struct LinearT MakeLinearT(const Vec& w, const Vec& b, int out, int in);
  Linear MakeLinear(const Vec& w, const Vec& b, int out, int in, int pad_to = 8);
  Linear MakeLinearNormFolded(const Vec& w, const Vec& b, const Vec& gamma, const Vec& beta, int out, int in);
  LinearF8 MakeLinearF8(const Vec& w, int out, int in);
  void GemmF8(const char* name, const uint8_t* A, const Linear& lin, const LinearF8& q, void* C, int M, int act,
              bool out_f8, float out_mul, hipStream_t st = nullptr, int out_stores = kStoresAuto);
  void RecordAbsMax(const half_t* x, size_t n, int slot, hipStream_t st = nullptr);
  // Slot of the calibration maxima: 4 per layer plus the last layer's output, then 3 per layer for the smolgen chain.
  int SmolgenSlot(size_t li, int which) const { return static_cast<int>(4 * encoders_.size() + 1 + 3 * li + which); }
  size_t CalibrationSlots() const { return 7 * encoders_.size() + 1; }
  void ApplyCalibration(const std::vector<float>& absmax);
  void CalibrateExclusive(int n, const uint64_t* masks, const float* values);
  void DefaultCalibration();
  float* UploadF(const Vec& v) { return arena_.Upload(v); }
  // Uploads a per-channel parameter vector after checking its length.
  float* UploadN(const Vec& v, int n, const char* what) {
    if (static_cast<int>(v.size()) != n) {
      throw Error(std::string(what) + " has " + std::to_string(v.size()) + " elements, expected " + std::to_string(n) + ".");
    }
    return arena_.Upload(v);
  }
  // n elements of the network's element type.
  half_t* AllocH(size_t n) { return static_cast<half_t*>(arena_.Alloc(n * es_)); }
  // p advanced by n elements of the network's element type.
  const half_t* ElemAt(const half_t* p, size_t n) const {
    return reinterpret_cast<const half_t*>(reinterpret_cast<const char*>(p) + n * es_);
  }
  // Uploads values converted to the network's element type.
  half_t* UploadElems(const std::vector<float>& v);
  float* AllocF(size_t n) { return static_cast<float*>(arena_.Alloc(n * sizeof(float))); }

  // Launch helpers (profiling aware).
  template <typename F>
  void Timed(const char* name, double flops, double bytes, F&& launch, hipStream_t st = nullptr);
  void Gemm(const char* name, const half_t* A, int lda, const Linear& lin, void* C, int ldc, int M, int act,
            bool out_f32 = false, hipStream_t st = nullptr, int split_k = 1, bool latency_first = false,
            const NormFold* fold = nullptr, int out_stores = kStoresAuto);
  GemmArgs MakeGemmArgs(const half_t* A, int lda, const Linear& lin, void* C, int ldc, int M, int act, bool out_f32,
                        int split_k, bool latency_first, const NormFold* fold) const;
  // Kernels other than the dense layers, by the network's element type (and, for 16-bit types, by whether the tuned
  // kernel takes the shape).
  void LayerNorm(const half_t* x, const half_t* skip, half_t* y, const float* gamma, const float* beta, int rows, int C,
                 float alpha, float eps, hipStream_t st = nullptr, uint8_t* y_f8 = nullptr, float f8_mul = 1.0f,
                 bool through = false);
  void LayerNormRows(const half_t* x, half_t* y, const float* gamma, const float* beta, int rows, int C,
                     hipStream_t st);
  void Attention(const half_t* qkv, const half_t* bias, half_t* out, int B, int heads, int depth, hipStream_t st);
  void SmolgenChain(const EncoderDev& e, const half_t* x, int emb, int heads, int hc, int hs, int gen, half_t* sg1,
                    half_t* sg2, half_t* sg3, half_t* sbias, int B, hipStream_t st, bool latency_first);
  bool CanFoldLayerNorms(int B) const;

  // ---- per-lane state: streams, activations, recorded graphs ----
  hipStream_t stream_ = nullptr;
  hipStream_t side_stream_ = nullptr;  // smolgen chain, overlapped with the QKV projection
  std::vector<hipEvent_t> fork_events_, join_events_;
  hipEvent_t heads_fork_ = nullptr, heads_join_ = nullptr;   // value / moves-left heads beside the policy head
  DeviceArena arena_;
  std::mutex eval_mutex_;
  std::shared_ptr<SlotPool> pool_ = std::make_shared<SlotPool>();

  // Device activations (sized for max_batch_).
  uint64_t* d_masks_ = nullptr;
  float* d_values_ = nullptr;
  half_t *in0_ = nullptr, *x_ = nullptr, *t_ = nullptr, *qkv_ = nullptr, *att_ = nullptr, *ffn_ = nullptr;
  half_t *sg1_ = nullptr, *sg2_ = nullptr, *sg3_ = nullptr, *sbias_ = nullptr;
  float* sg2f_ = nullptr;  // split-K accumulator of smolgen dense1
  // Partial row sums of the two un-normalised sums of an encoder layer (folded layer norms): [rows][parts][2].
  float *ln_stats_a_ = nullptr, *ln_stats_b_ = nullptr;
  half_t *pol_e_ = nullptr, *pol_qk_ = nullptr, *head1_ = nullptr, *head2_ = nullptr;
  half_t *pe_qkv_ = nullptr, *pe_att_ = nullptr, *pe_t_ = nullptr, *pe_ffn_ = nullptr;   // policy encoder scratch
  half_t *pe_sg1_ = nullptr, *pe_sg2_ = nullptr, *pe_sg3_ = nullptr, *pe_sbias_ = nullptr;
  float *pol_logits_ = nullptr, *d_policy_ = nullptr, *d_wdl_ = nullptr, *d_mlh_ = nullptr;
  // Legal-move softmax: per-sample offsets, policy indices and probabilities.
  int* d_legal_off_ = nullptr;
  uint16_t* d_legal_ids_ = nullptr;
  float* d_legal_probs_ = nullptr;
  half_t *pre_in_ = nullptr, *pre_out_ = nullptr;
  bool calibrating_ = false;
  float* d_absmax_ = nullptr;   // [4 * layers + 1] calibration maxima (float bits, non-negative)
  uint8_t *xq_ = nullptr, *attq_ = nullptr, *ffnq_ = nullptr;
  uint8_t *sg1q_ = nullptr, *sg2q_ = nullptr, *sg3q_ = nullptr;   // e4m3 operands of the smolgen chain
  void *r_in_ = nullptr, *r_x_ = nullptr, *r_y_ = nullptr, *r_v_ = nullptr, *r_m_ = nullptr, *r_h1_ = nullptr,
       *r_h2_ = nullptr;

  // Lanes: further instances that share this network's weights and own their streams and
  // activations, so that computations of several search threads run concurrently on the GPU
  // (option lanes=N; precedent: multi_stream in src/neural/backends/cuda/network_cuda.cc:634-706).
  std::vector<std::unique_ptr<Mi355xNetwork>> extra_lanes_;
  std::mutex lane_mutex_;
  std::condition_variable lane_cv_;
  std::vector<Mi355xNetwork*> free_lanes_;
  int lane_count_ = 1;
  bool is_lane_ = false;
  Mi355xNetwork* AcquireLane(bool* others_busy);
  void ReleaseLane(Mi355xNetwork* lane);
  void AcquireAllLanes();
  void ReleaseAllLanes();
  void EvaluateOnLane(HostSlot* slot, int batch);
  void DrainStreams();
  void CreateStreams();
  void AllocActivations();

  // Captured device passes, one per batch size (option graphs=true): replaying a graph
  // costs one launch instead of several hundred, which is what bounds small batches.
  std::map<int, hipGraphExec_t> graphs_;   // key: 2 * batch + single_stream_
  // Set for a pass that starts while another lane is busy: it stays on its main stream (see Evaluate).
  bool single_stream_ = false;
  void DropGraphs();
  void LaunchEager(int batch);

  // Profiling.
  std::atomic<bool> profiling_{false};   // read without the lane's mutex when a computation picks its lane
  struct Pending { std::string name; hipEvent_t start, stop; double flops, bytes; };
  std::vector<Pending> pending_;
  std::vector<hipEvent_t> event_pool_;
  std::vector<KernelTime> profile_;
  hipEvent_t NewEvent();
  void CollectPending();
};

// ----------------------------------------------------------------- helpers --
hipEvent_t Mi355xNetwork::NewEvent() {
  if (!event_pool_.empty()) {
    hipEvent_t e = event_pool_.back();
    event_pool_.pop_back();
    return e;
  }
  hipEvent_t e;
  HIP_CHECK(hipEventCreate(&e));
  return e;
}

template <typename F>
void Mi355xNetwork::Timed(const char* name, double flops, double bytes, F&& launch, hipStream_t st) {
  if (!profiling_) {
    launch();
    return;
  }
  if (st == nullptr) st = stream_;
  Pending p{name, NewEvent(), NewEvent(), flops, bytes};
  HIP_CHECK(hipEventRecord(p.start, st));
  launch();
  HIP_CHECK(hipEventRecord(p.stop, st));
  pending_.push_back(p);
}

void Mi355xNetwork::CollectPending() {
  for (Pending& p : pending_) {
    float ms = 0.0f;
    HIP_CHECK(hipEventElapsedTime(&ms, p.start, p.stop));
    auto it = std::find_if(profile_.begin(), profile_.end(), [&](const KernelTime& k) { return k.name == p.name; });
    if (it == profile_.end()) {
      profile_.push_back(KernelTime{p.name, 0.0, 0, 0.0, 0.0});
      it = profile_.end() - 1;
    }
    it->ms += ms;
    it->launches += 1;
    it->flops += p.flops;
    it->bytes += p.bytes;
    event_pool_.push_back(p.start);
    event_pool_.push_back(p.stop);
  }
  pending_.clear();
}

std::vector<KernelTime> Mi355xNetwork::TakeProfile() {
  std::lock_guard<std::mutex> lock(eval_mutex_);
  std::vector<KernelTime> out;
  out.swap(profile_);
  return out;
}

Linear Mi355xNetwork::MakeLinear(const Vec& w, const Vec& b, int out, int in, int pad_to) {
  if (static_cast<size_t>(out) * in != w.size()) {
    throw Error("Weight tensor has " + std::to_string(w.size()) + " elements, expected " + std::to_string(out) +
                " x " + std::to_string(in) + ".");
  }
  if (!b.empty() && static_cast<int>(b.size()) != out) throw Error("Bias size does not match the layer width.");
  Linear l;
  l.out = out;
  l.in = in;
  l.ld = RoundUp(in, pad_to);   // zero padding: the reduction may run over ld
  std::vector<float> h(static_cast<size_t>(out) * l.ld, 0.0f);
  for (int o = 0; o < out; o++)
    for (int i = 0; i < in; i++) h[static_cast<size_t>(o) * l.ld + i] = w[static_cast<size_t>(o) * in + i];
  l.w = UploadElems(h);
  if (!b.empty()) l.b = arena_.Upload(b);
  return l;
}

half_t* Mi355xNetwork::UploadElems(const std::vector<float>& v) {
  if (dtype_ == Dtype::kFloat) return reinterpret_cast<half_t*>(arena_.Upload(v));
  std::vector<uint16_t> bits(v.size());
  for (size_t i = 0; i < v.size(); i++) {
    if (dtype_ == Dtype::kBf16) {   // round to nearest even on the upper 16 bits of the float
      uint32_t u;
      std::memcpy(&u, &v[i], 4);
      if ((u & 0x7fffffffu) > 0x7f800000u) {
        bits[i] = static_cast<uint16_t>((u >> 16) | 0x40);   // NaN stays NaN
      } else {
        bits[i] = static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
      }
    } else {
      const half_t h = (half_t)v[i];
      std::memcpy(&bits[i], &h, 2);
    }
  }
  return reinterpret_cast<half_t*>(arena_.Upload(bits));
}

// A layer that reads layer-normalised rows, prepared for reading the un-normalised rows instead (the consumer
// side of GemmArgs): weights w[o][i] * gamma[i], their row sums as stored (after rounding to half, so that the
// mean cancels exactly), and the bias plus sum_i beta[i] w[o][i].
Linear Mi355xNetwork::MakeLinearNormFolded(const Vec& w, const Vec& b, const Vec& gamma, const Vec& beta, int out,
                                           int in) {
  if (w.size() != static_cast<size_t>(out) * in || gamma.size() != static_cast<size_t>(in) ||
      beta.size() != static_cast<size_t>(in) || (!b.empty() && b.size() != static_cast<size_t>(out))) {
    throw Error("A dense layer has a wrong number of weights.");
  }
  Linear l;
  l.out = out; l.in = in;
  l.ld = RoundUp(in, 8);
  std::vector<half_t> h(static_cast<size_t>(out) * l.ld, (half_t)0.0f);
  std::vector<float> c(out), d(out);
  for (int o = 0; o < out; o++) {
    double csum = 0.0, dsum = b.empty() ? 0.0 : b[o];
    for (int i = 0; i < in; i++) {
      const double wv = w[static_cast<size_t>(o) * in + i];
      const half_t hv = (half_t)static_cast<float>(wv * gamma[i]);
      h[static_cast<size_t>(o) * l.ld + i] = hv;
      csum += static_cast<double>(static_cast<float>(hv));
      dsum += wv * beta[i];
    }
    c[o] = static_cast<float>(csum);
    d[o] = static_cast<float>(dsum);
  }
  l.w = arena_.Upload(h);
  l.b = arena_.Upload(d);
  l.c = arena_.Upload(c);
  return l;
}

GemmArgs Mi355xNetwork::MakeGemmArgs(const half_t* A, int lda, const Linear& lin, void* C, int ldc, int M, int act,
                                     bool out_f32, int split_k, bool latency_first, const NormFold* fold) const {
  GemmArgs g;
  g.latency_first = latency_first;
  g.split_k = split_k;
  g.split_stride = static_cast<long long>(M) * ldc;
  g.A = A; g.lda = lda;
  g.W = lin.w; g.ldw = lin.ld;
  g.C = C; g.ldc = ldc;
  g.bias = lin.b;
  g.M = M; g.N = lin.out; g.K = lin.ld;
  g.act = act;
  g.out_f32 = out_f32;
  if (fold != nullptr) {
    g.row_stats = fold->row_stats; g.row_parts = fold->row_parts; g.col_c = lin.c;
    g.skip = fold->skip; g.ldskip = fold->ldskip;
    g.skip_stats = fold->skip_stats; g.skip_parts = fold->skip_parts;
    g.skip_gamma = fold->skip_gamma; g.skip_beta = fold->skip_beta;
    g.stats_out = fold->stats_out;
    g.norm_n = fold->norm_n; g.norm_eps = fold->eps;
    g.scale = fold->scale;
    if (fold->bias != nullptr) g.bias = fold->bias;
  }
  return g;
}

void Mi355xNetwork::Gemm(const char* name, const half_t* A, int lda, const Linear& lin, void* C, int ldc, int M,
                         int act, bool out_f32, hipStream_t st, int split_k, bool latency_first,
                         const NormFold* fold, int out_stores) {
  if (st == nullptr) st = stream_;
  if (dtype_ == Dtype::kFloat) {
    if (split_k != 1 || fold != nullptr) throw Error("internal: split or folded GEMM requested in the float configuration");
    GemmArgsF32 g;
    g.A = reinterpret_cast<const float*>(A); g.lda = lda;
    g.W = reinterpret_cast<const float*>(lin.w); g.ldw = lin.ld;
    g.C = static_cast<float*>(C); g.ldc = ldc;
    g.bias = lin.b;
    g.M = M; g.N = lin.out; g.K = lin.ld;
    g.act = act;
    const std::string label = std::string(name) + "|gemm_f32_mfma_32x32x2";
    Timed(label.c_str(), 2.0 * M * lin.out * lin.in,
          4.0 * (static_cast<double>(M) * lin.in + static_cast<double>(lin.out) * lin.in + static_cast<double>(M) * lin.out),
          [&] { LaunchGemmF32(g, st); }, st);
    return;
  }
  GemmArgs g = MakeGemmArgs(A, lda, lin, C, ldc, M, act, out_f32, split_k, latency_first, fold);
  g.bf16 = dtype_ == Dtype::kBf16;
  g.out_stores = out_stores;
  if (fold != nullptr && fold->parts_out != nullptr) *fold->parts_out = GemmStatsParts(g);
  const double flops = 2.0 * M * lin.out * lin.in;
  const double bytes = 2.0 * (static_cast<double>(M) * lin.in + static_cast<double>(lin.out) * lin.in) +
                       static_cast<double>(M) * lin.out * (out_f32 ? 4 : 2) +
                       (fold != nullptr && fold->skip != nullptr ? 2.0 * M * lin.out : 0.0);
  std::string label = std::string(name) + "|" + GemmVariantName(g);
  if (fold != nullptr) label += fold->skip != nullptr ? "+skip_stats" : "+row_norm";
  Timed(label.c_str(), flops, bytes, [&] { LaunchGemm(g, st); }, st);
}

void Mi355xNetwork::LayerNorm(const half_t* x, const half_t* skip, half_t* y, const float* gamma, const float* beta,
                              int rows, int C, float alpha, float eps, hipStream_t st, uint8_t* y_f8, float f8_mul,
                              bool through) {
  if (st == nullptr) st = stream_;
  if (dtype_ == Dtype::kFloat) {
    LaunchLayerNormGeneric<float>(reinterpret_cast<const float*>(x), reinterpret_cast<const float*>(skip),
                                  reinterpret_cast<float*>(y), gamma, beta, rows, C, alpha, eps, kActNone, st);
  } else {
    LaunchLayerNorm(x, skip, y, gamma, beta, rows, C, alpha, eps, st, y_f8, f8_mul, dtype_ == Dtype::kBf16, through);
  }
}

// Layer norm of few, long rows (the two norms of the smolgen chain).
void Mi355xNetwork::LayerNormRows(const half_t* x, half_t* y, const float* gamma, const float* beta, int rows, int C,
                                  hipStream_t st) {
  if (dtype_ == Dtype::kFloat) {
    LaunchLayerNormGeneric<float>(reinterpret_cast<const float*>(x), nullptr, reinterpret_cast<float*>(y), gamma, beta,
                                  rows, C, 1.0f, 1e-3f, kActNone, st);
  } else {
    LaunchLayerNormRows(nullptr, 0, 0, x, kActNone, nullptr, y, gamma, beta, rows, C, 1.0f, 1e-3f, st,
                        dtype_ == Dtype::kBf16);
  }
}

// Per-head attention: the matrix-core kernel for 16-bit elements and head depth 32, 64 or 128, the general one else.
void Mi355xNetwork::Attention(const half_t* qkv, const half_t* bias, half_t* out, int B, int heads, int depth,
                              hipStream_t st) {
  const float scale = 1.0f / std::sqrt(static_cast<float>(depth));
  if (dtype_ == Dtype::kFloat) {
    LaunchAttentionGeneric<float>(reinterpret_cast<const float*>(qkv), reinterpret_cast<const float*>(bias),
                                  reinterpret_cast<float*>(out), B, heads, depth, scale, st);
  } else if (AttentionDepthSupported(depth)) {
    LaunchAttention(qkv, bias, out, B, heads, scale, st, depth, dtype_ == Dtype::kBf16);
  } else if (dtype_ == Dtype::kBf16) {
    LaunchAttentionGeneric<bf16_t>(reinterpret_cast<const bf16_t*>(qkv), reinterpret_cast<const bf16_t*>(bias),
                                   reinterpret_cast<bf16_t*>(out), B, heads, depth, scale, st);
  } else {
    LaunchAttentionGeneric<half_t>(qkv, bias, out, B, heads, depth, scale, st);
  }
}

// The smolgen chain of one encoder layer, unfused (network_blas.cc:283-347): compression, two dense layers with
// their row norms, then the shared generator layer, which leaves the logits in sbias (SmolgenBiasIndex order).
void Mi355xNetwork::SmolgenChain(const EncoderDev& e, const half_t* x, int emb, int heads, int hc, int hs, int gen,
                                 half_t* sg1, half_t* sg2, half_t* sg3, half_t* sbias, int B, hipStream_t st,
                                 bool latency_first) {
  const int T = B * 64;
  Gemm("gemm_smolgen_compress", x, emb, e.sg_compress, sg1, hc, T, kActNone, false, st, 1, latency_first);
  Gemm("gemm_smolgen_dense1", sg1, 64 * hc, e.sg_dense1, sg2, hs, B, smolgen_act_, false, st, 1, latency_first);
  Timed("layer_norm_rows", 0.0, 2.0 * es_ * B * hs, [&] { LayerNormRows(sg2, sg2, e.sg_ln1_g, e.sg_ln1_b, B, hs, st); }, st);
  Gemm("gemm_smolgen_dense2", sg2, hs, e.sg_dense2, sg3, gen, B, smolgen_act_, false, st, 1, latency_first);
  Timed("layer_norm_rows", 0.0, 2.0 * es_ * B * gen, [&] { LayerNormRows(sg3, sg3, e.sg_ln2_g, e.sg_ln2_b, B, gen, st); }, st);
  Gemm("gemm_smolgen_global", sg3, gen / heads, smolgen_w_, sbias, 4096, B * heads, kActNone, false, st, 1, latency_first);
}

// Whether a pass over B positions can run the encoder stack with its layer norms folded into the GEMMs around
// them: every one of the five launches per layer must get a kernel variant that has the epilogue.
bool Mi355xNetwork::CanFoldLayerNorms(int B) const {
  if (!fold_layer_norm_ || encoders_.empty() || encoders_[0].ffn1_n.w == nullptr) return false;
  const int T = B * 64;
  const half_t* any_h = x_;
  const float* any_f = ln_stats_a_;
  const EncoderDev& e = encoders_.back();
  NormFold cons;
  cons.row_stats = any_f; cons.row_parts = 1; cons.norm_n = emb_;
  NormFold prod;
  prod.skip = any_h; prod.ldskip = emb_; prod.stats_out = ln_stats_a_; prod.norm_n = emb_;
  const bool chain_first = B <= chain_latency_max_batch_;
  if (!GemmSupportsNormFolding(MakeGemmArgs(x_, emb_, e.qkv_n, qkv_, 3 * d_model_, T, kActNone, false, 1, false, &cons)) ||
      !GemmSupportsNormFolding(MakeGemmArgs(x_, emb_, e.ffn1_n, ffn_, dff_, T, ffn_act_, false, 1, false, &cons)) ||
      !GemmSupportsNormFolding(MakeGemmArgs(att_, d_model_, e.dense, x_, emb_, T, kActNone, false, 1, false, &prod)) ||
      !GemmSupportsNormFolding(MakeGemmArgs(ffn_, dff_, e.ffn2, x_, emb_, T, kActNone, false, 1, false, &prod))) {
    return false;
  }
  if (e.has_smolgen &&
      !GemmSupportsNormFolding(
          MakeGemmArgs(x_, emb_, e.sg_compress_n, sg1_, sg_hc_, T, kActNone, false, 1, chain_first, &cons))) {
    return false;
  }
  return true;
}

// ------------------------------------------------------------------- fp8 --
namespace {
// float -> e4m3 code: round to nearest even, saturating at +-448 (the rule of
// FP32toFP8E4M3FN, src/utils/fp8_utils.h:111-138).
uint8_t EncodeE4M3(float v) {
  const uint8_t sign = std::signbit(v) ? 0x80 : 0;
  float a = std::fabs(v);
  if (std::isnan(a)) return 0x7f;
  if (a >= 448.0f) return sign | 0x7e;
  int ex;
  std::frexp(a, &ex);               // a = f * 2^ex, f in [0.5, 1)
  ex = std::max(ex - 1, -6);        // binade of a; subnormals share the spacing of the first one
  const float step = std::ldexp(1.0f, ex - 3);
  const float q = std::nearbyint(a / step);   // default rounding mode: ties to even
  const float mag = q * step;
  if (mag < std::ldexp(1.0f, -6)) return sign | static_cast<uint8_t>(q);
  int e2;
  const float f = std::frexp(mag, &e2);       // mag = f * 2^e2
  const int mant = static_cast<int>((f * 2.0f - 1.0f) * 8.0f);
  return sign | static_cast<uint8_t>(((e2 - 1 + 7) << 3) | mant);
}
}  // namespace

LinearF8 Mi355xNetwork::MakeLinearF8(const Vec& w, int out, int in) {
  if (static_cast<size_t>(out) * in != w.size()) throw Error("Weight tensor has an unexpected size.");
  LinearF8 q;
  q.wscale.resize(out);
  std::vector<uint8_t> codes(w.size());
  for (int o = 0; o < out; o++) {
    const float* row = &w[static_cast<size_t>(o) * in];
    float amax = 0.0f;
    for (int i = 0; i < in; i++) amax = std::max(amax, std::fabs(row[i]));
    const float scale = amax > 0.0f ? amax / 448.0f : 1.0f;
    q.wscale[o] = scale;
    for (int i = 0; i < in; i++) codes[static_cast<size_t>(o) * in + i] = EncodeE4M3(row[i] / scale);
  }
  q.w = arena_.Upload(codes);
  q.col_scale = AllocF(out);
  return q;
}

void Mi355xNetwork::GemmF8(const char* name, const uint8_t* A, const Linear& lin, const LinearF8& q, void* C, int M,
                           int act, bool out_f8, float out_mul, hipStream_t st, int out_stores) {
  if (st == nullptr) st = stream_;
  GemmF8Args g;
  g.A = A; g.lda = lin.in;
  g.W = q.w; g.ldw = lin.in;
  g.C = C; g.ldc = lin.out;
  g.col_scale = q.col_scale;
  g.bias = lin.b;
  g.M = M; g.N = lin.out; g.K = lin.in;
  g.act = act;
  g.out_f8 = out_f8;
  g.out_mul = out_mul;
  g.out_stores = out_stores;
  const double flops = 2.0 * M * lin.out * lin.in;
  const double bytes = static_cast<double>(M) * lin.in + static_cast<double>(lin.out) * lin.in +
                       static_cast<double>(M) * lin.out * (out_f8 ? 1 : 2);
  const std::string label = std::string(name) + "|" + GemmF8VariantName(g);
  Timed(label.c_str(), flops, bytes, [&] { LaunchGemmF8(g, st); }, st);
}

void Mi355xNetwork::RecordAbsMax(const half_t* x, size_t n, int slot, hipStream_t st) {
  LaunchAbsMax(x, static_cast<long long>(n), d_absmax_ + slot, st == nullptr ? stream_ : st);
}

// Activation scales from the maxima seen during calibration: the largest value maps to
// 224, half of the e4m3 range (headroom for unseen positions costs no precision in a
// floating-point format; anything beyond saturates).
void Mi355xNetwork::ApplyCalibration(const std::vector<float>& absmax) {
  auto scale_of = [](float amax) { return amax > 0.0f ? amax / 224.0f : 1.0f; };
  auto upload = [&](LinearF8& q, float s_act) {
    std::vector<float> cs(q.wscale.size());
    for (size_t i = 0; i < cs.size(); i++) cs[i] = s_act * q.wscale[i];
    HIP_CHECK(hipMemcpy(q.col_scale, cs.data(), cs.size() * sizeof(float), hipMemcpyHostToDevice));
  };
  for (size_t li = 0; li < encoders_.size(); li++) {
    EncoderDev& e = encoders_[li];
    e.s_x = scale_of(absmax[4 * li + 0]);
    e.s_att = scale_of(absmax[4 * li + 1]);
    e.s_x1 = scale_of(absmax[4 * li + 2]);
    e.s_ffn = scale_of(absmax[4 * li + 3]);
    upload(e.qkv8, e.s_x);
    upload(e.dense8, e.s_att);
    upload(e.ffn18, e.s_x1);
    upload(e.ffn28, e.s_ffn);
    if (q_smolgen_ && e.has_smolgen) {
      e.s_sg1 = scale_of(absmax[SmolgenSlot(li, 0)]);
      e.s_sg2 = scale_of(absmax[SmolgenSlot(li, 1)]);
      e.s_sg3 = scale_of(absmax[SmolgenSlot(li, 2)]);
      upload(e.sg_compress8, e.s_x);
      upload(e.sg_dense18, e.s_sg1);
      upload(e.sg_dense28, e.s_sg2);
      upload(e.sg_global8, e.s_sg3);
    }
  }
}

// Per layer: the scales of x, attention output, x1, FFN hidden, and of the three smolgen operands (1 when unused).
std::vector<float> Mi355xNetwork::Fp8Scales() const {
  if (!fp8_) throw Error("Fp8Scales needs a network created with precision=fp8.");
  std::vector<float> out;
  for (const EncoderDev& e : encoders_) {
    for (float v : {e.s_x, e.s_att, e.s_x1, e.s_ffn, e.s_sg1, e.s_sg2, e.s_sg3}) out.push_back(v);
  }
  return out;
}

void Mi355xNetwork::CalibrateFp8(int n, const uint64_t* masks, const float* values) {
  if (!fp8_) throw Error("CalibrateFp8 needs a network created with precision=fp8.");
  if (n < 1 || !masks || !values) throw Error("CalibrateFp8 needs at least one position.");
  AcquireAllLanes();
  try {
    CalibrateExclusive(n, masks, values);
  } catch (...) {
    ReleaseAllLanes();
    throw;
  }
  ReleaseAllLanes();
}

// Caller guarantees that no computation is in flight on any lane.
void Mi355xNetwork::CalibrateExclusive(int n, const uint64_t* masks, const float* values) {
  std::lock_guard<std::mutex> lock(eval_mutex_);
  HIP_CHECK(hipSetDevice(device_));
  const size_t slots = CalibrationSlots();
  std::vector<float> absmax(slots, 0.0f), part(slots);
  for (int done = 0; done < n; done += max_batch_) {
    const int b = std::min(max_batch_, n - done);
    HIP_CHECK(hipMemcpy(d_masks_, masks + static_cast<size_t>(done) * kInputPlanes, sizeof(uint64_t) * kInputPlanes * b,
                        hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(d_values_, values + static_cast<size_t>(done) * kInputPlanes, sizeof(float) * kInputPlanes * b,
                        hipMemcpyHostToDevice));
    LaunchZero(d_absmax_, static_cast<long long>(slots), stream_);
    calibrating_ = true;
    const bool was_profiling = profiling_.load();
    profiling_ = false;
    try {
      ForwardAttentionBody(b);   // fp16 pass that records the maxima
    } catch (...) {
      calibrating_ = false;
      profiling_ = was_profiling;
      throw;
    }
    calibrating_ = false;
    profiling_ = was_profiling;
    HIP_CHECK(hipStreamSynchronize(stream_));
    HIP_CHECK(hipStreamSynchronize(side_stream_));
    HIP_CHECK(hipMemcpy(part.data(), d_absmax_, slots * sizeof(float), hipMemcpyDeviceToHost));
    for (size_t i = 0; i < slots; i++) absmax[i] = std::max(absmax[i], part[i]);
  }
  ApplyCalibration(absmax);
  DropGraphs();   // recorded kernel arguments hold the old scales
  for (auto& lane : extra_lanes_) {
    static_cast<ModelState&>(*lane) = static_cast<const ModelState&>(*this);
    lane->DropGraphs();
  }
}

// Built-in calibration set used at load, so that precision=fp8 works without any caller
// support: 64 seeded pseudo-positions (two kings, a random subset of other pieces, eight
// history steps that differ by one moved piece, plausible auxiliary planes). Callers that
// own real positions replace it through CalibrateFp8.
void Mi355xNetwork::DefaultCalibration() {
  const int n = std::min(64, max_batch_);
  std::vector<uint64_t> masks(static_cast<size_t>(n) * kInputPlanes, 0);
  std::vector<float> values(static_cast<size_t>(n) * kInputPlanes, 1.0f);
  uint64_t state = 0x9e3779b97f4a7c15ULL;
  auto next = [&state]() {   // splitmix64
    uint64_t z = (state += 0x9e3779b97f4a7c15ULL);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
  };
  for (int p = 0; p < n; p++) {
    uint64_t* m = &masks[static_cast<size_t>(p) * kInputPlanes];
    float* v = &values[static_cast<size_t>(p) * kInputPlanes];
    // piece planes of the newest history step: 0-5 ours (P N B R Q K), 6-11 theirs
    int square_of[32], plane_of[32], count = 0;
    uint64_t used = 0;
    auto place = [&](int plane, int lo_rank, int hi_rank) {
      for (int tries = 0; tries < 64; tries++) {
        const int sq = static_cast<int>(next() % 64);
        if (sq / 8 < lo_rank || sq / 8 > hi_rank || (used >> sq) & 1) continue;
        used |= 1ULL << sq;
        square_of[count] = sq; plane_of[count] = plane; count++;
        return;
      }
    };
    place(5, 0, 7); place(11, 0, 7);
    static const int kMaxCount[5] = {8, 2, 2, 2, 1};
    for (int side = 0; side < 2; side++)
      for (int piece = 0; piece < 5; piece++) {
        const int k = static_cast<int>(next() % (kMaxCount[piece] + 1));
        for (int i = 0; i < k; i++) place(side * 6 + piece, piece == 0 ? 1 : 0, piece == 0 ? 6 : 7);
      }
    const int history = 1 + static_cast<int>(next() % 8);
    for (int h = 0; h < history; h++) {
      for (int i = 0; i < count; i++) m[h * 13 + plane_of[i]] |= 1ULL << square_of[i];
      if (next() % 16 == 0) m[h * 13 + 12] = ~0ULL;   // repetition marker
      // step back in time: move one piece to a free square
      const int i = static_cast<int>(next() % count);
      for (int tries = 0; tries < 64; tries++) {
        const int sq = static_cast<int>(next() % 64);
        if ((used >> sq) & 1) continue;
        used &= ~(1ULL << square_of[i]);
        used |= 1ULL << sq;
        square_of[i] = sq;
        break;
      }
    }
    for (int c = 104; c < 108; c++) m[c] = (next() & 1) ? ~0ULL : 0;   // castling rights
    m[108] = (next() & 1) ? ~0ULL : 0;                                  // side to move
    m[109] = ~0ULL; v[109] = static_cast<float>(next() % 100);          // rule-50 counter
    m[110] = 0;
    m[111] = ~0ULL;                                                     // all ones
  }
  CalibrateExclusive(n, masks.data(), values.data());
}

// ------------------------------------------------------------- construction --
Mi355xNetwork::Mi355xNetwork(const WeightsFile& file, Options& options) {
  const NetworkFormat& nf = file.format;
  caps_.input_format = nf.input;
  caps_.output_format = nf.output;
  caps_.moves_left = nf.moves_left;

  device_ = options.GetInt("gpu", 0);
  max_batch_ = options.GetInt("max_batch", 1024);
  if (max_batch_ < 1 || max_batch_ > 4096) throw Error("max_batch must be in 1..4096.");
  const std::string precision = options.GetString("precision", "fp16");
  if (precision != "fp16" && precision != "fp32" && precision != "fp8" && precision != "bf16") {
    throw Error("Precision '" + precision + "' is not supported (fp16, bf16, fp32 or fp8).");
  }
  fp32_ = precision == "fp32";
  fp8_ = precision == "fp8";
  dtype_ = fp32_ ? Dtype::kFloat : precision == "bf16" ? Dtype::kBf16 : Dtype::kHalf;
  es_ = fp32_ ? 4 : 2;
  {
    // Which layers of an encoder use e4m3 operands: names joined by '+'. The default, "auto", takes the four large
    // GEMMs and the smolgen chain where the chain's widths allow it (multiples of 128: the e4m3 k-tile).
    std::string which = options.GetString("fp8_gemms", "auto");
    q_qkv_ = q_dense_ = q_ffn1_ = q_ffn2_ = q_smolgen_ = false;
    if (which == "auto") {
      which = "qkv+dense+ffn1+ffn2";
      q_smolgen_auto_ = true;
    }
    size_t pos = 0;
    while (pos <= which.size()) {
      const size_t end = std::min(which.find('+', pos), which.size());
      const std::string name = which.substr(pos, end - pos);
      if (name == "qkv") q_qkv_ = true;
      else if (name == "dense") q_dense_ = true;
      else if (name == "ffn1") q_ffn1_ = true;
      else if (name == "ffn2") q_ffn2_ = true;
      else if (name == "smolgen") q_smolgen_ = true;
      else if (!name.empty()) throw Error("Unknown name '" + name + "' in fp8_gemms (qkv, dense, ffn1, ffn2, smolgen).");
      pos = end + 1;
    }
  }
  fold_layer_norm_ = options.GetBool("fold_layer_norm", false);
  // The generator layer of smolgen inside the attention kernel: ahead from 128 positions up (one workgroup serves two
  // samples and a quarter of the queries, and its two phases do not overlap: at fewer positions than fill the CUs the
  // separate GEMM and attention kernels are faster; 15x1024 net: batch 128 +4 %, 256 +1.5 %, 1024 +2 %, 64 -1 %, 16 -6 %).
  fused_smolgen_attention_ = options.GetBool("fused_smolgen_attention", true);
  fused_smolgen_min_batch_ = options.GetInt("fused_smolgen_min_batch", 72);
  dense1_split_min_batch_ = options.GetInt("dense1_split_min_batch", 112);
  qkv_first_ = options.GetBool("qkv_first", true);
  write_through_ = options.GetBool("write_through", true);
  chain_latency_max_batch_ = options.GetInt("chain_latency_max_batch", 128);
  fp8_fp16_layers_ = options.GetInt("fp8_fp16_layers", 0);
  if (fp8_fp16_layers_ < 0) throw Error("fp8_fp16_layers must not be negative.");
  use_graphs_ = options.GetBool("graphs", true);
  // Running the smolgen chain beside the QKV projection costs two cross-queue dependencies per layer; below
  // this batch size the chain on the main stream is faster (measured on the 15x1024 net, chain on the main stream
  // against beside the projection: fp16 batch 8 1.26 against 1.45 ms, batch 64 2.50 against 2.53, batch 96 3.43
  // against 3.24; fp8 batch 64 2.00 against 2.25, batch 96 2.60 against 2.54).
  overlap_min_batch_ = options.GetInt("overlap_min_batch", -1);
  if (overlap_min_batch_ < 0) overlap_min_batch_ = 80;
  heads_overlap_min_batch_ = options.GetInt("heads_overlap_min_batch", -1);
  lane_count_ = options.GetInt("lanes", 4);
  if (lane_count_ < 1 || lane_count_ > 8) throw Error("lanes must be in 1..8.");
  policy_head_ = options.GetString("policy_head", "vanilla");
  value_head_ = options.GetString("value_head", "winner");
  wdl_ = nf.value == kValueWdl;
  moves_left_ = nf.moves_left == kMovesLeftV1 && options.GetBool("mlh", true);
  conv_policy_ = nf.policy == kPolicyConvolution;
  attn_policy_ = nf.policy == kPolicyAttention;
  attn_body_ = nf.network == kNetworkAttentionBodyWithHeadformat ||
               nf.network == kNetworkAttentionBodyWithMultiheadformat;
  default_act_ = nf.default_activation == 1 ? kActMish : kActRelu;
  if (attn_body_) {
    smolgen_act_ = nf.smolgen_activation == kActDefault ? default_act_ : nf.smolgen_activation;
    ffn_act_ = nf.ffn_activation == kActDefault ? default_act_ : nf.ffn_activation;
  }
  if (file.weights.policy_heads.count(policy_head_) == 0) {
    throw Error("The policy head you specified '" + policy_head_ + "' does not exist in this net.");
  }
  if (file.weights.value_heads.count(value_head_) == 0) {
    throw Error("The value head you specified '" + value_head_ + "' does not exist in this net.");
  }

  int count = 0;
  hipError_t err = hipGetDeviceCount(&count);
  if (err != hipSuccess || count == 0) {
    throw Error("No HIP device is available: the mi355x backend needs a GPU (there is no CPU fallback).");
  }
  if (device_ < 0 || device_ >= count) throw Error("Invalid GPU id " + std::to_string(device_) + ".");
  CreateStreams();
  if (attn_body_) {
    BuildAttentionBody(file);
  } else if (fp8_) {
    throw Error("precision=fp8 is available for attention-body networks only.");
  } else if (dtype_ == Dtype::kBf16) {
    throw Error("precision=bf16 is available for attention-body networks only.");
  } else if (fp32_) {
    BuildResnet<float>(file);
  } else {
    BuildResnet<half_t>(file);
  }
  AllocActivations();
  if (fp8_) DefaultCalibration();
  HIP_CHECK(hipStreamSynchronize(stream_));
  for (int i = 1; i < lane_count_; i++) extra_lanes_.push_back(std::make_unique<Mi355xNetwork>(*this, LaneTag{}));
  ReleaseAllLanes();
}

Mi355xNetwork::Mi355xNetwork(const Mi355xNetwork& parent, LaneTag) : ModelState(parent) {
  pool_ = parent.pool_;
  is_lane_ = true;
  CreateStreams();
  AllocActivations();
}

Mi355xNetwork::~Mi355xNetwork() {
  if (!is_lane_) {   // the network that owns weights and lanes
    extra_lanes_.clear();
    std::lock_guard<std::mutex> lock(pool_->mutex);
    pool_->network_alive = false;
    pool_->free_slots.clear();
  }
  if (stream_) {
    (void)hipStreamSynchronize(stream_);
    DropGraphs();
    for (hipEvent_t e : event_pool_) (void)hipEventDestroy(e);
    for (hipEvent_t e : fork_events_) (void)hipEventDestroy(e);
    for (hipEvent_t e : join_events_) (void)hipEventDestroy(e);
    if (heads_fork_) (void)hipEventDestroy(heads_fork_);
    if (heads_join_) (void)hipEventDestroy(heads_join_);
    if (side_stream_) {
      (void)hipStreamSynchronize(side_stream_);
      (void)hipStreamDestroy(side_stream_);
    }
    (void)hipStreamDestroy(stream_);
  }
}

// Streams and events of one lane.
void Mi355xNetwork::CreateStreams() {
  HIP_CHECK(hipSetDevice(device_));
  HIP_CHECK(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking));
  HIP_CHECK(hipStreamCreateWithFlags(&side_stream_, hipStreamNonBlocking));
  HIP_CHECK(hipEventCreateWithFlags(&heads_fork_, hipEventDisableTiming));
  HIP_CHECK(hipEventCreateWithFlags(&heads_join_, hipEventDisableTiming));
}

// Device buffers of one lane (inputs, activations, outputs), sized for max_batch_.
void Mi355xNetwork::AllocActivations() {
  d_masks_ = static_cast<uint64_t*>(arena_.Alloc(sizeof(uint64_t) * kInputPlanes * max_batch_));
  d_values_ = AllocF(static_cast<size_t>(kInputPlanes) * max_batch_);
  d_policy_ = AllocF(static_cast<size_t>(kPolicyOutputs) * max_batch_);
  d_wdl_ = AllocF(3 * static_cast<size_t>(max_batch_));
  d_mlh_ = AllocF(max_batch_);
  d_legal_off_ = static_cast<int*>(arena_.Alloc(sizeof(int) * (static_cast<size_t>(max_batch_) + 1)));
  d_legal_ids_ = static_cast<uint16_t*>(arena_.Alloc(sizeof(uint16_t) * kMaxLegalMoves * max_batch_));
  d_legal_probs_ = AllocF(static_cast<size_t>(kMaxLegalMoves) * max_batch_);
  if (attn_policy_) {
    const size_t T = static_cast<size_t>(max_batch_) * 64;
    pol_e_ = AllocH(T * pol_emb_);
    pol_qk_ = AllocH(T * 2 * pol_d_);
    pol_logits_ = AllocF(static_cast<size_t>(max_batch_) * 4096);
    if (!pol_encoders_.empty()) {
      pe_qkv_ = AllocH(T * 3 * pe_dmodel_);
      pe_att_ = AllocH(T * pe_dmodel_);
      pe_t_ = AllocH(T * pol_emb_);
      pe_ffn_ = AllocH(T * pe_dff_);
      if (pe_smolgen_) {
        pe_sg1_ = AllocH(T * pe_sg_hc_);
        pe_sg2_ = AllocH(static_cast<size_t>(max_batch_) * pe_sg_hs_);
        pe_sg3_ = AllocH(static_cast<size_t>(max_batch_) * pe_sg_gen_);
        pe_sbias_ = AllocH(static_cast<size_t>(max_batch_) * pe_heads_ * 4096);
      }
    }
  }
  if (!attn_body_) {
    const size_t ts = fp32_ ? sizeof(float) : sizeof(half_t);
    const size_t B = static_cast<size_t>(max_batch_);
    const size_t cmax = res_cmax_;
    r_in_ = arena_.Alloc(ts * B * 64 * kInputPlanes);
    r_x_ = arena_.Alloc(ts * B * 64 * cmax);
    r_y_ = arena_.Alloc(ts * B * 64 * cmax);
    r_v_ = arena_.Alloc(ts * 36 * B * 4 * std::max<size_t>(filters_, RoundUp(kInputPlanes, 64)));
    r_m_ = arena_.Alloc(ts * 36 * B * 4 * cmax);
    r_h1_ = arena_.Alloc(ts * B * 64 * cmax);
    r_h2_ = arena_.Alloc(ts * B * res_max_fc_);
    return;
  }
  const size_t T = static_cast<size_t>(max_batch_) * 64;
  in0_ = AllocH(T * in_ld_);
  x_ = AllocH(T * emb_);
  t_ = AllocH(T * emb_);
  qkv_ = AllocH(T * 3 * d_model_);
  att_ = AllocH(T * d_model_);
  ffn_ = AllocH(T * std::max(dff_, emb_dff_));
  if (pe_dense_) {
    pre_in_ = AllocH(static_cast<size_t>(max_batch_) * 768);
    pre_out_ = AllocH(T * enc_ch_);
  }
  if (!encoders_.empty() && encoders_[0].ffn1_n.w != nullptr) {
    // at most one part per 64 columns (the narrowest column tile of the GEMM variants that write them)
    const size_t n = T * static_cast<size_t>((emb_ + 63) / 64) * 2;
    ln_stats_a_ = AllocF(n);
    ln_stats_b_ = AllocF(n);
  }
  if (any_smolgen_) {
    sg1_ = AllocH(T * sg_hc_);
    sg2_ = AllocH(static_cast<size_t>(max_batch_) * sg_hs_);
    sg2f_ = AllocF(static_cast<size_t>(max_batch_) * sg_hs_ * 16);  // up to 16 split-K slices
    for (size_t i = 0; i < encoders_.size(); i++) {
      hipEvent_t a, b;
      HIP_CHECK(hipEventCreateWithFlags(&a, hipEventDisableTiming));
      HIP_CHECK(hipEventCreateWithFlags(&b, hipEventDisableTiming));
      fork_events_.push_back(a);
      join_events_.push_back(b);
    }
    sg3_ = AllocH(static_cast<size_t>(max_batch_) * sg_gen_);
    sbias_ = AllocH(static_cast<size_t>(max_batch_) * heads_ * 4096);
  }
  if (fp8_) {
    xq_ = static_cast<uint8_t*>(arena_.Alloc(T * emb_));
    attq_ = static_cast<uint8_t*>(arena_.Alloc(T * d_model_));
    ffnq_ = static_cast<uint8_t*>(arena_.Alloc(T * dff_));
    d_absmax_ = AllocF(CalibrationSlots());
    if (q_smolgen_ && any_smolgen_) {
      sg1q_ = static_cast<uint8_t*>(arena_.Alloc(T * sg_hc_));
      sg2q_ = static_cast<uint8_t*>(arena_.Alloc(static_cast<size_t>(max_batch_) * sg_hs_));
      sg3q_ = static_cast<uint8_t*>(arena_.Alloc(static_cast<size_t>(max_batch_) * sg_gen_));
    }
  }
  head1_ = AllocH(T * std::max(val_ch_, mov_ch_));
  head2_ = AllocH(static_cast<size_t>(max_batch_) * std::max(val_fc_, mov_fc_));
}

// Weights of one post-LN encoder layer without smolgen (q, k and v stacked into one matrix).
EncoderDev Mi355xNetwork::MakeEncoderLayer(const EncoderLayer& l, int emb, int d_model, int dff) {
  EncoderDev e;
  if (static_cast<int>(l.mha.q_b.size()) != d_model || static_cast<int>(l.ffn.dense1_b.size()) != dff) {
    throw Error("Encoder layers of different sizes are not supported.");
  }
  Vec qkv_w, qkv_b;
  qkv_w.reserve(3 * l.mha.q_w.size());
  for (const Vec* v : {&l.mha.q_w, &l.mha.k_w, &l.mha.v_w}) qkv_w.insert(qkv_w.end(), v->begin(), v->end());
  for (const Vec* v : {&l.mha.q_b, &l.mha.k_b, &l.mha.v_b}) qkv_b.insert(qkv_b.end(), v->begin(), v->end());
  e.qkv = MakeLinear(qkv_w, qkv_b, 3 * d_model, emb);
  e.dense = MakeLinear(l.mha.dense_w, l.mha.dense_b, emb, d_model);
  e.ffn1 = MakeLinear(l.ffn.dense1_w, l.ffn.dense1_b, dff, emb);
  e.ffn2 = MakeLinear(l.ffn.dense2_w, l.ffn.dense2_b, emb, dff);
  e.ln1_g = UploadN(l.ln1_gammas, emb, "Encoder layer norm gamma"); e.ln1_b = UploadN(l.ln1_betas, emb, "Encoder layer norm beta");
  e.ln2_g = UploadN(l.ln2_gammas, emb, "Encoder layer norm gamma"); e.ln2_b = UploadN(l.ln2_betas, emb, "Encoder layer norm beta");
  return e;
}

void Mi355xNetwork::LoadSmolgen(const Smolgen& s, int emb, int heads, EncoderDev* e, int* hc_io, int* hs_io, int* gen_io,
                                bool* any) {
  const int hc = static_cast<int>(s.compress.size()) / emb;
  const int hs = static_cast<int>(s.dense1_b.size());
  const int gen = static_cast<int>(s.dense2_b.size());
  if (!*any) {
    *hc_io = hc; *hs_io = hs; *gen_io = gen;
  } else if (hc != *hc_io || hs != *hs_io || gen != *gen_io) {
    throw Error("Smolgen layers of different sizes are not supported.");
  }
  *any = true;
  if (hc <= 0 || hc % 8 || hs <= 0 || hs % 8 || gen % heads || (gen / heads) % 8 || hs > 8192 || gen > 8192) {
    throw Error("Unsupported smolgen sizes.");
  }
  e->has_smolgen = true;
  e->sg_compress = MakeLinear(s.compress, Vec(), hc, emb);
  e->sg_dense1 = MakeLinear(s.dense1_w, s.dense1_b, hs, 64 * hc);
  e->sg_dense2 = MakeLinear(s.dense2_w, s.dense2_b, gen, hs);
  e->sg_ln1_g = UploadN(s.ln1_gammas, hs, "Smolgen layer norm gamma"); e->sg_ln1_b = UploadN(s.ln1_betas, hs, "Smolgen layer norm beta");
  e->sg_ln2_g = UploadN(s.ln2_gammas, gen, "Smolgen layer norm gamma"); e->sg_ln2_b = UploadN(s.ln2_betas, gen, "Smolgen layer norm beta");
}

void Mi355xNetwork::EnsureSmolgenGlobal(const NetWeights& w, int g) {
  if (w.smolgen_w.size() != static_cast<size_t>(4096) * g) throw Error("Global smolgen weights have a wrong size.");
  if (smolgen_w_.w != nullptr) return;
  // Rows permuted so that the generated logits come out in the layout the
  // attention kernel reads with one 16-byte load per lane.
  Vec perm(w.smolgen_w.size());
  for (int q = 0; q < 64; q++)
    for (int k = 0; k < 64; k++)
      std::memcpy(&perm[static_cast<size_t>(SmolgenBiasIndex(q, k)) * g], &w.smolgen_w[static_cast<size_t>(q * 64 + k) * g],
                  sizeof(float) * g);
  smolgen_w_ = MakeLinear(perm, Vec(), 4096, g);
  if (fp8_ && q_smolgen_) {
    // One set of codes for all layers; every layer brings the scale of its own operand.
    LinearF8 shared = MakeLinearF8(perm, 4096, g);
    smolgen_w8_ = shared.w;
    smolgen_w8_scale_ = shared.wscale;
  }
}

// Attention policy head (network_blas.cc:806-914) on token-major input of in_channels channels.
void Mi355xNetwork::BuildAttentionPolicy(const NetWeights& w, const PolicyHead& ph, int in_channels) {
  pol_emb_ = static_cast<int>(ph.ip_pol_b.size());
  pol_d_ = static_cast<int>(ph.ip2_pol_b.size());
  if (pol_emb_ <= 0 || pol_emb_ % 8 || pol_d_ % 8 || pol_d_ <= 0 || in_channels % 8) {
    throw Error("Unsupported policy head sizes.");
  }
  pol_emb_lin_ = MakeLinear(ph.ip_pol_w, ph.ip_pol_b, pol_emb_, in_channels);
  if (!ph.pol_encoder.empty()) {
    pe_heads_ = ph.pol_encoder_head_count;
    pe_dmodel_ = static_cast<int>(ph.pol_encoder[0].mha.q_b.size());
    pe_dff_ = static_cast<int>(ph.pol_encoder[0].ffn.dense1_b.size());
    if (pe_heads_ <= 0 || pe_dmodel_ <= 0 || pe_dmodel_ % pe_heads_ || pe_dff_ <= 0 || pe_dff_ % 8) {
      throw Error("Unsupported policy encoder sizes.");
    }
    pe_depth_ = pe_dmodel_ / pe_heads_;
    if (!AttentionGenericDepthSupported(pe_depth_)) throw Error("Policy encoder head depth must be at most 128.");
    for (const EncoderLayer& l : ph.pol_encoder) {
      EncoderDev e = MakeEncoderLayer(l, pol_emb_, pe_dmodel_, pe_dff_);
      // The reference runs policy encoder layers through the same ForwardEncoderLayer as the body's
      // (network_blas.cc:836-842), smolgen and the shared generator layer included.
      if (l.mha.has_smolgen) LoadSmolgen(l.mha.smolgen, pol_emb_, pe_heads_, &e, &pe_sg_hc_, &pe_sg_hs_, &pe_sg_gen_, &pe_smolgen_);
      pol_encoders_.push_back(e);
    }
    if (pe_smolgen_) EnsureSmolgenGlobal(w, pe_sg_gen_ / pe_heads_);
  }
  {
    Vec qk_w(ph.ip2_pol_w), qk_b(ph.ip2_pol_b);
    qk_w.insert(qk_w.end(), ph.ip3_pol_w.begin(), ph.ip3_pol_w.end());
    qk_b.insert(qk_b.end(), ph.ip3_pol_b.begin(), ph.ip3_pol_b.end());
    pol_qk_lin_ = MakeLinear(qk_w, qk_b, 2 * pol_d_, pol_emb_);
  }
  if (ph.ip4_pol_w.size() != static_cast<size_t>(4) * pol_d_) throw Error("Promotion weights have a wrong size.");
  ppo_ = UploadF(ph.ip4_pol_w);
  inv_map_ = arena_.Upload(AttnPolicyInverseMap());
}

void Mi355xNetwork::ForwardAttentionPolicy(const half_t* x, int ld_x, int B) {
  const int T = B * 64;
  Gemm("gemm_policy_embed", x, ld_x, pol_emb_lin_, pol_e_, pol_emb_, T, pol_emb_act_);
  for (const EncoderDev& e : pol_encoders_) {   // alpha 1, eps 1e-6 (network_blas.cc:836-842)
    const half_t* bias = nullptr;
    if (e.has_smolgen) {
      SmolgenChain(e, pol_e_, pol_emb_, pe_heads_, pe_sg_hc_, pe_sg_hs_, pe_sg_gen_, pe_sg1_, pe_sg2_, pe_sg3_, pe_sbias_, B,
                   stream_, true);
      bias = pe_sbias_;
    }
    Gemm("gemm_pol_qkv", pol_e_, pol_emb_, e.qkv, pe_qkv_, 3 * pe_dmodel_, T, kActNone);
    Timed("attention", 4.0 * 64 * 64 * pe_depth_ * B * pe_heads_,
          B * pe_heads_ * (static_cast<double>(es_) * 4 * 64 * pe_depth_ + (bias ? es_ * 4096.0 : 0.0)),
          [&] { Attention(pe_qkv_, bias, pe_att_, B, pe_heads_, pe_depth_, stream_); });
    Gemm("gemm_pol_dense", pe_att_, pe_dmodel_, e.dense, pe_t_, pol_emb_, T, kActNone);
    Timed("layer_norm_skip", 0.0, 3.0 * es_ * T * pol_emb_,
          [&] { LayerNorm(pe_t_, pol_e_, pol_e_, e.ln1_g, e.ln1_b, T, pol_emb_, 1.0f, 1e-6f); });
    Gemm("gemm_pol_ffn1", pol_e_, pol_emb_, e.ffn1, pe_ffn_, pe_dff_, T, pe_ffn_act_);
    Gemm("gemm_pol_ffn2", pe_ffn_, pe_dff_, e.ffn2, pe_t_, pol_emb_, T, kActNone);
    Timed("layer_norm_skip", 0.0, 3.0 * es_ * T * pol_emb_,
          [&] { LayerNorm(pe_t_, pol_e_, pol_e_, e.ln2_g, e.ln2_b, T, pol_emb_, 1.0f, 1e-6f); });
  }
  Gemm("gemm_policy_qk", pol_e_, pol_emb_, pol_qk_lin_, pol_qk_, 2 * pol_d_, T, kActNone);
  // Per-sample Q.K^T / sqrt(d): 64 x 64 logits, float (network_blas.cc:850-872).
  const float logit_scale = 1.0f / std::sqrt(static_cast<float>(pol_d_));
  const double logit_flops = 2.0 * 64 * 64 * pol_d_ * B, logit_bytes = B * (2.0 * es_ * 64 * pol_d_ + 4.0 * 4096);
  if (dtype_ == Dtype::kFloat) {
    GemmArgsF32 g;
    g.A = reinterpret_cast<const float*>(pol_qk_); g.lda = 2 * pol_d_; g.strideA = 64LL * 2 * pol_d_;
    g.W = reinterpret_cast<const float*>(ElemAt(pol_qk_, pol_d_)); g.ldw = 2 * pol_d_; g.strideW = 64LL * 2 * pol_d_;
    g.C = pol_logits_; g.ldc = 64; g.strideC = 4096;
    g.M = 64; g.N = 64; g.K = pol_d_; g.batch = B;
    g.scale = logit_scale;
    g.act = kActNone;
    Timed("gemm_policy_logits|gemm_f32_mfma_32x32x2", logit_flops, logit_bytes, [&] { LaunchGemmF32(g, stream_); });
  } else {
    GemmArgs g;
    g.A = pol_qk_; g.lda = 2 * pol_d_; g.strideA = 64LL * 2 * pol_d_;
    g.W = pol_qk_ + pol_d_; g.ldw = 2 * pol_d_; g.strideW = 64LL * 2 * pol_d_;
    g.C = pol_logits_; g.ldc = 64; g.strideC = 4096;
    g.M = 64; g.N = 64; g.K = pol_d_; g.batch = B;
    g.scale = logit_scale;
    g.act = kActNone;
    g.out_f32 = true;
    g.bf16 = dtype_ == Dtype::kBf16;
    const std::string label = std::string("gemm_policy_logits|") + GemmVariantName(g);
    Timed(label.c_str(), logit_flops, logit_bytes, [&] { LaunchGemm(g, stream_); });
  }
  Timed("policy_gather", 0.0, B * (4.0 * 4288 + 4.0 * 1858), [&] {
    if (dtype_ == Dtype::kFloat) {
      LaunchAttnPolicyGather(pol_logits_, reinterpret_cast<const float*>(pol_qk_), 2 * pol_d_, pol_d_, ppo_, pol_d_,
                             inv_map_, d_policy_, B, stream_);
    } else if (dtype_ == Dtype::kBf16) {
      LaunchAttnPolicyGather(pol_logits_, reinterpret_cast<const bf16_t*>(pol_qk_), 2 * pol_d_, pol_d_, ppo_, pol_d_,
                             inv_map_, d_policy_, B, stream_);
    } else {
      LaunchAttnPolicyGather(pol_logits_, pol_qk_, 2 * pol_d_, pol_d_, ppo_, pol_d_, inv_map_, d_policy_, B, stream_);
    }
  });
}

void Mi355xNetwork::BuildAttentionBody(const WeightsFile& file) {
  const NetWeights& w = file.weights;
  const NetworkFormat& nf = file.format;
  if (!w.residual.empty()) throw Error("Attention body on top of a residual tower is not supported.");
  pe_dense_ = nf.input_embedding == kInputEmbeddingPeDense;
  if (!pe_dense_ && nf.input_embedding != kInputEmbeddingPeMap) {
    throw Error("The attention body needs the PE_MAP or PE_DENSE input embedding.");
  }
  gating_ = !w.ip_mult_gate.empty() && !w.ip_add_gate.empty();
  if (!attn_policy_) throw Error("Attention-body networks need the attention policy head.");
  const PolicyHead& ph = w.policy_heads.at(policy_head_);
  const ValueHead& vh = w.value_heads.at(value_head_);

  emb_ = static_cast<int>(w.ip_emb_b.size());
  heads_ = w.encoder_head_count;
  if (emb_ <= 0 || emb_ % 8 != 0 || emb_ > 8192) throw Error("Embedding size must be a multiple of 8 in 8..8192.");
  if (w.encoder.empty() || heads_ <= 0) throw Error("Attention body without encoder layers.");
  d_model_ = static_cast<int>(w.encoder[0].mha.q_b.size());
  dff_ = static_cast<int>(w.encoder[0].ffn.dense1_b.size());
  depth_ = d_model_ / heads_;
  if (d_model_ != heads_ * depth_ || !AttentionGenericDepthSupported(depth_)) {
    throw Error("Attention head depth must be a whole number up to 128 (got " + std::to_string(d_model_) + " / " +
                std::to_string(heads_) + ").");
  }
  if (fp8_ && !AttentionDepthSupported(depth_)) throw Error("precision=fp8 needs an attention head depth of 32, 64 or 128.");
  if (dff_ % 8 != 0) throw Error("FFN width must be a multiple of 8.");
  alpha_ = static_cast<float>(std::pow(2.0 * w.encoder.size(), -0.25));
  eps_ = pe_dense_ ? 1e-3f : 1e-6f;   // src/neural/backends/blas/network_blas.cc:719

  if (pe_dense_) {
    // src/neural/backends/blas/network_blas.cc:612-628, 662-712
    if (w.ip_emb_preproc_b.empty() || w.ip_emb_preproc_b.size() % 64) throw Error("Bad dense position-encoding weights.");
    enc_ch_ = static_cast<int>(w.ip_emb_preproc_b.size() / 64);
    preproc_lin_ = MakeLinear(w.ip_emb_preproc_w, w.ip_emb_preproc_b, 64 * enc_ch_, 64 * 12);
    emb_lin_ = MakeLinear(w.ip_emb_w, w.ip_emb_b, emb_, kInputPlanes + enc_ch_, 64);
    if (static_cast<int>(w.ip_emb_ln_gammas.size()) != emb_ || static_cast<int>(w.ip_emb_ln_betas.size()) != emb_) {
      throw Error("Embedding layer norm parameters do not match the embedding size.");
    }
    emb_ln_g_ = UploadN(w.ip_emb_ln_gammas, emb_, "Embedding layer norm gamma");
    emb_ln_b_ = UploadN(w.ip_emb_ln_betas, emb_, "Embedding layer norm beta");
    emb_dff_ = static_cast<int>(w.ip_emb_ffn.dense1_b.size());
    if (emb_dff_ <= 0 || emb_dff_ % 8) throw Error("Embedding FFN width must be a positive multiple of 8.");
    emb_ffn1_ = MakeLinear(w.ip_emb_ffn.dense1_w, w.ip_emb_ffn.dense1_b, emb_dff_, emb_);
    emb_ffn2_ = MakeLinear(w.ip_emb_ffn.dense2_w, w.ip_emb_ffn.dense2_b, emb_, emb_dff_);
    if (static_cast<int>(w.ip_emb_ffn_ln_gammas.size()) != emb_) throw Error("Embedding FFN layer norm has a wrong size.");
    emb_ffn_ln_g_ = UploadN(w.ip_emb_ffn_ln_gammas, emb_, "Embedding FFN layer norm gamma");
    emb_ffn_ln_b_ = UploadN(w.ip_emb_ffn_ln_betas, emb_, "Embedding FFN layer norm beta");
  } else {
    // (176 inputs padded to 192: whole k-tiles of 64 for the direct-to-LDS GEMM; the expansion kernel zeroes the padding)
    emb_lin_ = MakeLinear(w.ip_emb_w, w.ip_emb_b, emb_, kInputPlanes + 64, 64);
  }
  in_ld_ = emb_lin_.ld;
  if (gating_) {
    // Stored [channel][square] (network_blas.cc:670-682); kept [square][channel] like the activations.
    if (w.ip_mult_gate.size() != static_cast<size_t>(64) * emb_ || w.ip_add_gate.size() != w.ip_mult_gate.size()) {
      throw Error("Input gating weights have a wrong size.");
    }
    Vec mult(w.ip_mult_gate.size()), add(w.ip_add_gate.size());
    for (int c = 0; c < emb_; c++)
      for (int sq = 0; sq < 64; sq++) {
        mult[static_cast<size_t>(sq) * emb_ + c] = w.ip_mult_gate[static_cast<size_t>(c) * 64 + sq];
        add[static_cast<size_t>(sq) * emb_ + c] = w.ip_add_gate[static_cast<size_t>(c) * 64 + sq];
      }
    gate_mult_ = UploadF(mult); gate_add_ = UploadF(add);
  }
  {
    pos_enc_ = UploadElems(PosEncoding());
  }

  if (fp8_ && q_smolgen_auto_) {
    for (const EncoderLayer& l : w.encoder) {
      if (!l.mha.has_smolgen) continue;
      const Smolgen& sg = l.mha.smolgen;
      const size_t hc64 = 64 * (sg.compress.size() / emb_), hs = sg.dense1_b.size(), g = sg.dense2_b.size() / heads_;
      q_smolgen_ = hc64 % 128 == 0 && hs % 128 == 0 && g % 128 == 0 && sg.dense2_b.size() % heads_ == 0;
      break;
    }
  }
  for (const EncoderLayer& l : w.encoder) {
    EncoderDev e;
    if (static_cast<int>(l.mha.q_b.size()) != d_model_ || static_cast<int>(l.ffn.dense1_b.size()) != dff_) {
      throw Error("Encoder layers of different sizes are not supported.");
    }
    Vec qkv_w, qkv_b;
    qkv_w.reserve(3 * l.mha.q_w.size());
    for (const Vec* v : {&l.mha.q_w, &l.mha.k_w, &l.mha.v_w}) qkv_w.insert(qkv_w.end(), v->begin(), v->end());
    for (const Vec* v : {&l.mha.q_b, &l.mha.k_b, &l.mha.v_b}) qkv_b.insert(qkv_b.end(), v->begin(), v->end());
    e.qkv = MakeLinear(qkv_w, qkv_b, 3 * d_model_, emb_);
    e.dense = MakeLinear(l.mha.dense_w, l.mha.dense_b, emb_, d_model_);
    e.ffn1 = MakeLinear(l.ffn.dense1_w, l.ffn.dense1_b, dff_, emb_);
    e.ffn2 = MakeLinear(l.ffn.dense2_w, l.ffn.dense2_b, emb_, dff_);
    if (fp8_) {
      if (emb_ % 128 || d_model_ % 128 || dff_ % 128) {
        throw Error("precision=fp8 needs embedding, attention and FFN widths that are multiples of 128.");
      }
      e.qkv8 = MakeLinearF8(qkv_w, 3 * d_model_, emb_);
      e.dense8 = MakeLinearF8(l.mha.dense_w, emb_, d_model_);
      e.ffn18 = MakeLinearF8(l.ffn.dense1_w, dff_, emb_);
      e.ffn28 = MakeLinearF8(l.ffn.dense2_w, emb_, dff_);
    }
    e.ln1_g = UploadN(l.ln1_gammas, emb_, "Encoder layer norm gamma"); e.ln1_b = UploadN(l.ln1_betas, emb_, "Encoder layer norm beta");
    e.ln2_g = UploadN(l.ln2_gammas, emb_, "Encoder layer norm gamma"); e.ln2_b = UploadN(l.ln2_betas, emb_, "Encoder layer norm beta");
    if (static_cast<int>(l.ln1_gammas.size()) != emb_ || static_cast<int>(l.ln2_gammas.size()) != emb_) {
      throw Error("Layer norm parameters do not match the embedding size.");
    }
    if (l.mha.has_smolgen) {
      const Smolgen& s = l.mha.smolgen;
      LoadSmolgen(s, emb_, heads_, &e, &sg_hc_, &sg_hs_, &sg_gen_, &any_smolgen_);
      if (fp8_ && q_smolgen_) {
        if ((64 * sg_hc_) % 128 || sg_hs_ % 128 || (sg_gen_ / heads_) % 128) {
          throw Error("fp8_gemms=smolgen needs smolgen widths (64 x compression, hidden, generator per head) that are "
                      "multiples of 128.");
        }
        e.sg_compress8 = MakeLinearF8(s.compress, sg_hc_, emb_);
        e.sg_dense18 = MakeLinearF8(s.dense1_w, sg_hs_, 64 * sg_hc_);
        e.sg_dense28 = MakeLinearF8(s.dense2_w, sg_gen_, sg_hs_);
      }
    }
    if (fold_layer_norm_ && !fp8_ && dtype_ == Dtype::kHalf && emb_ % 8 == 0) {
      // Folded layer norms (fp16 path): the layers after a norm get its gamma and beta multiplied in, the layers
      // before one get alpha multiplied into their bias (the GEMM scales the sum by alpha).
      const size_t li = encoders_.size();
      e.ffn1_n = MakeLinearNormFolded(l.ffn.dense1_w, l.ffn.dense1_b, l.ln1_gammas, l.ln1_betas, dff_, emb_);
      if (li > 0) {
        const EncoderLayer& prev = w.encoder[li - 1];
        e.qkv_n = MakeLinearNormFolded(qkv_w, qkv_b, prev.ln2_gammas, prev.ln2_betas, 3 * d_model_, emb_);
        if (e.has_smolgen) {
          e.sg_compress_n = MakeLinearNormFolded(l.mha.smolgen.compress, Vec(), prev.ln2_gammas, prev.ln2_betas,
                                                 sg_hc_, emb_);
        }
      }
      Vec ab(l.mha.dense_b);
      for (float& v : ab) v *= alpha_;
      e.dense_ab = UploadF(ab);
      ab = l.ffn.dense2_b;
      for (float& v : ab) v *= alpha_;
      e.ffn2_ab = UploadF(ab);
    }
    encoders_.push_back(e);
  }
  if (any_smolgen_) {
    const int g = sg_gen_ / heads_;
    EnsureSmolgenGlobal(w, g);
    if (fp8_ && q_smolgen_) {
      for (EncoderDev& e : encoders_) {
        if (!e.has_smolgen) continue;
        e.sg_global8.w = smolgen_w8_;
        e.sg_global8.wscale = smolgen_w8_scale_;
        e.sg_global8.col_scale = AllocF(4096);
      }
    }
    if (fused_smolgen_attention_ && dtype_ != Dtype::kFloat && SmolgenAttentionSupported(heads_, depth_, g)) {
      // The same weights in the fragment order of the kernel that generates the logits inside the attention.
      std::vector<float> frag(w.smolgen_w.size());
      for (int row = 0; row < 4096; row++)
        for (int col = 0; col < g; col++)
          frag[SmolgenFragmentIndex(row, col, g)] = w.smolgen_w[static_cast<size_t>(row) * g + col];
      smolgen_wfrag_ = UploadElems(frag);
    }
  }

  // Heads.
  pol_emb_act_ = default_act_;
  pe_ffn_act_ = ffn_act_;
  BuildAttentionPolicy(w, ph, emb_);

  val_ch_ = static_cast<int>(vh.ip_val_b.size());
  val_fc_ = static_cast<int>(vh.ip1_val_b.size());
  val_out_ = wdl_ ? 3 : 1;
  if (val_ch_ % 8 || val_fc_ % 8) throw Error("Unsupported value head sizes.");
  val_emb_lin_ = MakeLinear(vh.ip_val_w, vh.ip_val_b, val_ch_, emb_);
  val_fc1_ = MakeLinear(vh.ip1_val_w, vh.ip1_val_b, val_fc_, 64 * val_ch_);
  val_fc2_ = MakeLinear(vh.ip2_val_w, vh.ip2_val_b, val_out_, val_fc_);
  if (moves_left_) {
    mov_ch_ = static_cast<int>(w.ip_mov_b.size());
    mov_fc_ = static_cast<int>(w.ip1_mov_b.size());
    if (mov_ch_ % 8 || mov_fc_ % 8) throw Error("Unsupported moves-left head sizes.");
    mov_emb_lin_ = MakeLinear(w.ip_mov_w, w.ip_mov_b, mov_ch_, emb_);
    mov_fc1_ = MakeLinear(w.ip1_mov_w, w.ip1_mov_b, mov_fc_, 64 * mov_ch_);
    mov_fc2_ = MakeLinear(w.ip2_mov_w, w.ip2_mov_b, 1, mov_fc_);
  }

}


// ------------------------------------------------------------ residual tower --
template <typename T>
LinearT Mi355xNetwork::MakeLinearT(const Vec& w, const Vec& b, int out, int in) {
  if (static_cast<size_t>(out) * in != w.size()) {
    throw Error("Weight tensor has " + std::to_string(w.size()) + " elements, expected " + std::to_string(out) +
                " x " + std::to_string(in) + ".");
  }
  if (!b.empty() && static_cast<int>(b.size()) != out) throw Error("Bias size does not match the layer width.");
  LinearT l;
  l.out = out; l.in = in; l.ld = RoundUp(in, 8);
  std::vector<T> h(static_cast<size_t>(out) * l.ld, (T)0.0f);
  for (int o = 0; o < out; o++)
    for (int i = 0; i < in; i++) h[static_cast<size_t>(o) * l.ld + i] = (T)w[static_cast<size_t>(o) * in + i];
  l.w = arena_.Upload(h);
  if (!b.empty()) l.b = arena_.Upload(b);
  return l;
}

template <typename T>
void Mi355xNetwork::GemmT(const char* name, const void* A, int lda, long long strideA, const void* W, int ldw,
                          long long strideW, void* C, int ldc, long long strideC, const float* bias, int M, int N,
                          int K, int batch, int act, bool out_f32) {
  const double flops = 2.0 * M * N * K * batch;
  const double bytes = sizeof(T) * batch * (static_cast<double>(M) * K + static_cast<double>(N) * K) +
                       static_cast<double>(batch) * M * N * (out_f32 ? 4 : sizeof(T));
  if constexpr (sizeof(T) == 2) {
    GemmArgs g;
    g.A = static_cast<const half_t*>(A); g.lda = lda; g.strideA = strideA;
    g.W = static_cast<const half_t*>(W); g.ldw = ldw; g.strideW = strideW;
    g.C = C; g.ldc = ldc; g.strideC = strideC;
    g.bias = bias; g.M = M; g.N = N; g.K = K; g.batch = batch; g.act = act; g.out_f32 = out_f32;
    const std::string label = std::string(name) + "|" + GemmVariantName(g);
    Timed(label.c_str(), flops, bytes, [&] { LaunchGemm(g, stream_); });
  } else {
    GemmArgsF32 g;
    g.A = static_cast<const float*>(A); g.lda = lda; g.strideA = strideA;
    g.W = static_cast<const float*>(W); g.ldw = ldw; g.strideW = strideW;
    g.C = static_cast<float*>(C); g.ldc = ldc; g.strideC = strideC;
    g.bias = bias; g.M = M; g.N = N; g.K = K; g.batch = batch; g.act = act;
    const std::string label = std::string(name) + "|gemm_f32_mfma_32x32x2";
    Timed(label.c_str(), flops, bytes, [&] { LaunchGemmF32(g, stream_); });
  }
}

template <typename T>
void Mi355xNetwork::BuildResnet(const WeightsFile& file) {
  const NetWeights& w = file.weights;
  const NetworkFormat& nf = file.format;
  if (w.residual.empty() && w.input.weights.empty()) throw Error("Network has no input convolution.");
  const PolicyHead& ph = w.policy_heads.at(policy_head_);
  const ValueHead& vh = w.value_heads.at(value_head_);
  filters_ = static_cast<int>(w.input.biases.size());
  if (filters_ <= 0 || filters_ % 8 != 0 || filters_ > 1024) {
    throw Error("The number of filters must be a multiple of 8 in 8..1024.");
  }
  classical_value_ = nf.value == kValueClassical;

  auto make_conv = [&](const ConvBlock& cb, int cout, int cin) {
    if (cb.weights.size() != static_cast<size_t>(cout) * cin * 9 || static_cast<int>(cb.biases.size()) != cout) {
      throw Error("3x3 convolution weights have an unexpected size.");
    }
    ConvDev c;
    // The input convolution's 112 planes are padded to 128 (whole k-tiles for the direct-to-LDS GEMM; the
    // input transform writes the padding as zeros).
    c.cin = cin; c.cout = cout; c.ld = (cin == kInputPlanes && sizeof(T) == 2) ? RoundUp(cin, 64) : RoundUp(cin, 8);
    std::vector<float> u(static_cast<size_t>(36) * cout * c.ld);
    WinogradFilterTransform4x4(cb.weights.data(), cout, cin, c.ld, u.data());
    std::vector<T> ut(u.size());
    for (size_t i = 0; i < u.size(); i++) ut[i] = (T)u[i];
    c.u = arena_.Upload(ut);
    c.bias = arena_.Upload(cb.biases);
    return c;
  };
  res_input_ = make_conv(w.input, filters_, kInputPlanes);
  for (const Residual& r : w.residual) {
    ResBlockDev b;
    b.conv1 = make_conv(r.conv1, filters_, filters_);
    b.conv2 = make_conv(r.conv2, filters_, filters_);
    b.has_se = r.has_se;
    if (r.has_se) {
      b.se.k = static_cast<int>(r.se.b1.size());
      if (b.se.k <= 0 || b.se.k > 256 || r.se.w1.size() != static_cast<size_t>(b.se.k) * filters_ ||
          r.se.w2.size() != static_cast<size_t>(2) * filters_ * b.se.k || r.se.b2.size() != 2u * filters_) {
        throw Error("SE unit weights have an unexpected size.");
      }
      b.se.w1 = arena_.Upload(r.se.w1); b.se.b1 = arena_.Upload(r.se.b1);
      {
        // [2C][K] -> [K][2C], so that threads of neighbouring channels read neighbouring addresses.
        Vec w2t(r.se.w2.size());
        for (int o = 0; o < 2 * filters_; o++)
          for (int k = 0; k < b.se.k; k++) w2t[static_cast<size_t>(k) * 2 * filters_ + o] = r.se.w2[static_cast<size_t>(o) * b.se.k + k];
        b.se.w2 = arena_.Upload(w2t);
      }
      b.se.b2 = arena_.Upload(r.se.b2);
    }
    res_blocks_.push_back(b);
  }

  // A dense layer fed by a flattened [C][64] head tensor: this backend keeps heads as
  // [64][C], so the columns are reordered once here (c*64+sq -> sq*C+c).
  auto make_fc_from_nchw = [&](const Vec& fw, const Vec& fb, int out, int channels) {
    if (fw.size() != static_cast<size_t>(out) * channels * 64) throw Error("Head dense layer has an unexpected size.");
    Vec perm(fw.size());
    for (int o = 0; o < out; o++)
      for (int c = 0; c < channels; c++)
        for (int sq = 0; sq < 64; sq++)
          perm[(static_cast<size_t>(o) * 64 + sq) * channels + c] = fw[(static_cast<size_t>(o) * channels + c) * 64 + sq];
    return MakeLinearT<T>(perm, fb, out, channels * 64);
  };
  auto make_conv1x1 = [&](const ConvBlock& cb, int cin) {
    const int cout = static_cast<int>(cb.biases.size());
    if (cout <= 0 || cout % 8 != 0 || cb.weights.size() != static_cast<size_t>(cout) * cin) {
      throw Error("1x1 head convolution has an unexpected size.");
    }
    return MakeLinearT<T>(cb.weights, cb.biases, cout, cin);
  };

  int max_head_ch = 8;
  if (attn_policy_) {
    // Attention policy on a convolutional body: SELU on the embedding and in the policy
    // encoders' FFN (hard-coded in the reference, network_blas.cc:822-842).
    pol_emb_act_ = kActSelu;
    pe_ffn_act_ = kActSelu;
    BuildAttentionPolicy(w, ph, filters_);
  } else if (conv_policy_) {
    res_policy1_ = make_conv(ph.policy1, filters_, filters_);
    const int pol_out = static_cast<int>(ph.policy.biases.size());
    if (pol_out < 73 || pol_out > 1024) throw Error("Convolutional policy head has an unexpected size.");
    res_policy_conv_ = make_conv(ph.policy, pol_out, filters_);
    conv_inv_map_ = arena_.Upload(ConvPolicyInverseMap());
    max_head_ch = std::max(max_head_ch, pol_out);
  } else {
    res_pol_conv1x1_ = make_conv1x1(ph.policy, filters_);
    res_pol_fc_ = make_fc_from_nchw(ph.ip_pol_w, ph.ip_pol_b, kPolicyOutputs, res_pol_conv1x1_.out);
    max_head_ch = std::max(max_head_ch, res_pol_conv1x1_.out);
  }
  res_val_conv_ = make_conv1x1(vh.value, filters_);
  val_fc_ = static_cast<int>(vh.ip1_val_b.size());
  val_out_ = wdl_ ? 3 : 1;
  if (val_fc_ <= 0 || val_fc_ % 8) throw Error("Unsupported value head sizes.");
  res_val_fc1_ = make_fc_from_nchw(vh.ip1_val_w, vh.ip1_val_b, val_fc_, res_val_conv_.out);
  res_val_fc2_ = MakeLinearT<T>(vh.ip2_val_w, vh.ip2_val_b, val_out_, val_fc_);
  max_head_ch = std::max(max_head_ch, res_val_conv_.out);
  int max_fc = val_fc_;
  if (moves_left_) {
    res_mov_conv_ = make_conv1x1(w.moves_left, filters_);
    mov_fc_ = static_cast<int>(w.ip1_mov_b.size());
    if (mov_fc_ <= 0 || mov_fc_ % 8) throw Error("Unsupported moves-left head sizes.");
    res_mov_fc1_ = make_fc_from_nchw(w.ip1_mov_w, w.ip1_mov_b, mov_fc_, res_mov_conv_.out);
    res_mov_fc2_ = MakeLinearT<T>(w.ip2_mov_w, w.ip2_mov_b, 1, mov_fc_);
    max_head_ch = std::max(max_head_ch, res_mov_conv_.out);
    max_fc = std::max(max_fc, mov_fc_);
  }

  res_max_fc_ = static_cast<size_t>(max_fc);
  res_cmax_ = static_cast<size_t>(std::max(filters_, max_head_ch));
}

// One 3x3 convolution: input transform (unless the previous convolution's output transform
// has already produced it: have_v), 36 batched GEMMs, output transform with the fused tail.
// next: the convolution that consumes the result; when the shapes allow it, its input
// transform is fused into this output transform (returns true), and `out` may be null if
// nothing else reads the activations.
template <typename T>
bool Mi355xNetwork::WinogradConv(const char* name, const ConvDev& conv, const void* x, const void* skip,
                                 const SeDev* se, int act, void* out, int B, bool have_v, const ConvDev* next) {
  const int tiles = B * 4;
  if (!have_v) {
    Timed("winograd_input_transform", 0.0, sizeof(T) * B * (64.0 + 144.0) * conv.cin, [&] {
      LaunchWinogradInputTransform<T>(static_cast<const T*>(x), static_cast<T*>(r_v_), B, conv.cin, conv.ld, stream_);
    });
  }
  // Winograd-domain products M in the tower's own type (half products are accurate enough
  // because the transform matrices are row-balanced; float M would double the traffic of
  // both the GEMM epilogue and the output transform).
  GemmT<T>(name, r_v_, conv.ld, static_cast<long long>(tiles) * conv.ld, conv.u, conv.ld,
           static_cast<long long>(conv.cout) * conv.ld, r_m_, conv.cout, static_cast<long long>(tiles) * conv.cout,
           nullptr, tiles, conv.cout, conv.ld, 36, kActNone, /*out_f32=*/false);
  const bool fuse = next != nullptr && next->cin == conv.cout && next->ld == conv.cout &&
                    WinogradFusedInputTransform(conv.cout, sizeof(T), se ? se->k : 0);
  Timed(fuse ? "winograd_output_input_transform" : "winograd_output_transform", 0.0,
        B * conv.cout * sizeof(T) * (144.0 + 64.0 * ((skip ? 1 : 0) + (out ? 1 : 0)) + (fuse ? 144.0 : 0.0)), [&] {
    LaunchWinogradOutputTransform<T, T>(static_cast<const T*>(r_m_), conv.bias, static_cast<const T*>(skip),
                                        se ? se->w1 : nullptr, se ? se->b1 : nullptr, se ? se->w2 : nullptr,
                                        se ? se->b2 : nullptr, se ? se->k : 0, static_cast<T*>(out), B, conv.cout,
                                        act, stream_, fuse ? static_cast<T*>(r_v_) : nullptr, fuse ? next->ld : 0);
  });
  return fuse;
}

template <typename T>
void Mi355xNetwork::ForwardResnet(int B) {
  const int T64 = B * 64;
  Timed("expand_planes", 0.0, B * (112.0 * 12 + sizeof(T) * 64.0 * 112), [&] {
    LaunchExpandPlanesNhwc<T>(d_masks_, d_values_, static_cast<T*>(r_in_), B, stream_);
  });
  // Every output transform also produces the next convolution's transformed input when the
  // shapes allow it; r_y_ (a block's inner activations) is then never written.
  const ConvDev* after_tower = (conv_policy_ && !attn_policy_) ? &res_policy1_ : nullptr;
  const ConvDev* first = res_blocks_.empty() ? after_tower : &res_blocks_[0].conv1;
  bool have_v = WinogradConv<T>("gemm_winograd_input", res_input_, r_in_, nullptr, nullptr, default_act_, r_x_, B,
                                false, first);
  for (size_t i = 0; i < res_blocks_.size(); i++) {
    const ResBlockDev& blk = res_blocks_[i];
    const ConvDev* next = i + 1 < res_blocks_.size() ? &res_blocks_[i + 1].conv1 : after_tower;
    const bool inner = WinogradFusedInputTransform(blk.conv1.cout, sizeof(T), 0) && blk.conv2.cin == blk.conv1.cout &&
                       blk.conv2.ld == blk.conv1.cout;
    have_v = WinogradConv<T>("gemm_winograd", blk.conv1, r_x_, nullptr, nullptr, default_act_, inner ? nullptr : r_y_, B,
                             have_v, &blk.conv2);
    have_v = WinogradConv<T>("gemm_winograd", blk.conv2, r_y_, r_x_, blk.has_se ? &blk.se : nullptr, default_act_, r_x_,
                             B, have_v, next);
  }
  const bool policy_have_v = have_v;
  auto fc = [&](const char* name, const void* a, const LinearT& l, void* c, int m, int act, bool out_f32) {
    GemmT<T>(name, a, l.ld, 0, l.w, l.ld, 0, c, l.out, 0, l.b, m, l.out, l.ld, 1, act, out_f32);
  };
  // Value head.
  fc("gemm_value_conv", r_x_, res_val_conv_, r_h1_, T64, default_act_, false);
  fc("gemm_value_fc1", r_h1_, res_val_fc1_, r_h2_, B, default_act_, false);
  fc("gemm_value_fc2", r_h2_, res_val_fc2_, d_wdl_, B, kActNone, true);
  if (moves_left_) {
    fc("gemm_mlh_conv", r_x_, res_mov_conv_, r_h1_, T64, default_act_, false);
    fc("gemm_mlh_fc1", r_h1_, res_mov_fc1_, r_h2_, B, default_act_, false);
    fc("gemm_mlh_fc2", r_h2_, res_mov_fc2_, d_mlh_, B, kActRelu, true);
  }
  // Policy head.
  if (attn_policy_) {
    ForwardAttentionPolicy(static_cast<const half_t*>(r_x_), filters_, B);
  } else if (conv_policy_) {
    // (the heads above do not touch r_v_, so the tower's last fused transform is still there)
    const bool v2 = WinogradConv<T>("gemm_winograd_policy", res_policy1_, r_x_, nullptr, nullptr, default_act_, r_y_, B,
                                    policy_have_v, &res_policy_conv_);
    WinogradConv<T>("gemm_winograd_policy", res_policy_conv_, r_y_, nullptr, nullptr, kActNone, r_h1_, B, v2);
    Timed("policy_gather", 0.0, B * (sizeof(T) * 73.0 * 64 + 4.0 * 1858), [&] {
      LaunchConvPolicyGather<T>(static_cast<const T*>(r_h1_), res_policy_conv_.cout, conv_inv_map_, d_policy_, B,
                                stream_);
    });
  } else {
    fc("gemm_policy_conv", r_x_, res_pol_conv1x1_, r_h1_, T64, default_act_, false);
    fc("gemm_policy_fc", r_h1_, res_pol_fc_, d_policy_, B, kActNone, true);
  }
}

// ------------------------------------------------------------------ forward --
void Mi355xNetwork::ForwardAttentionBody(int B) {
  const int T = B * 64;
  // Element-typed views of the plane kernels (the activations are half_t* storage whatever the type).
  auto by_type = [&](auto&& f) {
    if (dtype_ == Dtype::kFloat) f(static_cast<float*>(nullptr));
    else if (dtype_ == Dtype::kBf16) f(static_cast<bf16_t*>(nullptr));
    else f(static_cast<half_t*>(nullptr));
  };
  if (pe_dense_) {
    Timed("piece_planes", 0.0, B * (12.0 * 12 + 768.0 * es_), [&] {
      by_type([&](auto* tag) {
        using E = std::remove_pointer_t<decltype(tag)>;
        LaunchPiecePlanes(d_masks_, d_values_, reinterpret_cast<E*>(pre_in_), B, stream_);
      });
    });
    Gemm("gemm_pos_encoding", pre_in_, 768, preproc_lin_, pre_out_, 64 * enc_ch_, B, kActNone);
    Timed("expand_planes", 0.0, B * (112.0 * 12 + 64.0 * in_ld_ * es_ + 64.0 * enc_ch_ * es_), [&] {
      by_type([&](auto* tag) {
        using E = std::remove_pointer_t<decltype(tag)>;
        LaunchExpandPlanesDense(d_masks_, d_values_, reinterpret_cast<const E*>(pre_out_), enc_ch_,
                                reinterpret_cast<E*>(in0_), in_ld_, B, stream_);
      });
    });
  } else {
    Timed("expand_planes", 0.0, B * (112.0 * 12 + 64.0 * in_ld_ * es_), [&] {
      by_type([&](auto* tag) {
        using E = std::remove_pointer_t<decltype(tag)>;
        LaunchExpandPlanesAttn<E>(d_masks_, d_values_, reinterpret_cast<const E*>(pos_enc_), reinterpret_cast<E*>(in0_),
                                  in_ld_, B, stream_);
      });
    });
  }
  Gemm("gemm_embedding", in0_, in_ld_, emb_lin_, x_, emb_, T, default_act_);
  if (pe_dense_) {
    Timed("layer_norm_skip", 0.0, 2.0 * es_ * T * emb_,
          [&] { LayerNorm(x_, nullptr, x_, emb_ln_g_, emb_ln_b_, T, emb_, 1.0f, 1e-3f); });
  }
  if (gating_) {
    Timed("input_gating", 0.0, 2.0 * es_ * T * emb_, [&] {
      by_type([&](auto* tag) {
        using E = std::remove_pointer_t<decltype(tag)>;
        LaunchInputGating(reinterpret_cast<E*>(x_), gate_mult_, gate_add_, B, 64 * emb_, stream_);
      });
    });
  }
  if (pe_dense_) {
    Gemm("gemm_emb_ffn1", x_, emb_, emb_ffn1_, ffn_, emb_dff_, T, ffn_act_);
    Gemm("gemm_emb_ffn2", ffn_, emb_dff_, emb_ffn2_, t_, emb_, T, kActNone);
    Timed("layer_norm_skip", 0.0, 3.0 * es_ * T * emb_,
          [&] { LayerNorm(t_, x_, x_, emb_ffn_ln_g_, emb_ffn_ln_b_, T, emb_, alpha_, 1e-3f); });
  }
  // fp8: the large GEMMs read e4m3 operands written by the kernel that produces each tensor. The last
  // fp8_fp16_layers_ layers (closest to the heads) can be kept in fp16.
  const bool f8_any = fp8_ && !calibrating_;
  const size_t n_f8_layers = encoders_.size() - std::min<size_t>(encoders_.size(), static_cast<size_t>(fp8_fp16_layers_));
  const size_t nx = static_cast<size_t>(T) * emb_;
  if (calibrating_) RecordAbsMax(x_, nx, 0);
  if (f8_any && n_f8_layers > 0 && (q_qkv_ || q_smolgen_)) {
    Timed("quantize_f8", 0.0, 3.0 * nx,
          [&] { LaunchQuantizeF8(x_, xq_, static_cast<long long>(nx), 1.0f / encoders_[0].s_x, stream_); });
  }

  // Folded layer norms (fp16 arithmetic, batches whose GEMMs all run on the direct-to-LDS kernels): the two
  // norms of a layer run inside the GEMM before them (residual + row sums) and the GEMMs after them (row
  // normalisation of the product), and x_ carries the un-normalised sums from layer to layer.
  const bool fold = !fp8_ && !calibrating_ && CanFoldLayerNorms(B);
  // Where the outputs of a layer's kernels go. A layer writes about eight [T x d_model] tensors of two bytes (the
  // projection's counts for three); while two layers' worth fit the 256 MiB memory-side cache (up to 512 positions
  // at d_model 1024), the large GEMMs whose output is read next by a kernel that is bound by memory (QKV before the
  // attention, attention output and FFN2 before the layer norms) write it through to that cache instead of streaming
  // it past it, and the layer norms do the same. FFN1 keeps streaming: FFN2 does not mind where its operand comes
  // from, and 1.5 tensors' worth of cache stay free for the others. Same-machine runs of the 15x1024 net, fp16
  // 384 positions +1.5 %, 256 +1.8 % (the attention kernel inside a pass 59 -> 46-52 us, both layer norms together
  // 43 -> 37), 512 +0 %, 1024 -4.5 % if forced there; e4m3 256 +1.9 %, 512 +0.5 %, 1024 -1.2 % if forced.
  const bool cache_fits = write_through_ && static_cast<size_t>(T) * d_model_ * 16 <= (static_cast<size_t>(512) << 20);
  const int keep = cache_fits ? kStoresAutoKeep : kStoresAuto;
  const bool ln_through = cache_fits && dtype_ != Dtype::kFloat && static_cast<size_t>(T) * emb_ * 2 >= (32u << 20);
  const float* pend_stats = nullptr;   // row sums of x_ when it holds an un-normalised sum
  const float *pend_gamma = nullptr, *pend_beta = nullptr;
  int pend_parts = 0, mid_parts = 0;
  for (size_t li = 0; li < encoders_.size(); li++) {
    const EncoderDev& e = encoders_[li];
    const bool last = li + 1 == encoders_.size();
    const bool f8 = f8_any && li < n_f8_layers;
    const half_t* bias = nullptr;
    // Folded layer norms: x_ holds the un-normalised sum u when `pending` is set; the layers that read it take
    // the consumer epilogue, the two layers before a norm add the residual in place and leave the row sums.
    NormFold cons_in, cons_mid, prod_mid, prod_out;
    if (fold) {
      cons_in.row_stats = pend_stats; cons_in.row_parts = pend_parts; cons_in.norm_n = emb_; cons_in.eps = eps_;
      prod_mid.skip = x_; prod_mid.ldskip = emb_; prod_mid.skip_stats = pend_stats; prod_mid.skip_parts = pend_parts;
      prod_mid.skip_gamma = pend_gamma; prod_mid.skip_beta = pend_beta;
      prod_mid.stats_out = ln_stats_b_; prod_mid.parts_out = &mid_parts;
      prod_mid.bias = e.dense_ab; prod_mid.scale = alpha_; prod_mid.norm_n = emb_; prod_mid.eps = eps_;
    }
    const bool norm_in = fold && pend_stats != nullptr;   // this layer reads an un-normalised x_
    const bool bf16 = dtype_ == Dtype::kBf16;
    // The smolgen chain depends only on x: it runs on the side stream next to the
    // QKV projection (on the main stream when profiling, for clean per-kernel times).
    hipStream_t ss = (profiling_ || single_stream_ || B < overlap_min_batch_) ? stream_ : side_stream_;
    // The generator layer (smolgen_w) runs inside the attention kernel where that kernel serves the shape.
    // (not with e4m3 operands in the chain: the generator is then an fp8 GEMM of its own)
    const bool chain_f8 = f8 && q_smolgen_ && e.has_smolgen;
    // The generator layer inside the attention kernel (fp16 operands there). With the chain in e4m3 by the default
    // fp8_gemms=auto that still holds - the three layers before it run on e4m3 operands, the generator on the halves
    // the last row norm writes: 4 to 8 % of a pass at 96 to 512 positions against an e4m3 generator GEMM of its own
    // plus the plain attention kernel. An explicit fp8_gemms=...+smolgen keeps all four layers in e4m3.
    const bool fused_gen = e.has_smolgen && smolgen_wfrag_ != nullptr && B >= fused_smolgen_min_batch_ &&
                           (!chain_f8 || q_smolgen_auto_);
    auto launch_qkv = [&] {
      if (f8 && q_qkv_) {
        GemmF8("gemm_qkv", xq_, e.qkv, e.qkv8, qkv_, T, kActNone, false, 1.0f, nullptr, keep);
      } else {
        Gemm("gemm_qkv", x_, emb_, norm_in ? e.qkv_n : e.qkv, qkv_, 3 * d_model_, T, kActNone, false, nullptr, 1, false,
             norm_in ? &cons_in : nullptr, keep);
      }
    };
    // With two streams the projection is recorded before the chain: a replayed graph then keeps it on the hardware
    // queue of the layer norm before it and of the attention after it, and only the chain, which has slack, pays the
    // dependencies between queues.
    const bool qkv_before_chain = e.has_smolgen && ss != stream_ && qkv_first_;
    if (e.has_smolgen) {
      const int g = sg_gen_ / heads_;
      if (ss != stream_) {
        HIP_CHECK(hipEventRecord(fork_events_[li], stream_));
        if (qkv_before_chain) launch_qkv();
        HIP_CHECK(hipStreamWaitEvent(ss, fork_events_[li], 0));
      }
      // The chain is the critical path of this phase when the QKV projection beside it is short (e4m3 operands,
      // or at most 128 positions): its kernels then take the variants with the shortest latency. At larger fp16
      // batches the two are balanced and the leaner variants disturb the projection less (batch 256: 1.5 %).
      const bool chain_first = f8 || B <= chain_latency_max_batch_;
      if (chain_f8) {
        // The whole chain on e4m3 operands: the compression reads the e4m3 copy of x that the QKV projection reads
        // and writes e4m3 itself; the two row norms write halves and their e4m3 copies.
        GemmF8("gemm_smolgen_compress", xq_, e.sg_compress, e.sg_compress8, sg1q_, T, kActNone, true, 1.0f / e.s_sg1, ss);
        GemmF8("gemm_smolgen_dense1", sg1q_, e.sg_dense1, e.sg_dense18, sg2_, B, smolgen_act_, false, 1.0f, ss);
        Timed("layer_norm_rows", 0.0, 5.0 * B * sg_hs_, [&] {
          LaunchLayerNormRows(nullptr, 0, 0, sg2_, kActNone, nullptr, sg2_, e.sg_ln1_g, e.sg_ln1_b, B, sg_hs_, 1.0f,
                              1e-3f, ss, false, sg2q_, 1.0f / e.s_sg2);
        }, ss);
        GemmF8("gemm_smolgen_dense2", sg2q_, e.sg_dense2, e.sg_dense28, sg3_, B, smolgen_act_, false, 1.0f, ss);
        Timed("layer_norm_rows", 0.0, (fused_gen ? 4.0 : 5.0) * B * sg_gen_, [&] {
          LaunchLayerNormRows(nullptr, 0, 0, sg3_, kActNone, nullptr, sg3_, e.sg_ln2_g, e.sg_ln2_b, B, sg_gen_, 1.0f,
                              1e-3f, ss, false, fused_gen ? nullptr : sg3q_, 1.0f / e.s_sg3);
        }, ss);
        if (!fused_gen) {
          GemmF8("gemm_smolgen_global", sg3q_, smolgen_w_, e.sg_global8, sbias_, B * heads_, kActNone, false, 1.0f, ss);
        }
      } else if (dtype_ == Dtype::kFloat) {
        SmolgenChain(e, x_, emb_, heads_, sg_hc_, sg_hs_, sg_gen_, sg1_, sg2_, sg3_, sbias_, B, ss, chain_first);
      } else {
      Gemm("gemm_smolgen_compress", x_, emb_, norm_in ? e.sg_compress_n : e.sg_compress, sg1_, sg_hc_, T, kActNone,
           false, ss, 1, chain_first, norm_in ? &cons_in : nullptr);
      // dense1 has a long reduction and few outputs. With few rows one workgroup per 16x16 outputs splits K over
      // its waves; from dense1_split_min_batch_ rows on, workgroups split K between them, accumulate in float, and
      // the layer norm kernel adds the slices and applies the activation.
      if (B < dense1_split_min_batch_) {
        Gemm("gemm_smolgen_dense1", sg1_, 64 * sg_hc_, e.sg_dense1, sg2_, sg_hs_, B, smolgen_act_, false, ss, 1,
             chain_first);
        Timed("layer_norm_rows", 0.0, 4.0 * B * sg_hs_, [&] {
          LaunchLayerNormRows(nullptr, 0, 0, sg2_, kActNone, nullptr, sg2_, e.sg_ln1_g, e.sg_ln1_b, B, sg_hs_, 1.0f,
                              1e-3f, ss, bf16);
        }, ss);
      } else {
        const int split = std::max(1, std::min(16, (64 * sg_hc_) / 256));
        Gemm("gemm_smolgen_dense1", sg1_, 64 * sg_hc_, e.sg_dense1, sg2f_, sg_hs_, B, kActNone, true, ss, split);
        Timed("layer_norm_rows", 0.0, (4.0 * split + 2.0) * B * sg_hs_, [&] {
          LaunchLayerNormRows(sg2f_, split, static_cast<long long>(B) * sg_hs_, nullptr, smolgen_act_, nullptr, sg2_,
                              e.sg_ln1_g, e.sg_ln1_b, B, sg_hs_, 1.0f, 1e-3f, ss, bf16);
        }, ss);
      }
      if (calibrating_ && q_smolgen_) {
        RecordAbsMax(sg1_, static_cast<size_t>(T) * sg_hc_, SmolgenSlot(li, 0), ss);
        RecordAbsMax(sg2_, static_cast<size_t>(B) * sg_hs_, SmolgenSlot(li, 1), ss);
      }
      Gemm("gemm_smolgen_dense2", sg2_, sg_hs_, e.sg_dense2, sg3_, sg_gen_, B, smolgen_act_, false, ss, 1, chain_first);
      Timed("layer_norm_rows", 0.0, 4.0 * B * sg_gen_, [&] {
        LaunchLayerNormRows(nullptr, 0, 0, sg3_, kActNone, nullptr, sg3_, e.sg_ln2_g, e.sg_ln2_b, B, sg_gen_, 1.0f, 1e-3f,
                            ss, bf16);
      }, ss);
      if (calibrating_ && q_smolgen_) RecordAbsMax(sg3_, static_cast<size_t>(B) * sg_gen_, SmolgenSlot(li, 2), ss);
      if (!fused_gen) {
        Gemm("gemm_smolgen_global", sg3_, g, smolgen_w_, sbias_, 4096, B * heads_, kActNone, false, ss, 1, chain_first);
      }
      }
      if (ss != stream_) HIP_CHECK(hipEventRecord(join_events_[li], ss));
      bias = sbias_;
    }
    if (!qkv_before_chain) launch_qkv();
    if (e.has_smolgen && ss != stream_) HIP_CHECK(hipStreamWaitEvent(stream_, join_events_[li], 0));
    const int gen_sz = e.has_smolgen ? sg_gen_ / heads_ : 0;
    const double att_flops = 4.0 * 64 * 64 * depth_ * B * heads_ + (fused_gen ? 2.0 * 4096 * gen_sz * B * heads_ : 0.0);
    const bool att_f8 = f8 && q_dense_;
    const double att_bytes =
        B * heads_ * (2.0 * 3 * 64 * depth_ + (att_f8 ? 1.0 : 2.0) * 64 * depth_ +
                      (fused_gen ? 2.0 * gen_sz : bias ? 2.0 * 4096 : 0.0));
    const float att_scale = 1.0f / std::sqrt(static_cast<float>(depth_));
    if (att_f8 && fused_gen) {
      Timed("smolgen_attention", att_flops, att_bytes, [&] {
        LaunchSmolgenAttentionF8Out(qkv_, sg3_, smolgen_wfrag_, attq_, 1.0f / e.s_att, B, heads_, depth_, gen_sz,
                                    att_scale, stream_);
      });
      GemmF8("gemm_mha_dense", attq_, e.dense, e.dense8, t_, T, kActNone, false, 1.0f, nullptr, keep);
    } else if (att_f8) {
      Timed("attention", att_flops, att_bytes,
            [&] { LaunchAttentionF8Out(qkv_, bias, attq_, 1.0f / e.s_att, B, heads_, att_scale, stream_, depth_); });
      GemmF8("gemm_mha_dense", attq_, e.dense, e.dense8, t_, T, kActNone, false, 1.0f, nullptr, keep);
    } else {
      if (fused_gen) {
        Timed("smolgen_attention", att_flops, att_bytes, [&] {
          LaunchSmolgenAttention(qkv_, sg3_, smolgen_wfrag_, att_, B, heads_, depth_, gen_sz, att_scale, stream_, bf16);
        });
      } else {
        Timed("attention", att_flops, att_bytes, [&] { Attention(qkv_, bias, att_, B, heads_, depth_, stream_); });
      }
      if (calibrating_) RecordAbsMax(att_, static_cast<size_t>(T) * d_model_, static_cast<int>(4 * li + 1));
      if (fold) {
        // x_ <- alpha * (att . dense + b) + LN2_prev(x_), with the row sums of the new x_
        Gemm("gemm_mha_dense", att_, d_model_, e.dense, x_, emb_, T, kActNone, false, nullptr, 1, false, &prod_mid);
        cons_mid.row_stats = ln_stats_b_; cons_mid.row_parts = mid_parts; cons_mid.norm_n = emb_; cons_mid.eps = eps_;
        Gemm("gemm_ffn1", x_, emb_, e.ffn1_n, ffn_, dff_, T, ffn_act_, false, nullptr, 1, false, &cons_mid);
        prod_out.skip = x_; prod_out.ldskip = emb_; prod_out.skip_stats = ln_stats_b_; prod_out.skip_parts = mid_parts;
        prod_out.skip_gamma = e.ln1_g; prod_out.skip_beta = e.ln1_b;
        prod_out.stats_out = ln_stats_a_; prod_out.parts_out = &pend_parts;
        prod_out.bias = e.ffn2_ab; prod_out.scale = alpha_; prod_out.norm_n = emb_; prod_out.eps = eps_;
        Gemm("gemm_ffn2", ffn_, dff_, e.ffn2, x_, emb_, T, kActNone, false, nullptr, 1, false, &prod_out);
        pend_stats = ln_stats_a_; pend_gamma = e.ln2_g; pend_beta = e.ln2_b;
        if (last) {   // the heads read normalised rows
          Timed("layer_norm", 0.0, 4.0 * T * emb_, [&] {
            LaunchLayerNorm(x_, nullptr, x_, pend_gamma, pend_beta, T, emb_, 1.0f, eps_, stream_, nullptr, 1.0f);
          });
        }
        continue;
      }
      Gemm("gemm_mha_dense", att_, d_model_, e.dense, t_, emb_, T, kActNone, false, nullptr, 1, false, nullptr, keep);
    }
    const bool ln1_f8 = f8 && q_ffn1_;
    Timed("layer_norm_skip", 0.0, (ln1_f8 ? 7.0 : 3.0 * es_) * T * emb_, [&] {
      LayerNorm(t_, x_, x_, e.ln1_g, e.ln1_b, T, emb_, alpha_, eps_, stream_, ln1_f8 ? xq_ : nullptr, 1.0f / e.s_x1,
                ln_through);
    });
    if (calibrating_) RecordAbsMax(x_, nx, static_cast<int>(4 * li + 2));
    const bool ffn_f8 = f8 && q_ffn2_;   // FFN2 reads an e4m3 operand
    if (f8 && q_ffn1_) {
      GemmF8("gemm_ffn1", xq_, e.ffn1, e.ffn18, ffn_f8 ? static_cast<void*>(ffnq_) : ffn_, T, ffn_act_, ffn_f8,
             1.0f / e.s_ffn);
    } else {
      Gemm("gemm_ffn1", x_, emb_, e.ffn1, ffn_, dff_, T, ffn_act_);
      if (calibrating_) RecordAbsMax(ffn_, static_cast<size_t>(T) * dff_, static_cast<int>(4 * li + 3));
      if (ffn_f8) {
        const size_t nf = static_cast<size_t>(T) * dff_;
        Timed("quantize_f8", 0.0, 3.0 * nf,
              [&] { LaunchQuantizeF8(ffn_, ffnq_, static_cast<long long>(nf), 1.0f / e.s_ffn, stream_); });
      }
    }
    if (ffn_f8) {
      GemmF8("gemm_ffn2", ffnq_, e.ffn2, e.ffn28, t_, T, kActNone, false, 1.0f, nullptr, keep);
    } else {
      Gemm("gemm_ffn2", ffn_, dff_, e.ffn2, t_, emb_, T, kActNone, false, nullptr, 1, false, nullptr, keep);
    }
    const bool ln2_f8 = f8_any && li + 1 < n_f8_layers && (q_qkv_ || q_smolgen_);   // the next layer reads an e4m3 copy
    Timed("layer_norm_skip", 0.0, (ln2_f8 ? 7.0 : 3.0 * es_) * T * emb_, [&] {
      LayerNorm(t_, x_, x_, e.ln2_g, e.ln2_b, T, emb_, alpha_, eps_, stream_, ln2_f8 ? xq_ : nullptr,
                last ? 1.0f : 1.0f / encoders_[li + 1].s_x, ln_through);
    });
    if (calibrating_) RecordAbsMax(x_, nx, static_cast<int>(4 * li + 4));
  }

  // Value and moves-left heads: six small GEMMs that leave most CUs idle. From a batch size on (two
  // cross-queue dependencies must be paid for) they run on the side stream beside the policy head.
  // Measured on one machine: 15x1024 net, fp16, -0.7 % (batch 256) to -2 % (batch 16) of the pass; fp8 -2 % from
  // batch 64, +11 % at batch 16 where nothing else uses the side stream; a 10x256 net loses 1-10 % at every
  // batch size (its six head GEMMs are shorter than the two dependencies). Hence the automatic rule: wide
  // bodies only, and only where the smolgen chain already runs on the side stream.
  const int heads_min = heads_overlap_min_batch_ >= 0 ? heads_overlap_min_batch_
                                                      : (emb_ >= 768 ? std::max(overlap_min_batch_, 16) : 1 << 30);
  const bool heads_beside = !profiling_ && !single_stream_ && B >= heads_min;
  hipStream_t hs = heads_beside ? side_stream_ : stream_;
  if (heads_beside) {
    HIP_CHECK(hipEventRecord(heads_fork_, stream_));
    HIP_CHECK(hipStreamWaitEvent(hs, heads_fork_, 0));
  }
  Gemm("gemm_value_embed", x_, emb_, val_emb_lin_, head1_, val_ch_, T, default_act_, false, hs);
  Gemm("gemm_value_fc1", head1_, 64 * val_ch_, val_fc1_, head2_, val_fc_, B, default_act_, false, hs);
  Gemm("gemm_value_fc2", head2_, val_fc_, val_fc2_, d_wdl_, val_out_, B, kActNone, /*out_f32=*/true, hs);
  if (moves_left_) {
    Gemm("gemm_mlh_embed", x_, emb_, mov_emb_lin_, head1_, mov_ch_, T, default_act_, false, hs);
    Gemm("gemm_mlh_fc1", head1_, 64 * mov_ch_, mov_fc1_, head2_, mov_fc_, B, default_act_, false, hs);
    Gemm("gemm_mlh_fc2", head2_, mov_fc_, mov_fc2_, d_mlh_, 1, B, kActRelu, /*out_f32=*/true, hs);
  }
  if (heads_beside) HIP_CHECK(hipEventRecord(heads_join_, hs));
  // Policy head.
  ForwardAttentionPolicy(x_, emb_, B);
  if (heads_beside) HIP_CHECK(hipStreamWaitEvent(stream_, heads_join_, 0));
}

void Mi355xNetwork::LaunchEager(int batch) {
  if (attn_body_) {
    ForwardAttentionBody(batch);
  } else if (fp32_) {
    ForwardResnet<float>(batch);
  } else {
    ForwardResnet<half_t>(batch);
  }
}

void Mi355xNetwork::DropGraphs() {
  for (auto& g : graphs_) (void)hipGraphExecDestroy(g.second);
  graphs_.clear();
}

void Mi355xNetwork::ForwardDevice(int batch) {
  constexpr size_t kMaxGraphs = 192;
  if (!use_graphs_ || profiling_ || calibrating_) {
    LaunchEager(batch);
    return;
  }
  const int key = 2 * batch + (single_stream_ ? 1 : 0);
  auto it = graphs_.find(key);
  if (it == graphs_.end()) {
    if (graphs_.size() >= kMaxGraphs) {
      LaunchEager(batch);
      return;
    }
    // Record the launch sequence of this batch size once. All buffers are allocated at
    // construction and kernel arguments depend only on the batch size, so the recorded
    // graph stays valid (calibration, which changes fp8 scales, drops the graphs).
    hipGraph_t graph = nullptr;
    HIP_CHECK(hipStreamBeginCapture(stream_, hipStreamCaptureModeThreadLocal));
    try {
      LaunchEager(batch);
    } catch (...) {
      (void)hipStreamEndCapture(stream_, &graph);
      if (graph) (void)hipGraphDestroy(graph);
      use_graphs_ = false;
      throw;
    }
    HIP_CHECK(hipStreamEndCapture(stream_, &graph));
    hipGraphExec_t exec = nullptr;
    hipError_t err = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (err != hipSuccess) {
      use_graphs_ = false;
      throw Error(std::string("HIP error: ") + hipGetErrorString(err) + " (hipGraphInstantiate)");
    }
    it = graphs_.emplace(key, exec).first;
  }
  HIP_CHECK(hipGraphLaunch(it->second, stream_));
}

Mi355xNetwork* Mi355xNetwork::AcquireLane(bool* others_busy) {
  std::unique_lock<std::mutex> lock(lane_mutex_);
  lane_cv_.wait(lock, [&] { return !free_lanes_.empty(); });
  Mi355xNetwork* lane = free_lanes_.back();   // most recently used first
  free_lanes_.pop_back();
  *others_busy = lane_count_ - static_cast<int>(free_lanes_.size()) > 1;
  return lane;
}

void Mi355xNetwork::ReleaseLane(Mi355xNetwork* lane) {
  {
    std::lock_guard<std::mutex> lock(lane_mutex_);
    free_lanes_.push_back(lane);
  }
  lane_cv_.notify_all();
}

// Exclusive use of the network (profiling, timing, calibration): waits until no
// computation is in flight on any lane.
void Mi355xNetwork::AcquireAllLanes() {
  std::unique_lock<std::mutex> lock(lane_mutex_);
  lane_cv_.wait(lock, [&] { return static_cast<int>(free_lanes_.size()) == lane_count_; });
  free_lanes_.clear();
}

void Mi355xNetwork::ReleaseAllLanes() {
  {
    std::lock_guard<std::mutex> lock(lane_mutex_);
    free_lanes_.clear();
    for (auto it = extra_lanes_.rbegin(); it != extra_lanes_.rend(); ++it) free_lanes_.push_back(it->get());
    free_lanes_.push_back(this);
  }
  lane_cv_.notify_all();
}

void Mi355xNetwork::Evaluate(HostSlot* slot, int batch) {
  if (batch <= 0) return;
  if (profiling_.load()) {   // per-kernel timing records live in this object: run alone, on this lane
    AcquireAllLanes();
    single_stream_ = false;
    try {
      EvaluateOnLane(slot, batch);
    } catch (...) {
      DrainStreams();
      ReleaseAllLanes();
      throw;
    }
    ReleaseAllLanes();
    return;
  }
  // A pass that starts while another lane is busy keeps to its main stream: the other passes fill the GPU,
  // and two streams per lane are more than the hardware queues of the process (with 2 threads on the 15x1024
  // net: batch 16 8.0k -> 14.2k evals/s, batch 64 24.9k -> 31.6k, batch 256 42.3k -> 44.9k). A lone pass
  // uses the second stream as the batch-size rules say (single thread, batch 256: 41.8k against 38.1k without).
  bool others_busy = false;
  Mi355xNetwork* lane = AcquireLane(&others_busy);
  lane->single_stream_ = others_busy && attn_body_;   // (a residual tower uses one stream anyway)
  try {
    lane->EvaluateOnLane(slot, batch);
  } catch (...) {
    lane->DrainStreams();
    ReleaseLane(lane);
    throw;
  }
  ReleaseLane(lane);
}

// After a failed pass work may still be queued on the lane's streams (copies from the pinned slot, kernels on the
// lane's buffers): wait for it, ignoring errors, before the lane and the slot are reused.
void Mi355xNetwork::DrainStreams() {
  (void)hipSetDevice(device_);
  if (stream_) (void)hipStreamSynchronize(stream_);
  if (side_stream_) (void)hipStreamSynchronize(side_stream_);
  (void)hipGetLastError();
}

void Mi355xNetwork::EvaluateOnLane(HostSlot* slot, int batch) {
  std::lock_guard<std::mutex> lock(eval_mutex_);
  // Argument errors are reported before anything is enqueued: the lane's streams stay idle.
  if (slot->legal_samples > 0 && slot->legal_samples != batch) {
    throw Error("legal moves were given for some inputs of the batch only");
  }
  HIP_CHECK(hipSetDevice(device_));
  HIP_CHECK(hipMemcpyAsync(d_masks_, slot->masks, sizeof(uint64_t) * kInputPlanes * batch, hipMemcpyHostToDevice,
                           stream_));
  HIP_CHECK(hipMemcpyAsync(d_values_, slot->values, sizeof(float) * kInputPlanes * batch, hipMemcpyHostToDevice,
                           stream_));
  const bool legal = slot->legal_samples > 0;
  if (legal) {
    const int total = slot->legal_off[batch];
    HIP_CHECK(hipMemcpyAsync(d_legal_off_, slot->legal_off, sizeof(int) * (batch + 1), hipMemcpyHostToDevice, stream_));
    if (total > 0) {
      HIP_CHECK(hipMemcpyAsync(d_legal_ids_, slot->legal_ids, sizeof(uint16_t) * total, hipMemcpyHostToDevice,
                               stream_));
    }
  }
  ForwardDevice(batch);
  HIP_CHECK(hipGetLastError());
  if (legal) {
    // Only the probabilities of the listed moves are downloaded (tens of floats per sample instead of 1858).
    const int total = slot->legal_off[batch];
    Timed("legal_softmax", 0.0, total * 10.0 + batch * 4.0, [&] {
      LaunchLegalSoftmax(d_policy_, d_legal_off_, d_legal_ids_, slot->inv_temperature, d_legal_probs_, batch, stream_);
    });
    HIP_CHECK(hipGetLastError());
    if (total > 0) {
      HIP_CHECK(hipMemcpyAsync(slot->legal_probs, d_legal_probs_, sizeof(float) * total, hipMemcpyDeviceToHost,
                               stream_));
    }
  } else {
    HIP_CHECK(hipMemcpyAsync(slot->policy, d_policy_, sizeof(float) * kPolicyOutputs * batch, hipMemcpyDeviceToHost,
                             stream_));
  }
  HIP_CHECK(hipMemcpyAsync(slot->wdl, d_wdl_, sizeof(float) * (wdl_ ? 3 : 1) * batch, hipMemcpyDeviceToHost,
                           stream_));
  if (moves_left_) {
    HIP_CHECK(hipMemcpyAsync(slot->mlh, d_mlh_, sizeof(float) * batch, hipMemcpyDeviceToHost, stream_));
  }
  HIP_CHECK(hipStreamSynchronize(stream_));
  if (profiling_) CollectPending();
  // Value post-processing on the host (3 numbers per sample).
  for (int i = 0; i < batch; i++) {
    if (wdl_) {
      float* v = slot->wdl + 3 * i;
      float m = std::max(v[0], std::max(v[1], v[2]));
      float e0 = std::exp(v[0] - m), e1 = std::exp(v[1] - m), e2 = std::exp(v[2] - m);
      float s = e0 + e1 + e2;
      v[0] = e0 / s; v[1] = e1 / s; v[2] = e2 / s;
    } else {
      slot->wdl[i] = std::tanh(slot->wdl[i]);
    }
  }
}

double Mi355xNetwork::TimeResidentForward(int batch, int iters) {
  if (batch < 1 || batch > max_batch_) throw Error("batch out of range");
  if (iters < 1) throw Error("iters must be positive");
  AcquireAllLanes();
  struct Release {
    Mi355xNetwork* n;
    ~Release() { n->ReleaseAllLanes(); }
  } release{this};
  std::lock_guard<std::mutex> lock(eval_mutex_);
  HIP_CHECK(hipSetDevice(device_));
  const bool was_profiling = profiling_.load();
  profiling_ = false;
  single_stream_ = false;
  hipEvent_t start = NewEvent(), stop = NewEvent();
  HIP_CHECK(hipEventRecord(start, stream_));
  for (int i = 0; i < iters; i++) ForwardDevice(batch);
  HIP_CHECK(hipEventRecord(stop, stream_));
  HIP_CHECK(hipStreamSynchronize(stream_));
  HIP_CHECK(hipGetLastError());
  float ms = 0.0f;
  HIP_CHECK(hipEventElapsedTime(&ms, start, stop));
  event_pool_.push_back(start);
  event_pool_.push_back(stop);
  profiling_ = was_profiling;
  return ms / iters;
}

std::unique_ptr<HostSlot> Mi355xNetwork::GetSlot() {
  {
    std::lock_guard<std::mutex> lock(pool_->mutex);
    if (!pool_->free_slots.empty()) {
      auto s = std::move(pool_->free_slots.back());
      pool_->free_slots.pop_back();
      s->legal_samples = 0;
      return s;
    }
  }
  HIP_CHECK(hipSetDevice(device_));
  auto s = std::make_unique<HostSlot>();
  s->capacity = max_batch_;
  HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&s->masks), sizeof(uint64_t) * kInputPlanes * max_batch_));
  HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&s->values), sizeof(float) * kInputPlanes * max_batch_));
  HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&s->policy), sizeof(float) * kPolicyOutputs * max_batch_));
  HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&s->wdl), sizeof(float) * 3 * max_batch_));
  HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&s->mlh), sizeof(float) * max_batch_));
  return s;
}

void Mi355xNetwork::ReleaseSlot(std::unique_ptr<HostSlot> slot) {
  std::lock_guard<std::mutex> lock(pool_->mutex);
  pool_->free_slots.push_back(std::move(slot));
}

// -------------------------------------------------------------- computation --
Mi355xComputation::~Mi355xComputation() {
  std::lock_guard<std::mutex> lock(pool_->mutex);
  if (pool_->network_alive) {
    for (auto& s : slots_) pool_->free_slots.push_back(std::move(s));
  }
  // Otherwise the slots are simply freed here (pinned memory outlives the network object).
}

HostSlot* Mi355xComputation::SlotFor(int index) {
  Mi355xNetwork* net = Net();
  if (max_batch_ == 0) {
    max_batch_ = net->GetMaxBatchSize();
    wdl_ = net->wdl();
    moves_left_ = net->moves_left();
  }
  const size_t si = static_cast<size_t>(index / max_batch_);
  while (slots_.size() <= si) slots_.push_back(net->GetSlot());
  return slots_[si].get();
}

void Mi355xComputation::AddInput(InputPlanes&& input) {
  if (input.size() != static_cast<size_t>(kInputPlanes)) {
    throw Error("AddInput expects exactly 112 input planes, got " + std::to_string(input.size()) + ".");
  }
  HostSlot* s = SlotFor(batch_);
  const int at = batch_ % max_batch_;
  uint64_t* m = s->masks + static_cast<size_t>(at) * kInputPlanes;
  float* v = s->values + static_cast<size_t>(at) * kInputPlanes;
  for (int i = 0; i < kInputPlanes; i++) {
    m[i] = input[i].mask;
    v[i] = input[i].value;
  }
  batch_++;
  computed_ = false;
}

void Mi355xComputation::AddInputs(int n, const uint64_t* masks, const float* values) {
  if (n < 0) throw Error("negative input count");
  for (int i = 0; i < n; i++) {
    HostSlot* s = SlotFor(batch_);
    const int at = batch_ % max_batch_;
    std::memcpy(s->masks + static_cast<size_t>(at) * kInputPlanes, masks + static_cast<size_t>(i) * kInputPlanes,
                sizeof(uint64_t) * kInputPlanes);
    std::memcpy(s->values + static_cast<size_t>(at) * kInputPlanes, values + static_cast<size_t>(i) * kInputPlanes,
                sizeof(float) * kInputPlanes);
    batch_++;
  }
  computed_ = false;
}

void Mi355xComputation::ComputeBlocking() {
  Mi355xNetwork* net = Net();
  for (size_t si = 0; si < slots_.size(); si++) {
    const int n = std::min(max_batch_, batch_ - static_cast<int>(si) * max_batch_);
    HostSlot* s = slots_[si].get();
    if (legal_mode_ && s->legal_samples != n) {
      throw Error("AddLegalMoves must be called for every input, right after it is added");
    }
    // The same reciprocal the search wrapper keeps (src/neural/wrapper.cc:81-82).
    s->inv_temperature = 1.0f / temperature_;
    net->Evaluate(s, n);
  }
  computed_ = true;
}

const float* Mi355xComputation::GetPolicyRow(int sample) const {
  CheckSample(sample);
  if (legal_mode_) {
    throw Error("raw policy logits are not downloaded when legal moves were given: use GetLegalPolicy");
  }
  const int cap = max_batch_;
  return slots_[sample / cap]->policy + static_cast<size_t>(sample % cap) * kPolicyOutputs;
}

void Mi355xComputation::AddLegalMoves(int n, const uint16_t* move_ids) {
  if (batch_ == 0) throw Error("AddLegalMoves needs an input: call it after AddInput");
  if (n < 0 || n > kMaxLegalMoves) throw Error("legal move count out of range (0.." + std::to_string(kMaxLegalMoves) + ")");
  if (n > 0 && !move_ids) throw Error("null move list");
  const int sample = batch_ - 1;
  HostSlot* s = slots_[static_cast<size_t>(sample / max_batch_)].get();
  const int at = sample % max_batch_;
  if (s->legal_samples != at) {
    throw Error(s->legal_samples > at ? "AddLegalMoves was already called for this input"
                                      : "AddLegalMoves must be called for every input, right after it is added");
  }
  if (sample > 0 && !legal_mode_) throw Error("AddLegalMoves must be called for every input, right after it is added");
  for (int i = 0; i < n; i++) {
    if (move_ids[i] >= kPolicyOutputs) throw Error("move id out of range");
  }
  if (!s->legal_off) {
    HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&s->legal_off), sizeof(int) * (s->capacity + 1)));
    HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&s->legal_ids), sizeof(uint16_t) * kMaxLegalMoves * s->capacity));
    HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&s->legal_probs), sizeof(float) * kMaxLegalMoves * s->capacity));
  }
  if (at == 0) s->legal_off[0] = 0;
  const int off = s->legal_off[at];
  if (n > 0) std::memcpy(s->legal_ids + off, move_ids, sizeof(uint16_t) * n);
  s->legal_off[at + 1] = off + n;
  s->legal_samples = at + 1;
  legal_mode_ = true;
}

void Mi355xComputation::SetPolicySoftmaxTemperature(float temperature) {
  if (!(temperature > 0.0f)) throw Error("policy softmax temperature must be positive");
  temperature_ = temperature;
}

const float* Mi355xComputation::GetLegalPolicy(int sample, int* n) const {
  CheckSample(sample);
  if (!legal_mode_) throw Error("no legal moves were given to this computation");
  const HostSlot* s = slots_[static_cast<size_t>(sample / max_batch_)].get();
  const int at = sample % max_batch_;
  if (n) *n = s->legal_off[at + 1] - s->legal_off[at];
  return s->legal_probs + s->legal_off[at];
}

float Mi355xComputation::GetQVal(int sample) const {
  CheckSample(sample);
  const int cap = max_batch_;
  const float* w = slots_[sample / cap]->wdl;
  if (wdl_) return w[3 * (sample % cap)] - w[3 * (sample % cap) + 2];
  return w[sample % cap];
}

float Mi355xComputation::GetDVal(int sample) const {
  CheckSample(sample);
  if (!wdl_) return 0.0f;
  const int cap = max_batch_;
  return slots_[sample / cap]->wdl[3 * (sample % cap) + 1];
}

float Mi355xComputation::GetMVal(int sample) const {
  CheckSample(sample);
  if (!moves_left_) return 0.0f;
  const int cap = max_batch_;
  return slots_[sample / cap]->mlh[sample % cap];
}

}  // namespace

std::unique_ptr<Network> MakeMi355xNetwork(const WeightsFile& weights, Options& options) {
  const NetworkFormat& nf = weights.format;
  switch (nf.network) {
    case kNetworkClassicalWithHeadformat:
    case kNetworkSeWithHeadformat:
    case kNetworkAttentionBodyWithHeadformat:
    case kNetworkAttentionBodyWithMultiheadformat:
      break;
    default:
      throw Error("Network format " + std::to_string(nf.network) + " is not supported by the mi355x backend.");
  }
  if (nf.policy != kPolicyClassical && nf.policy != kPolicyConvolution && nf.policy != kPolicyAttention) {
    throw Error("Policy format " + std::to_string(nf.policy) + " is not supported by the mi355x backend.");
  }
  if (nf.value != kValueClassical && nf.value != kValueWdl) {
    throw Error("Value format " + std::to_string(nf.value) + " is not supported by the mi355x backend.");
  }
  if (nf.moves_left != kMovesLeftNone && nf.moves_left != kMovesLeftV1) {
    throw Error("Moves left head format " + std::to_string(nf.moves_left) + " is not supported by the mi355x backend.");
  }
  if (nf.default_activation != 0 && nf.default_activation != 1) {
    throw Error("Default activation " + std::to_string(nf.default_activation) + " is not supported by the mi355x backend.");
  }
  if (nf.input_embedding != kInputEmbeddingNone && nf.input_embedding != kInputEmbeddingPeMap &&
      nf.input_embedding != kInputEmbeddingPeDense) {
    throw Error("Input embedding " + std::to_string(nf.input_embedding) + " is not supported by the mi355x backend.");
  }
  auto net = std::make_unique<Mi355xNetwork>(weights, options);
  options.CheckAllOptionsRead("mi355x");
  return net;
}

}  // namespace lc0mi
