// Host-side model of an lc0 weights file: gzip + protobuf wire parsing of
// pblczero.Net and the float tensors of the network, resolved the way lc0's
// MultiHeadWeights does (src/neural/network_legacy.h:28-229).
#pragma once

#include <cstddef>
#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace lc0mi {

// Error type of the host library; the C ABI turns it into an error string and
// the lc0 adapter rethrows it as lczero::Exception.
class Error : public std::runtime_error {
 public:
  explicit Error(const std::string& what) : std::runtime_error(what) {}
};

using Vec = std::vector<float>;

// pblczero.NetworkFormat (proto/net.proto:275-366), already upgraded by the
// rules of FixOlderWeightsFile (src/neural/loader.cc:108-158).
struct NetworkFormat {
  int input = 0, output = 0, network = 0, policy = 0, value = 0, moves_left = 0;
  int default_activation = 0, smolgen_activation = 0, ffn_activation = 0;
  int input_embedding = 0;
  bool has_input_embedding = false;
};

enum : int {
  kNetworkClassical = 1, kNetworkSe = 2, kNetworkClassicalWithHeadformat = 3,
  kNetworkSeWithHeadformat = 4, kNetworkOnnx = 5, kNetworkAttentionBodyWithHeadformat = 6,
  kNetworkAttentionBodyWithMultiheadformat = 7, kNetworkAbLegacyWithMultiheadformat = 134,
  kPolicyClassical = 1, kPolicyConvolution = 2, kPolicyAttention = 3,
  kValueClassical = 1, kValueWdl = 2, kMovesLeftNone = 0, kMovesLeftV1 = 1,
  kInputEmbeddingNone = 0, kInputEmbeddingPeMap = 1, kInputEmbeddingPeDense = 2,
};

// src/neural/tables/activation_function.h:24-35 (same numbering as net.proto).
enum Activation : int {
  kActDefault = 0, kActMish = 1, kActRelu = 2, kActNone = 3, kActTanh = 4,
  kActSigmoid = 5, kActSelu = 6, kActSwish = 7, kActRelu2 = 8, kActSoftmax = 9,
};

struct ConvBlock { Vec weights, biases; };  // batch norm already folded
struct SeUnit { Vec w1, b1, w2, b2; };
struct Residual { ConvBlock conv1, conv2; SeUnit se; bool has_se = false; };
struct Smolgen { Vec compress, dense1_w, dense1_b, ln1_gammas, ln1_betas, dense2_w, dense2_b, ln2_gammas, ln2_betas; };
struct Mha { Vec q_w, q_b, k_w, k_b, v_w, v_b, dense_w, dense_b; Smolgen smolgen; bool has_smolgen = false; };
struct Ffn { Vec dense1_w, dense1_b, dense2_w, dense2_b; };
struct EncoderLayer { Mha mha; Vec ln1_gammas, ln1_betas; Ffn ffn; Vec ln2_gammas, ln2_betas; };

struct PolicyHead {
  Vec ip_pol_w, ip_pol_b;  // head's own or the shared embedding
  ConvBlock policy1, policy;
  Vec ip2_pol_w, ip2_pol_b, ip3_pol_w, ip3_pol_b, ip4_pol_w;
  int pol_encoder_head_count = 0;
  std::vector<EncoderLayer> pol_encoder;
};

struct ValueHead {
  ConvBlock value;
  Vec ip_val_w, ip_val_b, ip1_val_w, ip1_val_b, ip2_val_w, ip2_val_b;
};

struct NetWeights {
  ConvBlock input;
  std::vector<Residual> residual;
  Vec ip_emb_preproc_w, ip_emb_preproc_b, ip_emb_w, ip_emb_b, ip_emb_ln_gammas, ip_emb_ln_betas;
  Vec ip_mult_gate, ip_add_gate;
  Ffn ip_emb_ffn;
  Vec ip_emb_ffn_ln_gammas, ip_emb_ffn_ln_betas;
  std::vector<EncoderLayer> encoder;
  int encoder_head_count = 0;
  ConvBlock moves_left;
  Vec ip_mov_w, ip_mov_b, ip1_mov_w, ip1_mov_b, ip2_mov_w, ip2_mov_b;
  Vec smolgen_w;
  bool has_smolgen = false;
  std::map<std::string, PolicyHead> policy_heads;
  std::map<std::string, ValueHead> value_heads;
};

struct WeightsFile {
  NetworkFormat format;
  NetWeights weights;
};

// Parses raw (already gunzipped) pblczero.Net bytes. Throws Error.
WeightsFile ParseWeightsProto(const void* data, size_t len);
// Reads a .pb.gz (or an uncompressed .pb) file. Throws Error.
WeightsFile LoadWeightsFromFile(const std::string& path);
// Inflates a gzip stream held in memory; returns the input unchanged when it
// does not start with the gzip magic.
std::string MaybeGunzip(const void* data, size_t len);

}  // namespace lc0mi
