// Weights-file reader of the MI355X backend.
//
// What it reproduces from lc0 (reference file:line):
//   gzip container, "1\n"/"2\n" text-format rejection   src/neural/loader.cc:59-106,190-208
//   magic / min_version / encoding checks               src/neural/loader.cc:160-188
//   FixOlderWeightsFile format upgrades                 src/neural/loader.cc:108-158
//   Layer decoding (LINEAR16/FLOAT16/BFLOAT16/FLOAT32)  src/utils/weights_adapter.cc:38-80
//   batch-norm folding of ConvBlock                     src/neural/network_legacy.cc:78-133
//   legacy vs multi-head field resolution               src/neural/network_legacy.cc:232-307
//   message/field numbers                               proto/net.proto:31-411
//
// The protobuf wire format is walked directly (varint keys, length-delimited
// sub-messages); no generated code and no protobuf runtime are needed.
#include "weights.h"

#include <zlib.h>

#include <cmath>
#include <cstdio>
#include <cstring>

namespace lc0mi {
namespace {

struct Span {
  const uint8_t* p = nullptr;
  size_t n = 0;
  bool present = false;
};

// One decoded field occurrence.
struct Field {
  uint32_t number;
  uint32_t wire_type;
  uint64_t varint;  // wire types 0, 1 (as bits), 5 (as bits)
  Span bytes;       // wire type 2
};

class Reader {
 public:
  Reader(const uint8_t* p, size_t n) : p_(p), end_(p + n) {}
  bool Next(Field* f) {
    if (p_ >= end_) return false;
    uint64_t key = Varint();
    f->number = static_cast<uint32_t>(key >> 3);
    f->wire_type = static_cast<uint32_t>(key & 7);
    f->bytes = Span();
    switch (f->wire_type) {
      case 0: f->varint = Varint(); break;
      case 1: Need(8); std::memcpy(&f->varint, p_, 8); p_ += 8; break;
      case 2: {
        uint64_t len = Varint();
        Need(len);
        f->bytes.p = p_; f->bytes.n = static_cast<size_t>(len); f->bytes.present = true;
        p_ += len;
        break;
      }
      case 5: { Need(4); uint32_t v; std::memcpy(&v, p_, 4); f->varint = v; p_ += 4; break; }
      default: throw Error("Invalid weight file: unsupported protobuf wire type.");
    }
    return true;
  }

 private:
  void Need(uint64_t n) {
    if (static_cast<uint64_t>(end_ - p_) < n) throw Error("Invalid weight file: truncated protobuf.");
  }
  uint64_t Varint() {
    uint64_t v = 0;
    for (int shift = 0; shift < 64; shift += 7) {
      Need(1);
      uint8_t b = *p_++;
      v |= static_cast<uint64_t>(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
    }
    throw Error("Invalid weight file: bad varint.");
  }
  const uint8_t* p_;
  const uint8_t* end_;
};

// A parsed message: last occurrence of every singular field plus all
// occurrences of repeated sub-messages, addressed by field number.
struct Msg {
  std::map<uint32_t, Span> sub;                  // last length-delimited value
  std::map<uint32_t, std::vector<Span>> repeated;
  std::map<uint32_t, uint64_t> scalar;           // last varint/fixed value
  explicit Msg(Span s) {
    if (!s.present) return;
    Reader r(s.p, s.n);
    Field f;
    while (r.Next(&f)) {
      if (f.wire_type == 2) {
        sub[f.number] = f.bytes;
        repeated[f.number].push_back(f.bytes);
      } else {
        scalar[f.number] = f.varint;
      }
    }
  }
  bool Has(uint32_t n) const { return sub.count(n) || scalar.count(n); }
  Span Sub(uint32_t n) const { auto it = sub.find(n); return it == sub.end() ? Span() : it->second; }
  uint64_t Scalar(uint32_t n, uint64_t def = 0) const {
    auto it = scalar.find(n);
    return it == scalar.end() ? def : it->second;
  }
  const std::vector<Span>& Repeated(uint32_t n) const {
    static const std::vector<Span> kEmpty;
    auto it = repeated.find(n);
    return it == repeated.end() ? kEmpty : it->second;
  }
};

float BitsToFloat(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

float HalfToFloat(uint16_t h) {
  uint32_t sign = static_cast<uint32_t>(h & 0x8000) << 16;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ff;
  if (exp == 0) {
    if (man == 0) return BitsToFloat(sign);
    // subnormal: man * 2^-24
    float f = std::ldexp(static_cast<float>(man), -24);
    return sign ? -f : f;
  }
  if (exp == 31) return BitsToFloat(sign | 0x7f800000u | (man << 13));
  return BitsToFloat(sign | ((exp + 112) << 23) | (man << 13));
}

// Weights.Layer -> floats.
Vec DecodeLayer(Span s) {
  Vec out;
  if (!s.present) return out;
  Msg l(s);
  const int encoding = l.scalar.count(4) ? static_cast<int>(l.Scalar(4)) : 1;  // default LINEAR16
  const Span params = l.Sub(3);
  const float lo = BitsToFloat(static_cast<uint32_t>(l.Scalar(1)));
  const float hi = BitsToFloat(static_cast<uint32_t>(l.Scalar(2)));
  switch (encoding) {
    case 1: {
      size_t n = params.n / 2;
      out.resize(n);
      for (size_t i = 0; i < n; i++) {
        uint16_t u; std::memcpy(&u, params.p + 2 * i, 2);
        float theta = u / static_cast<float>(0xffff);
        out[i] = lo * (1 - theta) + hi * theta;
      }
      break;
    }
    case 2: {
      size_t n = params.n / 2;
      out.resize(n);
      for (size_t i = 0; i < n; i++) { uint16_t u; std::memcpy(&u, params.p + 2 * i, 2); out[i] = HalfToFloat(u); }
      break;
    }
    case 3: {
      size_t n = params.n / 2;
      out.resize(n);
      for (size_t i = 0; i < n; i++) { uint16_t u; std::memcpy(&u, params.p + 2 * i, 2); out[i] = BitsToFloat(static_cast<uint32_t>(u) << 16); }
      break;
    }
    case 4: {
      size_t n = params.n / 4;
      out.resize(n);
      if (n) std::memcpy(out.data(), params.p, n * 4);
      break;
    }
    default:
      throw Error("Unknown layer encoding " + std::to_string(encoding));
  }
  return out;
}

ConvBlock DecodeConvBlock(Span s) {
  ConvBlock cb;
  if (!s.present) return cb;
  Msg m(s);
  cb.weights = DecodeLayer(m.Sub(1));
  cb.biases = DecodeLayer(m.Sub(2));
  Vec means = DecodeLayer(m.Sub(3)), stddivs = DecodeLayer(m.Sub(4));
  Vec gammas = DecodeLayer(m.Sub(5)), betas = DecodeLayer(m.Sub(6));
  if (cb.weights.empty()) return cb;
  if (betas.empty()) { betas.assign(means.size(), 0.0f); gammas.assign(means.size(), 1.0f); }
  if (cb.biases.empty()) cb.biases.assign(means.size(), 0.0f);
  if (means.empty()) return cb;
  constexpr float kEpsilon = 1e-5f;
  for (size_t i = 0; i < stddivs.size(); i++) {
    gammas[i] *= 1.0f / std::sqrt(stddivs[i] + kEpsilon);
    means[i] -= cb.biases[i];
  }
  const size_t outputs = cb.biases.size();
  const size_t inputs = cb.weights.size() / outputs;
  for (size_t o = 0; o < outputs; o++) {
    for (size_t c = 0; c < inputs; c++) cb.weights[o * inputs + c] *= gammas[o];
    cb.biases[o] = -gammas[o] * means[o] + betas[o];
  }
  return cb;
}

Ffn DecodeFfn(Span s) {
  Ffn f;
  Msg m(s);
  f.dense1_w = DecodeLayer(m.Sub(1)); f.dense1_b = DecodeLayer(m.Sub(2));
  f.dense2_w = DecodeLayer(m.Sub(3)); f.dense2_b = DecodeLayer(m.Sub(4));
  return f;
}

EncoderLayer DecodeEncoderLayer(Span s) {
  EncoderLayer e;
  Msg m(s);
  Msg mha(m.Sub(1));
  if (mha.Has(10) || mha.Has(11) || mha.Has(12)) throw Error("RPE weights file not supported.");
  e.mha.q_w = DecodeLayer(mha.Sub(1)); e.mha.q_b = DecodeLayer(mha.Sub(2));
  e.mha.k_w = DecodeLayer(mha.Sub(3)); e.mha.k_b = DecodeLayer(mha.Sub(4));
  e.mha.v_w = DecodeLayer(mha.Sub(5)); e.mha.v_b = DecodeLayer(mha.Sub(6));
  e.mha.dense_w = DecodeLayer(mha.Sub(7)); e.mha.dense_b = DecodeLayer(mha.Sub(8));
  e.mha.has_smolgen = mha.Has(9);
  if (e.mha.has_smolgen) {
    Msg sg(mha.Sub(9));
    Smolgen& g = e.mha.smolgen;
    g.compress = DecodeLayer(sg.Sub(1));
    g.dense1_w = DecodeLayer(sg.Sub(2)); g.dense1_b = DecodeLayer(sg.Sub(3));
    g.ln1_gammas = DecodeLayer(sg.Sub(4)); g.ln1_betas = DecodeLayer(sg.Sub(5));
    g.dense2_w = DecodeLayer(sg.Sub(6)); g.dense2_b = DecodeLayer(sg.Sub(7));
    g.ln2_gammas = DecodeLayer(sg.Sub(8)); g.ln2_betas = DecodeLayer(sg.Sub(9));
  }
  e.ln1_gammas = DecodeLayer(m.Sub(2)); e.ln1_betas = DecodeLayer(m.Sub(3));
  e.ffn = DecodeFfn(m.Sub(4));
  e.ln2_gammas = DecodeLayer(m.Sub(5)); e.ln2_betas = DecodeLayer(m.Sub(6));
  return e;
}

PolicyHead DecodePolicyHead(Span s, const Vec& shared_w, const Vec& shared_b) {
  PolicyHead h;
  Msg m(s);
  h.ip_pol_w = DecodeLayer(m.Sub(1)); h.ip_pol_b = DecodeLayer(m.Sub(2));
  if (h.ip_pol_w.empty()) h.ip_pol_w = shared_w;
  if (h.ip_pol_b.empty()) h.ip_pol_b = shared_b;
  h.ip2_pol_w = DecodeLayer(m.Sub(3)); h.ip2_pol_b = DecodeLayer(m.Sub(4));
  h.ip3_pol_w = DecodeLayer(m.Sub(5)); h.ip3_pol_b = DecodeLayer(m.Sub(6));
  h.ip4_pol_w = DecodeLayer(m.Sub(7));
  for (const Span& e : m.Repeated(8)) h.pol_encoder.push_back(DecodeEncoderLayer(e));
  h.pol_encoder_head_count = static_cast<int>(m.Scalar(9));
  h.policy1 = DecodeConvBlock(m.Sub(10));
  h.policy = DecodeConvBlock(m.Sub(11));
  return h;
}

ValueHead DecodeValueHead(Span s) {
  ValueHead h;
  Msg m(s);
  h.ip_val_w = DecodeLayer(m.Sub(1)); h.ip_val_b = DecodeLayer(m.Sub(2));
  h.ip1_val_w = DecodeLayer(m.Sub(3)); h.ip1_val_b = DecodeLayer(m.Sub(4));
  h.ip2_val_w = DecodeLayer(m.Sub(5)); h.ip2_val_b = DecodeLayer(m.Sub(6));
  h.value = DecodeConvBlock(m.Sub(11));
  return h;
}

NetWeights DecodeWeights(const Msg& w) {
  NetWeights W;
  W.input = DecodeConvBlock(w.Sub(1));
  for (const Span& r : w.Repeated(2)) {
    Msg m(r);
    Residual res;
    res.conv1 = DecodeConvBlock(m.Sub(1));
    res.conv2 = DecodeConvBlock(m.Sub(2));
    res.has_se = m.Has(3);
    if (res.has_se) {
      Msg se(m.Sub(3));
      res.se.w1 = DecodeLayer(se.Sub(1)); res.se.b1 = DecodeLayer(se.Sub(2));
      res.se.w2 = DecodeLayer(se.Sub(3)); res.se.b2 = DecodeLayer(se.Sub(4));
    }
    W.residual.push_back(std::move(res));
  }
  W.ip_emb_preproc_w = DecodeLayer(w.Sub(37)); W.ip_emb_preproc_b = DecodeLayer(w.Sub(38));
  W.ip_emb_w = DecodeLayer(w.Sub(25)); W.ip_emb_b = DecodeLayer(w.Sub(26));
  W.ip_emb_ln_gammas = DecodeLayer(w.Sub(39)); W.ip_emb_ln_betas = DecodeLayer(w.Sub(40));
  W.ip_mult_gate = DecodeLayer(w.Sub(33)); W.ip_add_gate = DecodeLayer(w.Sub(34));
  W.ip_emb_ffn = DecodeFfn(w.Sub(41));
  W.ip_emb_ffn_ln_gammas = DecodeLayer(w.Sub(42)); W.ip_emb_ffn_ln_betas = DecodeLayer(w.Sub(43));
  for (const Span& e : w.Repeated(27)) W.encoder.push_back(DecodeEncoderLayer(e));
  W.encoder_head_count = static_cast<int>(w.Scalar(28));
  W.moves_left = DecodeConvBlock(w.Sub(12));
  W.ip_mov_w = DecodeLayer(w.Sub(31)); W.ip_mov_b = DecodeLayer(w.Sub(32));
  W.ip1_mov_w = DecodeLayer(w.Sub(13)); W.ip1_mov_b = DecodeLayer(w.Sub(14));
  W.ip2_mov_w = DecodeLayer(w.Sub(15)); W.ip2_mov_b = DecodeLayer(w.Sub(16));
  W.smolgen_w = DecodeLayer(w.Sub(35));
  W.has_smolgen = w.Has(35);

  const bool has_policy_heads = w.Has(45);
  Msg ph(w.Sub(45));
  Vec shared_w = DecodeLayer(ph.Has(1) ? ph.Sub(1) : w.Sub(4));
  Vec shared_b = DecodeLayer(ph.Has(2) ? ph.Sub(2) : w.Sub(5));
  W.policy_heads.emplace("vanilla", DecodePolicyHead(ph.Sub(3), shared_w, shared_b));
  if (has_policy_heads) {
    if (ph.Has(4)) W.policy_heads.emplace("optimistic", DecodePolicyHead(ph.Sub(4), shared_w, shared_b));
    if (ph.Has(5)) W.policy_heads.emplace("soft", DecodePolicyHead(ph.Sub(5), shared_w, shared_b));
    if (ph.Has(6)) W.policy_heads.emplace("opponent", DecodePolicyHead(ph.Sub(6), shared_w, shared_b));
  } else {
    if (w.Has(3) || w.Has(11) || w.Has(4)) {
      PolicyHead& v = W.policy_heads.at("vanilla");
      v.policy1 = DecodeConvBlock(w.Sub(11));
      v.policy = DecodeConvBlock(w.Sub(3));
      v.ip2_pol_w = DecodeLayer(w.Sub(17)); v.ip2_pol_b = DecodeLayer(w.Sub(18));
      v.ip3_pol_w = DecodeLayer(w.Sub(19)); v.ip3_pol_b = DecodeLayer(w.Sub(20));
      v.ip4_pol_w = DecodeLayer(w.Sub(22));
      v.pol_encoder_head_count = static_cast<int>(w.Scalar(24));
      for (const Span& e : w.Repeated(21)) v.pol_encoder.push_back(DecodeEncoderLayer(e));
    } else {
      throw Error("Could not find valid policy head weights.");
    }
  }

  const bool has_value_heads = w.Has(44);
  Msg vh(w.Sub(44));
  W.value_heads.emplace("winner", DecodeValueHead(vh.Sub(1)));
  if (has_value_heads) {
    if (vh.Has(2)) W.value_heads.emplace("q", DecodeValueHead(vh.Sub(2)));
    if (vh.Has(3)) W.value_heads.emplace("st", DecodeValueHead(vh.Sub(3)));
  } else {
    if (w.Has(6) || w.Has(29)) {
      ValueHead& win = W.value_heads.at("winner");
      win.value = DecodeConvBlock(w.Sub(6));
      win.ip_val_w = DecodeLayer(w.Sub(29)); win.ip_val_b = DecodeLayer(w.Sub(30));
      win.ip1_val_w = DecodeLayer(w.Sub(7)); win.ip1_val_b = DecodeLayer(w.Sub(8));
      win.ip2_val_w = DecodeLayer(w.Sub(9)); win.ip2_val_b = DecodeLayer(w.Sub(10));
    } else {
      throw Error("Could not find valid value head weights.");
    }
  }
  return W;
}

uint32_t VersionInt(uint64_t major, uint64_t minor, uint64_t patch) {
  return static_cast<uint32_t>(major * 1000000 + minor * 1000 + patch);
}

}  // namespace

WeightsFile ParseWeightsProto(const void* data, size_t len) {
  Span top;
  top.p = static_cast<const uint8_t*>(data); top.n = len; top.present = true;
  Msg net(top);
  if (static_cast<uint32_t>(net.Scalar(1)) != 0x1c0u) throw Error("Invalid weight file: bad header.");
  Msg mv(net.Sub(3));
  const uint32_t net_ver = VersionInt(mv.Scalar(1), mv.Scalar(2), mv.Scalar(3));
  Msg fmt(net.Sub(4));
  const bool has_nf = fmt.Has(2);
  Msg nfm(fmt.Sub(2));
  WeightsFile file;
  NetworkFormat& nf = file.format;
  nf.input = static_cast<int>(nfm.Scalar(1)); nf.output = static_cast<int>(nfm.Scalar(2));
  nf.network = static_cast<int>(nfm.Scalar(3)); nf.policy = static_cast<int>(nfm.Scalar(4));
  nf.value = static_cast<int>(nfm.Scalar(5)); nf.moves_left = static_cast<int>(nfm.Scalar(6));
  nf.default_activation = static_cast<int>(nfm.Scalar(7));
  nf.smolgen_activation = static_cast<int>(nfm.Scalar(8));
  nf.ffn_activation = static_cast<int>(nfm.Scalar(9));
  nf.input_embedding = static_cast<int>(nfm.Scalar(10));
  nf.has_input_embedding = nfm.Has(10);
  const bool has_weights = net.Has(10);
  if (net.Has(11) && !has_weights) throw Error("ONNX networks are not supported by the mi355x backend.");
  Msg w(net.Sub(10));

  if (!has_nf) {
    nf.input = 1; nf.output = 1;
    nf.network = kNetworkClassicalWithHeadformat; nf.value = kValueClassical; nf.policy = kPolicyClassical;
  } else if (nf.network == kNetworkClassical) {
    nf.network = kNetworkClassicalWithHeadformat; nf.value = kValueClassical; nf.policy = kPolicyClassical;
  } else if (nf.network == kNetworkSe) {
    nf.network = kNetworkSeWithHeadformat; nf.value = kValueClassical; nf.policy = kPolicyClassical;
  } else if (nf.network == kNetworkSeWithHeadformat && !w.Repeated(27).empty()) {
    nf.network = kNetworkAttentionBodyWithHeadformat;
    if (w.Has(35)) { nf.ffn_activation = kActRelu2; nf.smolgen_activation = kActSwish; }
  } else if (nf.network == kNetworkAbLegacyWithMultiheadformat) {
    nf.network = kNetworkAttentionBodyWithMultiheadformat;
  }
  if (nf.network == kNetworkAttentionBodyWithHeadformat) {
    if (w.Has(45) && w.Has(44)) {
      nf.network = kNetworkAttentionBodyWithMultiheadformat;
      nf.input_embedding = kInputEmbeddingPeDense; nf.has_input_embedding = true;
    }
    if (!nf.has_input_embedding) { nf.input_embedding = kInputEmbeddingPeMap; nf.has_input_embedding = true; }
  }
  if (net_ver != 0x5c99973u && net_ver > VersionInt(0, 33, 0)) {
    throw Error("Invalid weight file: lc0 version >= " + std::to_string(mv.Scalar(1)) + "." +
                std::to_string(mv.Scalar(2)) + "." + std::to_string(mv.Scalar(3)) + " required.");
  }
  if (has_weights && fmt.Scalar(1) != 1 && net_ver < VersionInt(0, 33, 0)) {
    throw Error("Invalid weight file: unsupported encoding.");
  }
  file.weights = DecodeWeights(w);
  return file;
}

std::string MaybeGunzip(const void* data, size_t len) {
  const uint8_t* p = static_cast<const uint8_t*>(data);
  if (len < 2 || p[0] != 0x1f || p[1] != 0x8b) return std::string(reinterpret_cast<const char*>(p), len);
  z_stream zs;
  std::memset(&zs, 0, sizeof(zs));
  if (inflateInit2(&zs, 15 + 16) != Z_OK) throw Error("Cannot initialise zlib.");
  std::string out;
  out.resize(std::max<size_t>(len * 4, 1 << 20));
  zs.next_in = const_cast<Bytef*>(p);
  zs.avail_in = static_cast<uInt>(len);
  size_t produced = 0;
  for (;;) {
    zs.next_out = reinterpret_cast<Bytef*>(&out[produced]);
    zs.avail_out = static_cast<uInt>(std::min<size_t>(out.size() - produced, 1u << 30));
    int rc = inflate(&zs, Z_NO_FLUSH);
    produced = zs.total_out;
    if (rc == Z_STREAM_END) break;
    if (rc != Z_OK && rc != Z_BUF_ERROR) {
      inflateEnd(&zs);
      throw Error(std::string("Invalid weight file: gzip error: ") + (zs.msg ? zs.msg : "corrupt stream"));
    }
    if (zs.avail_out == 0) out.resize(out.size() * 2);
    else if (zs.avail_in == 0) { inflateEnd(&zs); throw Error("Invalid weight file: truncated gzip stream."); }
  }
  inflateEnd(&zs);
  out.resize(produced);
  return out;
}

WeightsFile LoadWeightsFromFile(const std::string& path) {
  FILE* fp = std::fopen(path.c_str(), "rb");
  if (!fp) throw Error("Cannot read weights from " + path);
  std::string raw;
  char buf[1 << 16];
  size_t n;
  while ((n = std::fread(buf, 1, sizeof(buf), fp)) > 0) raw.append(buf, n);
  std::fclose(fp);
  std::string buffer = MaybeGunzip(raw.data(), raw.size());
  if (buffer.size() < 2) throw Error("Invalid weight file: too small.");
  if (buffer[0] == '1' && buffer[1] == '\n') throw Error("Invalid weight file: no longer supported.");
  if (buffer[0] == '2' && buffer[1] == '\n') {
    throw Error("Text format weights files are no longer supported. Use a command line tool to convert it to the new format.");
  }
  return ParseWeightsProto(buffer.data(), buffer.size());
}

}  // namespace lc0mi
