"""Seeded synthetic lc0 networks (random-init weights of a given architecture).

Produces nested dicts for `netproto.write_pb_gz`; the files are loadable by a
real lc0 (FLOAT32 layers, legacy top-level head fields so that
src/neural/loader.cc:146-153 does not switch the net to PE_DENSE).

Tensor shapes follow src/neural/network_legacy.h and the consumers in
src/neural/backends/blas/network_blas.cc: dense weights are [out][in]
row-major, convolution filters [out][in][3][3].
"""
import os

import numpy as np

from . import netproto

# pblczero.NetworkFormat enums (proto/net.proto:275-366)
INPUT_CLASSICAL_112_PLANE = 1
INPUT_112_WITH_CANONICALIZATION_HECTOPLIES = 4
OUTPUT_WDL = 2
NETWORK_SE_WITH_HEADFORMAT = 4
NETWORK_ATTENTIONBODY_WITH_HEADFORMAT = 6
NETWORK_ATTENTIONBODY_WITH_MULTIHEADFORMAT = 7
POLICY_CLASSICAL, POLICY_CONVOLUTION, POLICY_ATTENTION = 1, 2, 3
VALUE_WDL = 2
MOVES_LEFT_NONE, MOVES_LEFT_V1 = 0, 1
DEFAULT_ACTIVATION_RELU, DEFAULT_ACTIVATION_MISH = 0, 1
ACTIVATION_DEFAULT, ACTIVATION_SWISH = 0, 7
INPUT_EMBEDDING_PE_MAP, INPUT_EMBEDDING_PE_DENSE = 1, 2


class _Gen:
    def __init__(self, seed):
        self.rng = np.random.default_rng(seed)

    def normal(self, shape, std):
        return (self.rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float32)


def _encoder_layer(g, emb, d_model, dff, std, bias_std, smolgen=None, heads=None, perturb_ln=False):
    """One EncoderLayer message (q/k/v/dense, layer norms, FFN, optional smolgen)."""
    def fc(cout, cin, bias=True):
        w = g.normal((cout, cin), std)
        return (w, g.normal((cout,), bias_std)) if bias else w

    def ln(n):
        if perturb_ln:
            return 1.0 + g.normal((n,), 0.1), g.normal((n,), 0.1)
        return np.ones(n, np.float32), np.zeros(n, np.float32)

    mha = {}
    mha["q_w"], mha["q_b"] = fc(d_model, emb)
    mha["k_w"], mha["k_b"] = fc(d_model, emb)
    mha["v_w"], mha["v_b"] = fc(d_model, emb)
    mha["dense_w"], mha["dense_b"] = fc(emb, d_model)
    if smolgen:
        hc, hs, gsz = smolgen
        sg = {"compress": fc(hc, emb, bias=False)}
        sg["dense1_w"], sg["dense1_b"] = fc(hs, 64 * hc)
        sg["ln1_gammas"], sg["ln1_betas"] = ln(hs)
        sg["dense2_w"], sg["dense2_b"] = fc(heads * gsz, hs)
        sg["ln2_gammas"], sg["ln2_betas"] = ln(heads * gsz)
        mha["smolgen"] = sg
    layer = {"mha": mha}
    layer["ln1_gammas"], layer["ln1_betas"] = ln(emb)
    ffn = {}
    ffn["dense1_w"], ffn["dense1_b"] = fc(dff, emb)
    ffn["dense2_w"], ffn["dense2_b"] = fc(emb, dff)
    layer["ffn"] = ffn
    layer["ln2_gammas"], layer["ln2_betas"] = ln(emb)
    return layer


def se_resnet(filters, blocks, se_channels, seed, policy_channels=32, value_channels=32,
              value_fc=128, bias_std=0.02, moves_left=False, conv_policy=False, attn_policy=None):
    """Classical SE-ResNet: weights N(0, 1/fan_in) (std = fan_in**-0.5).

    attn_policy = (embedding, d_model, encoder_layers, encoder_heads, encoder_dff): attention policy
    head on the convolutional body (the "apmish" family, network_blas.cc:806-842)."""
    g = _Gen(seed)

    def conv(cout, cin, k):
        fan_in = cin * k * k
        return {"weights": g.normal((cout, cin, k, k), fan_in ** -0.5),
                "biases": g.normal((cout,), bias_std)}

    def fc(cout, cin):
        return g.normal((cout, cin), cin ** -0.5), g.normal((cout,), bias_std)

    w = {"input": conv(filters, 112, 3), "residual": []}
    for _ in range(blocks):
        blk = {"conv1": conv(filters, filters, 3), "conv2": conv(filters, filters, 3)}
        if se_channels:
            w1, b1 = fc(se_channels, filters)
            w2, b2 = fc(2 * filters, se_channels)
            blk["se"] = {"w1": w1, "b1": b1, "w2": w2, "b2": b2}
        w["residual"].append(blk)
    if attn_policy:
        pe, pd, n_enc, enc_heads, enc_dff = attn_policy
        w["ip_pol_w"], w["ip_pol_b"] = fc(pe, filters)
        w["pol_encoder"] = [_encoder_layer(g, pe, pe, enc_dff, pe ** -0.5, bias_std, perturb_ln=True)
                            for _ in range(n_enc)]
        w["pol_headcount"] = enc_heads
        w["ip2_pol_w"], w["ip2_pol_b"] = fc(pd, pe)
        w["ip3_pol_w"], w["ip3_pol_b"] = fc(pd, pe)
        w["ip4_pol_w"] = g.normal((4, pd), pd ** -0.5)
    elif conv_policy:
        w["policy1"] = conv(filters, filters, 3)
        w["policy"] = conv(80, filters, 3)
    else:
        w["policy"] = conv(policy_channels, filters, 1)
        w["ip_pol_w"], w["ip_pol_b"] = fc(1858, policy_channels * 64)
    w["value"] = conv(value_channels, filters, 1)
    w["ip1_val_w"], w["ip1_val_b"] = fc(value_fc, value_channels * 64)
    w["ip2_val_w"], w["ip2_val_b"] = fc(3, value_fc)
    if moves_left:
        w["moves_left"] = conv(8, filters, 1)
        w["ip1_mov_w"], w["ip1_mov_b"] = fc(value_fc, 8 * 64)
        w["ip2_mov_w"], w["ip2_mov_b"] = fc(1, value_fc)
    nf = {"input": INPUT_CLASSICAL_112_PLANE, "output": OUTPUT_WDL,
          "network": NETWORK_SE_WITH_HEADFORMAT,
          "policy": POLICY_ATTENTION if attn_policy else POLICY_CONVOLUTION if conv_policy else POLICY_CLASSICAL,
          "value": VALUE_WDL,
          "moves_left": MOVES_LEFT_V1 if moves_left else MOVES_LEFT_NONE,
          "default_activation": DEFAULT_ACTIVATION_RELU}
    return {"format": {"weights_encoding": netproto.LINEAR16, "network_format": nf}, "weights": w}


def attention_body(emb, layers, heads, dff, seed, smolgen=None, std=0.02, bias_std=0.02,
                   policy_d=None, value_channels=32, value_fc=128, mlh_channels=32, mlh_fc=128,
                   perturb_ln=False, pe_dense=None, gating=False, multihead=False, d_model=None, pol_encoder=None):
    """Attention-body net (attention policy, WDL, MLH).

    smolgen = (hidden_channels, hidden_sz, gen_sz) or None. Weights N(0, std),
    LayerNorm gamma=1 / beta=0 unless perturb_ln (tests).
    pe_dense = (enc_channels, emb_ffn_width): PE_DENSE input embedding with its layer norm and
    embedding FFN (src/neural/backends/blas/network_blas.cc:612-712) instead of PE_MAP.
    gating: ip_mult_gate / ip_add_gate. multihead: network format 7 with policy heads
    vanilla / optimistic_st / soft (shared embedding) and value heads winner / q / st.
    pol_encoder = (layers, heads, dff[, smolgen]): encoder layers inside the policy head (legacy format only);
    their optional smolgen = (hidden_channels, hidden_sz, gen_sz) shares the net's smolgen_w, so gen_sz must be
    the body's.
    """
    g = _Gen(seed)
    d_model = d_model or emb          # heads * head depth
    policy_d = policy_d or emb

    def fc(cout, cin, bias=True):
        w = g.normal((cout, cin), std)
        return (w, g.normal((cout,), bias_std)) if bias else w

    def ln(n):
        if perturb_ln:
            return 1.0 + g.normal((n,), 0.1), g.normal((n,), 0.1)
        return np.ones(n, np.float32), np.zeros(n, np.float32)

    w = {}
    if pe_dense:
        enc_ch, emb_dff = pe_dense
        w["ip_emb_preproc_w"], w["ip_emb_preproc_b"] = fc(64 * enc_ch, 64 * 12)
        w["ip_emb_w"], w["ip_emb_b"] = fc(emb, 112 + enc_ch)
        w["ip_emb_ln_gammas"], w["ip_emb_ln_betas"] = ln(emb)
        w["ip_emb_ffn"] = {}
        w["ip_emb_ffn"]["dense1_w"], w["ip_emb_ffn"]["dense1_b"] = fc(emb_dff, emb)
        w["ip_emb_ffn"]["dense2_w"], w["ip_emb_ffn"]["dense2_b"] = fc(emb, emb_dff)
        w["ip_emb_ffn_ln_gammas"], w["ip_emb_ffn_ln_betas"] = ln(emb)
    else:
        w["ip_emb_w"], w["ip_emb_b"] = fc(emb, 112 + 64)
    if gating:
        w["ip_mult_gate"] = 1.0 + g.normal((emb * 64,), 0.1)
        w["ip_add_gate"] = g.normal((emb * 64,), 0.1)
    w["encoder"] = [_encoder_layer(g, emb, d_model, dff, std, bias_std, smolgen=smolgen, heads=heads,
                                   perturb_ln=perturb_ln) for _ in range(layers)]
    w["headcount"] = heads

    def policy_head():
        h = {}
        h["ip2_pol_w"], h["ip2_pol_b"] = fc(policy_d, policy_d)
        h["ip3_pol_w"], h["ip3_pol_b"] = fc(policy_d, policy_d)
        h["ip4_pol_w"] = fc(4, policy_d, bias=False)
        return h

    def value_head():
        h = {}
        h["ip_val_w"], h["ip_val_b"] = fc(value_channels, emb)
        h["ip1_val_w"], h["ip1_val_b"] = fc(value_fc, 64 * value_channels)
        h["ip2_val_w"], h["ip2_val_b"] = fc(3, value_fc)
        return h

    if multihead:
        ph = {}
        ph["ip_pol_w"], ph["ip_pol_b"] = fc(policy_d, emb)
        for name in ("vanilla", "optimistic_st", "soft"):
            ph[name] = policy_head()
        w["policy_heads"] = ph
        w["value_heads"] = {name: value_head() for name in ("winner", "q", "st")}
    else:
        w["ip_pol_w"], w["ip_pol_b"] = fc(policy_d, emb)
        if pol_encoder:
            n_enc, enc_heads, enc_dff = pol_encoder[:3]
            enc_smolgen = pol_encoder[3] if len(pol_encoder) > 3 else None
            w["pol_encoder"] = [_encoder_layer(g, policy_d, policy_d, enc_dff, std, bias_std, smolgen=enc_smolgen,
                                               heads=enc_heads, perturb_ln=perturb_ln) for _ in range(n_enc)]
            w["pol_headcount"] = enc_heads
        w.update(policy_head())
        w.update(value_head())
    w["ip_mov_w"], w["ip_mov_b"] = fc(mlh_channels, emb)
    w["ip1_mov_w"], w["ip1_mov_b"] = fc(mlh_fc, 64 * mlh_channels)
    w["ip2_mov_w"], w["ip2_mov_b"] = fc(1, mlh_fc)
    if smolgen:
        w["smolgen_w"] = fc(64 * 64, smolgen[2], bias=False)
    nf = {"input": INPUT_CLASSICAL_112_PLANE, "output": OUTPUT_WDL,
          "network": NETWORK_ATTENTIONBODY_WITH_MULTIHEADFORMAT if multihead else NETWORK_ATTENTIONBODY_WITH_HEADFORMAT,
          "policy": POLICY_ATTENTION,
          "value": VALUE_WDL, "moves_left": MOVES_LEFT_V1,
          "default_activation": DEFAULT_ACTIVATION_MISH,
          "smolgen_activation": ACTIVATION_SWISH if smolgen else ACTIVATION_DEFAULT,
          "ffn_activation": ACTIVATION_DEFAULT,
          "input_embedding": INPUT_EMBEDDING_PE_DENSE if pe_dense else INPUT_EMBEDDING_PE_MAP}
    return {"format": {"weights_encoding": netproto.LINEAR16, "network_format": nf}, "weights": w}


def _with_input_format(net, input_format):
    net["format"]["network_format"]["input"] = input_format
    return net


def with_batch_norm(net, seed):
    """Adds batch-norm statistics to every convolution block, the form older nets are stored in
    (src/neural/network_legacy.cc:62-131 folds them at load). The first residual block's conv1 takes the oldest
    form: no biases and no gammas/betas; its conv2 has biases but no gammas/betas."""
    g = _Gen(seed)

    def bn(block, old=0):
        n = block["biases"].size
        block["bn_means"] = g.normal((n,), 0.1)
        block["bn_stddivs"] = (0.5 + g.rng.random(n)).astype(np.float32)
        if old == 0:
            block["bn_gammas"] = 1.0 + g.normal((n,), 0.1)
            block["bn_betas"] = g.normal((n,), 0.1)
        if old == 2:
            del block["biases"]

    w = net["weights"]
    bn(w["input"])
    for i, r in enumerate(w["residual"]):
        bn(r["conv1"], old=2 if i == 0 else 0)
        bn(r["conv2"], old=1 if i == 0 else 0)
    for key in ("policy1", "policy", "value", "moves_left"):
        if key in w:
            bn(w[key])
    return net


def with_classical_value(net, seed):
    """Scalar tanh value head (VALUE_CLASSICAL, src/neural/backends/blas/network_blas.cc:763-771)."""
    g = _Gen(seed)
    w = net["weights"]
    fan_in = w["ip2_val_w"].shape[1]
    w["ip2_val_w"] = g.normal((1, fan_in), fan_in ** -0.5)
    w["ip2_val_b"] = g.normal((1,), 0.02)
    net["format"]["network_format"]["value"] = 1
    net["format"]["network_format"]["output"] = 1
    return net


def _old_format(net, network=None, drop=()):
    """Rewrites the format block the way files written before a format revision look; the loader's
    FixOlderWeightsFile (src/neural/loader.cc:108-158) has one branch per case."""
    nf = net["format"]["network_format"]
    if network is None:
        del net["format"]["network_format"]
    else:
        nf["network"] = network
        for key in drop:
            nf.pop(key, None)
    return net


# The benchmark configurations (name -> builder). Seeds are part of the spec.
CONFIGS = {
    # 6 blocks x 64 filters SE-ResNet, SE ratio 4, classical policy, WDL.
    "c0_resnet_6x64": lambda: se_resnet(64, 6, 16, seed=1000),
    # 10-layer d=256 attention body, 8 heads, dff 1024, no smolgen.
    "c1_attn_10x256": lambda: attention_body(256, 10, 8, 1024, seed=1001),
    # BT4 shape: 15 layers, d=1024, 32 heads, dff 1536, smolgen 32/256/256.
    "c2_bt4_15x1024": lambda: attention_body(1024, 15, 32, 1536, seed=1002, smolgen=(32, 256, 256)),
    # 20 blocks x 256 filters SE-ResNet, SE ratio 4.
    "c3_resnet_20x256": lambda: se_resnet(256, 20, 64, seed=1003),
    # tiny nets for fast parity tests
    "tiny_resnet": lambda: se_resnet(32, 2, 8, seed=2000, moves_left=True),
    "tiny_resnet_convpolicy": lambda: se_resnet(32, 2, 8, seed=2003, conv_policy=True),
    "tiny_resnet_nose": lambda: se_resnet(24, 3, 0, seed=2004, moves_left=True),
    # 40 filters with SE: a channel count that is not a multiple of 16 (separate transform kernels)
    "tiny_resnet_40se": lambda: se_resnet(40, 2, 8, seed=2009, moves_left=True),
    # (std 0.1 instead of 0.02: at width 64 that gives policy logits of order 0.1-1, so absolute
    # tolerances in the parity tests mean something)
    "tiny_attn": lambda: attention_body(64, 2, 2, 96, seed=2001, smolgen=(8, 32, 32), perturb_ln=True, std=0.1),
    # smallest shape the fp8 configuration accepts (all widths multiples of 128)
    "tiny_attn_f8": lambda: attention_body(128, 3, 4, 256, seed=2005, smolgen=(8, 32, 32), perturb_ln=True, std=0.07),
    # the same with smolgen widths the fp8 form of the smolgen chain accepts (multiples of 128)
    "tiny_attn_f8_sg": lambda: attention_body(128, 2, 4, 256, seed=2021, smolgen=(8, 128, 128), perturb_ln=True, std=0.07),
    # modern format: dense position encoding + embedding FFN, input gating, multi-head format
    "tiny_attn_dense": lambda: attention_body(64, 2, 2, 96, seed=2006, smolgen=(8, 32, 32), perturb_ln=True,
                                              pe_dense=(16, 128), gating=True, multihead=True, std=0.1),
    # BT4 as published: 15 layers, d=1024, 32 heads, dff 1536, smolgen, PE_DENSE (64 channels, FFN 1536), multi-head
    "bt4_dense_15x1024": lambda: attention_body(1024, 15, 32, 1536, seed=1004, smolgen=(32, 256, 256),
                                                pe_dense=(64, 1536), multihead=True),
    # head depth 64 (d_model 128 over 2 heads) and two encoder layers inside the policy head
    "tiny_attn_d64": lambda: attention_body(128, 2, 2, 128, seed=2007, smolgen=(8, 32, 32), perturb_ln=True, std=0.07,
                                            pol_encoder=(2, 4, 96)),
    # convolutional body with the attention policy head and one policy encoder layer
    "tiny_resnet_attnpolicy": lambda: se_resnet(32, 2, 8, seed=2008, attn_policy=(64, 64, 1, 2, 96)),
    # fp8-capable widths with the dense position encoding, gating and the multi-head format
    "tiny_attn_dense_f8": lambda: attention_body(128, 2, 4, 256, seed=2010, smolgen=(8, 32, 32), perturb_ln=True, std=0.07,
                                                 pe_dense=(16, 128), gating=True, multihead=True),
    # head depth 48: none of the depths the matrix-core attention kernel takes
    "tiny_attn_d48": lambda: attention_body(96, 2, 2, 128, seed=2022, smolgen=(8, 32, 32), perturb_ln=True, std=0.08),
    # smolgen inside the policy head's encoder layer as well (it shares the body's generator layer)
    "tiny_attn_polenc_sg": lambda: attention_body(64, 2, 2, 96, seed=2023, smolgen=(8, 32, 32), perturb_ln=True, std=0.1,
                                                  pol_encoder=(1, 2, 96, (8, 32, 32))),
    # 24 heads of depth 32 at a width that is not a power of two (the shape family of the T78 / T82 nets), a few layers
    "mid_attn_4x768": lambda: attention_body(768, 4, 24, 1024, seed=2024, smolgen=(32, 256, 256), perturb_ln=True,
                                             std=0.03),
    "tiny_attn_nosmolgen": lambda: attention_body(64, 2, 2, 128, seed=2002, perturb_ln=True, std=0.1),
    # ---- what real files contain beyond FLOAT32 layers of the current format ----
    # batch-norm statistics on every convolution block, incl. the bias-less and gamma-less old forms
    "tiny_resnet_bn": lambda: with_batch_norm(se_resnet(32, 2, 8, seed=2012, moves_left=True), seed=3012),
    "tiny_resnet_convpolicy_bn": lambda: with_batch_norm(se_resnet(32, 2, 8, seed=2013, conv_policy=True), seed=3013),
    # scalar tanh value head
    "tiny_resnet_classical_value": lambda: with_classical_value(se_resnet(32, 2, 8, seed=2014), seed=3014),
    # no network_format at all: plain residual tower, classical heads (loader.cc:115-121)
    "old_noformat": lambda: _old_format(with_classical_value(se_resnet(24, 2, 0, seed=2015), seed=3015)),
    # NETWORK_CLASSICAL (1) and NETWORK_SE (2): head formats are implied (loader.cc:122-132)
    "old_classical": lambda: _old_format(with_classical_value(se_resnet(24, 2, 0, seed=2016), seed=3016), network=1,
                                         drop=("policy", "value")),
    "old_se": lambda: _old_format(with_batch_norm(with_classical_value(se_resnet(24, 2, 8, seed=2017), seed=3017), seed=4017),
                                  network=2, drop=("policy", "value")),
    # attention body stored as SE_WITH_HEADFORMAT with smolgen: squared-ReLU FFN and swish are implied (:133-142)
    "old_attn_as_se": lambda: _old_format(
        attention_body(64, 2, 2, 96, seed=2018, smolgen=(8, 32, 32), perturb_ln=True, std=0.1), network=4,
        drop=("smolgen_activation", "ffn_activation", "input_embedding")),
    # NETWORK_AB_LEGACY_WITH_MULTIHEADFORMAT (134) (:143-145)
    "old_ab_legacy": lambda: _old_format(
        attention_body(64, 2, 2, 96, seed=2019, smolgen=(8, 32, 32), perturb_ln=True, pe_dense=(16, 128),
                       multihead=True, std=0.1), network=134),
    # format 6 carrying policy_heads and value_heads: becomes format 7 with PE_DENSE (:148-154)
    "old_format6_with_heads": lambda: _old_format(
        attention_body(64, 2, 2, 96, seed=2020, smolgen=(8, 32, 32), perturb_ln=True, pe_dense=(16, 128),
                       multihead=True, std=0.1), network=6, drop=("input_embedding",)),
    # canonical input format with hectoplies: board transforms, en-passant plane, fractional rule-50 plane values
    "tiny_attn_canonical": lambda: _with_input_format(
        attention_body(64, 2, 2, 96, seed=2011, smolgen=(8, 32, 32), perturb_ln=True, std=0.1),
        INPUT_112_WITH_CANONICALIZATION_HECTOPLIES),
}


# Part of the cache file name: bump when a generator or a configuration changes.
CACHE_VERSION = "-g4"


ENCODINGS = {"float32": netproto.FLOAT32, "linear16": netproto.LINEAR16, "float16": netproto.FLOAT16,
             "bfloat16": netproto.BFLOAT16}


def write_config(name, path, encoding="float32"):
    """Generates config `name` into `path` (a .pb.gz) with every layer stored in `encoding`
    (Weights.Layer.Encoding, proto/net.proto:42-48; real lc0 files use LINEAR16); returns the path."""
    net = CONFIGS[name]()
    netproto.write_pb_gz(path, net, layer_encoding=ENCODINGS[encoding])
    return path


def cached_config(name, cache_dir=None, encoding="float32"):
    """Path of the generated file for `name`, generating it on first use."""
    cache_dir = cache_dir or os.environ.get("LC0MI_NET_CACHE", "/tmp/lc0mi_nets")
    os.makedirs(cache_dir, exist_ok=True)
    suffix = "" if encoding == "float32" else "-" + encoding
    path = os.path.join(cache_dir, name + suffix + CACHE_VERSION + ".pb.gz")
    if not os.path.exists(path):
        tmp = path + ".tmp%d" % os.getpid()
        write_config(name, tmp, encoding)
        os.replace(tmp, path)
    return path
