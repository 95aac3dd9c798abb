"""TEST INFRASTRUCTURE -- independent reader of lc0 weight files for the CPU
oracle: gzip -> protobuf wire walk -> float32 numpy weights with the same
resolution rules as the reference.

Follows (reference file:line):
  DecompressGzip / ParseWeightsProto / FixOlderWeightsFile  src/neural/loader.cc:59-212
  LayerAdapter decode                                       src/utils/weights_adapter.cc:38-80
  BaseWeights / ConvBlock (BN fold) / MultiHeadWeights      src/neural/network_legacy.cc:33-307
  field numbers                                             proto/net.proto:31-411

Pinned by: round trip against the independent writer in lc0_amd/netproto.py,
the LINEAR16/FLOAT16/BFLOAT16 closed forms and the batch-norm fold identity
(tests/test_oracle_nn.py).
"""
import gzip
import struct
from types import SimpleNamespace as NS

import numpy as np

WEIGHT_MAGIC = 0x1C0

# NetworkFormat enums (proto/net.proto:275-366)
NETWORK_CLASSICAL, NETWORK_SE = 1, 2
NETWORK_CLASSICAL_WITH_HEADFORMAT, NETWORK_SE_WITH_HEADFORMAT = 3, 4
NETWORK_ATTENTIONBODY_WITH_HEADFORMAT, NETWORK_ATTENTIONBODY_WITH_MULTIHEADFORMAT = 6, 7
NETWORK_AB_LEGACY_WITH_MULTIHEADFORMAT = 134
POLICY_CLASSICAL, POLICY_CONVOLUTION, POLICY_ATTENTION = 1, 2, 3
VALUE_CLASSICAL, VALUE_WDL = 1, 2
MOVES_LEFT_V1 = 1
INPUT_EMBEDDING_NONE, INPUT_EMBEDDING_PE_MAP, INPUT_EMBEDDING_PE_DENSE = 0, 1, 2
ACT_DEFAULT, ACT_MISH, ACT_RELU, ACT_NONE, ACT_TANH, ACT_SIGMOID, ACT_SELU, ACT_SWISH, ACT_RELU_2 = range(9)


class WeightsError(Exception):
    pass


def _walk(buf):
    """Protobuf wire walk: bytes -> {field number: [raw values]}."""
    out = {}
    pos, n = 0, len(buf)
    while pos < n:
        key = 0
        shift = 0
        while True:
            b = buf[pos]
            pos += 1
            key |= (b & 0x7F) << shift
            shift += 7
            if not b & 0x80:
                break
        num, wt = key >> 3, key & 7
        if wt == 0:
            v = 0
            shift = 0
            while True:
                b = buf[pos]
                pos += 1
                v |= (b & 0x7F) << shift
                shift += 7
                if not b & 0x80:
                    break
        elif wt == 1:
            v = bytes(buf[pos:pos + 8])
            pos += 8
        elif wt == 2:
            ln = 0
            shift = 0
            while True:
                b = buf[pos]
                pos += 1
                ln |= (b & 0x7F) << shift
                shift += 7
                if not b & 0x80:
                    break
            v = buf[pos:pos + ln]
            if len(v) != ln:
                raise WeightsError("truncated protobuf field")
            pos += ln
        elif wt == 5:
            v = bytes(buf[pos:pos + 4])
            pos += 4
        else:
            raise WeightsError("unsupported wire type %d" % wt)
        out.setdefault(num, []).append(v)
    return out


def _sub(tree, num):
    """Last occurrence of an embedded message field, walked; {} if absent."""
    if num not in tree:
        return None
    return _walk(tree[num][-1])


def _uint(tree, num, default=0):
    return tree[num][-1] if tree is not None and num in tree else default


def _layer(tree, num):
    """Weights.Layer -> float32 vector (weights_adapter.cc:38-62); empty if absent."""
    if tree is None or num not in tree:
        return np.zeros(0, np.float32)
    l = _walk(tree[num][-1])
    enc = _uint(l, 4, 1)  # default LINEAR16 (weights_adapter.cc:65-66)
    params = bytes(l[3][-1]) if 3 in l else b""
    lo = struct.unpack("<f", l[1][-1])[0] if 1 in l else 0.0
    hi = struct.unpack("<f", l[2][-1])[0] if 2 in l else 0.0
    if enc == 1:
        theta = np.frombuffer(params, "<u2").astype(np.float32) / np.float32(0xFFFF)
        return (np.float32(lo) * (np.float32(1) - theta) + np.float32(hi) * theta).astype(np.float32)
    if enc == 2:
        return np.frombuffer(params, "<f2").astype(np.float32)
    if enc == 3:
        return (np.frombuffer(params, "<u2").astype(np.uint32) << 16).view(np.float32).copy()
    if enc == 4:
        return np.frombuffer(params, "<f4").astype(np.float32)
    raise WeightsError("Unknown layer encoding %d" % enc)


def _conv_block(tree, num):
    """ConvBlock with batch norm folded (network_legacy.cc:78-133)."""
    t = _sub(tree, num) if tree is not None else None
    w = _layer(t, 1)
    b = _layer(t, 2)
    means, stddivs = _layer(t, 3), _layer(t, 4)
    gammas, betas = _layer(t, 5), _layer(t, 6)
    cb = NS(weights=w, biases=b)
    if w.size == 0:
        return cb
    if betas.size == 0:
        betas = np.zeros(means.size, np.float32)
        gammas = np.ones(means.size, np.float32)
    if b.size == 0:
        b = np.zeros(means.size, np.float32)
    if means.size == 0:
        cb.biases = b
        return cb
    gammas = gammas * (np.float32(1.0) / np.sqrt(stddivs + np.float32(1e-5)))
    means = means - b
    outputs = b.size
    w = (w.reshape(outputs, -1) * gammas[:, None]).reshape(-1).astype(np.float32)
    cb.weights = w
    cb.biases = (-gammas * means + betas).astype(np.float32)
    return cb


def _ffn(t):
    return NS(dense1_w=_layer(t, 1), dense1_b=_layer(t, 2), dense2_w=_layer(t, 3), dense2_b=_layer(t, 4))


def _encoder_layer(raw):
    t = _walk(raw)
    m = _sub(t, 1) or {}
    if 10 in m or 11 in m or 12 in m:
        raise WeightsError("RPE weights file not supported.")
    s = _sub(m, 9)
    mha = NS(q_w=_layer(m, 1), q_b=_layer(m, 2), k_w=_layer(m, 3), k_b=_layer(m, 4),
             v_w=_layer(m, 5), v_b=_layer(m, 6), dense_w=_layer(m, 7), dense_b=_layer(m, 8),
             has_smolgen=s is not None,
             smolgen=NS(compress=_layer(s, 1), dense1_w=_layer(s, 2), dense1_b=_layer(s, 3),
                        ln1_gammas=_layer(s, 4), ln1_betas=_layer(s, 5), dense2_w=_layer(s, 6),
                        dense2_b=_layer(s, 7), ln2_gammas=_layer(s, 8), ln2_betas=_layer(s, 9)))
    return NS(mha=mha, ln1_gammas=_layer(t, 2), ln1_betas=_layer(t, 3), ffn=_ffn(_sub(t, 4)),
              ln2_gammas=_layer(t, 5), ln2_betas=_layer(t, 6))


def _policy_head(t, shared_w, shared_b):
    """MultiHeadWeights::PolicyHead (network_legacy.cc:177-194); t may be None."""
    own_w, own_b = _layer(t, 1), _layer(t, 2)
    return NS(ip_pol_w=own_w if own_w.size else shared_w, ip_pol_b=own_b if own_b.size else shared_b,
              policy1=_conv_block(t, 10), policy=_conv_block(t, 11),
              ip2_pol_w=_layer(t, 3), ip2_pol_b=_layer(t, 4), ip3_pol_w=_layer(t, 5),
              ip3_pol_b=_layer(t, 6), ip4_pol_w=_layer(t, 7),
              pol_encoder=[_encoder_layer(r) for r in (t or {}).get(8, [])],
              pol_encoder_head_count=_uint(t, 9))


def _value_head(t):
    return NS(value=_conv_block(t, 11), ip_val_w=_layer(t, 1), ip_val_b=_layer(t, 2),
              ip1_val_w=_layer(t, 3), ip1_val_b=_layer(t, 4), ip2_val_w=_layer(t, 5),
              ip2_val_b=_layer(t, 6))


def _multi_head_weights(w):
    """pblczero.Weights tree -> MultiHeadWeights (network_legacy.cc:33-76,232-307)."""
    W = NS()
    W.input = _conv_block(w, 1)
    W.residual = []
    for raw in w.get(2, []):
        r = _walk(raw)
        s = _sub(r, 3)
        W.residual.append(NS(conv1=_conv_block(r, 1), conv2=_conv_block(r, 2), has_se=s is not None,
                             se=NS(w1=_layer(s, 1), b1=_layer(s, 2), w2=_layer(s, 3), b2=_layer(s, 4))))
    for name, num in [("ip_emb_preproc_w", 37), ("ip_emb_preproc_b", 38), ("ip_emb_w", 25),
                      ("ip_emb_b", 26), ("ip_emb_ln_gammas", 39), ("ip_emb_ln_betas", 40),
                      ("ip_mult_gate", 33), ("ip_add_gate", 34), ("ip_emb_ffn_ln_gammas", 42),
                      ("ip_emb_ffn_ln_betas", 43), ("ip_mov_w", 31), ("ip_mov_b", 32),
                      ("ip1_mov_w", 13), ("ip1_mov_b", 14), ("ip2_mov_w", 15), ("ip2_mov_b", 16),
                      ("smolgen_w", 35)]:
        setattr(W, name, _layer(w, num))
    W.ip_emb_ffn = _ffn(_sub(w, 41))
    W.moves_left = _conv_block(w, 12)
    W.has_smolgen = 35 in w
    W.encoder_head_count = _uint(w, 28)
    W.encoder = [_encoder_layer(r) for r in w.get(27, [])]

    ph = _sub(w, 45)
    shared_w = _layer(ph, 1) if ph is not None and 1 in ph else _layer(w, 4)
    shared_b = _layer(ph, 2) if ph is not None and 2 in ph else _layer(w, 5)
    W.policy_heads = {"vanilla": _policy_head(_sub(ph, 3) if ph else None, shared_w, shared_b)}
    if ph is not None:
        for name, num in [("optimistic", 4), ("soft", 5), ("opponent", 6)]:
            if num in ph:
                W.policy_heads[name] = _policy_head(_sub(ph, num), shared_w, shared_b)
    else:
        if 3 in w or 11 in w or 4 in w:
            v = W.policy_heads["vanilla"]
            v.policy1 = _conv_block(w, 11)
            v.policy = _conv_block(w, 3)
            v.ip2_pol_w, v.ip2_pol_b = _layer(w, 17), _layer(w, 18)
            v.ip3_pol_w, v.ip3_pol_b = _layer(w, 19), _layer(w, 20)
            v.ip4_pol_w = _layer(w, 22)
            v.pol_encoder_head_count = _uint(w, 24)
            v.pol_encoder = [_encoder_layer(r) for r in w.get(21, [])]
        else:
            raise WeightsError("Could not find valid policy head weights.")

    vh = _sub(w, 44)
    W.value_heads = {"winner": _value_head(_sub(vh, 1) if vh else None)}
    if vh is not None:
        for name, num in [("q", 2), ("st", 3)]:
            if num in vh:
                W.value_heads[name] = _value_head(_sub(vh, num))
    else:
        if 6 in w or 29 in w:
            win = W.value_heads["winner"]
            win.value = _conv_block(w, 6)
            win.ip_val_w, win.ip_val_b = _layer(w, 29), _layer(w, 30)
            win.ip1_val_w, win.ip1_val_b = _layer(w, 7), _layer(w, 8)
            win.ip2_val_w, win.ip2_val_b = _layer(w, 9), _layer(w, 10)
        else:
            raise WeightsError("Could not find valid value head weights.")
    return W


def _version_int(major, minor, patch):
    return major * 1000000 + minor * 1000 + patch


def parse_net(buf):
    """Raw protobuf bytes -> NS(format=NS(...), weights=MultiHeadWeights)."""
    net = _walk(memoryview(buf))
    magic = struct.unpack("<I", net[1][-1])[0] if 1 in net else 0
    if magic != WEIGHT_MAGIC:
        raise WeightsError("Invalid weight file: bad header.")
    mv = _sub(net, 3) or {}
    net_ver = _version_int(_uint(mv, 1), _uint(mv, 2), _uint(mv, 3))
    fmt = _sub(net, 4) or {}
    nf_tree = _sub(fmt, 2)
    has_nf = nf_tree is not None
    nf_tree = nf_tree or {}
    nf = NS(input=_uint(nf_tree, 1), output=_uint(nf_tree, 2), network=_uint(nf_tree, 3),
            policy=_uint(nf_tree, 4), value=_uint(nf_tree, 5), moves_left=_uint(nf_tree, 6),
            default_activation=_uint(nf_tree, 7), smolgen_activation=_uint(nf_tree, 8),
            ffn_activation=_uint(nf_tree, 9), input_embedding=_uint(nf_tree, 10),
            has_input_embedding=10 in nf_tree)
    w = _sub(net, 10)
    has_weights = w is not None
    w = w or {}
    # FixOlderWeightsFile (loader.cc:108-158)
    if not has_nf:
        nf.input, nf.output = 1, 1
        nf.network, nf.value, nf.policy = NETWORK_CLASSICAL_WITH_HEADFORMAT, VALUE_CLASSICAL, POLICY_CLASSICAL
    elif nf.network == NETWORK_CLASSICAL:
        nf.network, nf.value, nf.policy = NETWORK_CLASSICAL_WITH_HEADFORMAT, VALUE_CLASSICAL, POLICY_CLASSICAL
    elif nf.network == NETWORK_SE:
        nf.network, nf.value, nf.policy = NETWORK_SE_WITH_HEADFORMAT, VALUE_CLASSICAL, POLICY_CLASSICAL
    elif nf.network == NETWORK_SE_WITH_HEADFORMAT and len(w.get(27, [])) > 0:
        nf.network = NETWORK_ATTENTIONBODY_WITH_HEADFORMAT
        if 35 in w:
            nf.ffn_activation, nf.smolgen_activation = ACT_RELU_2, ACT_SWISH
    elif nf.network == NETWORK_AB_LEGACY_WITH_MULTIHEADFORMAT:
        nf.network = NETWORK_ATTENTIONBODY_WITH_MULTIHEADFORMAT
    if nf.network == NETWORK_ATTENTIONBODY_WITH_HEADFORMAT:
        if 45 in w and 44 in w:
            nf.network = NETWORK_ATTENTIONBODY_WITH_MULTIHEADFORMAT
            nf.input_embedding, nf.has_input_embedding = INPUT_EMBEDDING_PE_DENSE, True
        if not nf.has_input_embedding:
            nf.input_embedding, nf.has_input_embedding = INPUT_EMBEDDING_PE_MAP, True
    if net_ver != 0x5C99973 and net_ver > _version_int(0, 33, 0):
        raise WeightsError("Invalid weight file: lc0 version >= %d.%d.%d required." %
                           (_uint(mv, 1), _uint(mv, 2), _uint(mv, 3)))
    if has_weights and _uint(fmt, 1) != 1 and net_ver < _version_int(0, 33, 0):
        raise WeightsError("Invalid weight file: unsupported encoding.")
    return NS(format=nf, weights=_multi_head_weights(w))


def load(path):
    with gzip.open(path, "rb") as f:
        buf = f.read()
    if len(buf) < 2:
        raise WeightsError("Invalid weight file: too small.")
    return parse_net(buf)
