"""Writer for lc0 weight files (`.pb.gz` = gzip(protobuf pblczero.Net)).

Only what is needed to emit networks a real lc0 can load: the protobuf wire
encoder and the message/field numbers of proto/net.proto:31-411.  A network is
described as nested dicts keyed by the proto field names; numpy arrays become
`Weights.Layer` messages with FLOAT32 encoding (net.proto:38-51).
"""
import gzip
import struct

import numpy as np

WEIGHT_MAGIC = 0x1C0  # src/neural/loader.cc:57

# Layer.Encoding (net.proto:42-48)
LINEAR16, FLOAT16, BFLOAT16, FLOAT32 = 1, 2, 3, 4

# message name -> field name -> (number, kind); kind is a scalar kind or the
# name of a nested message; a leading '*' marks a repeated field.
SCHEMA = {
    "Net": {"magic": (1, "fixed32"), "license": (2, "string"), "min_version": (3, "EngineVersion"),
            "format": (4, "Format"), "weights": (10, "Weights")},
    "EngineVersion": {"major": (1, "uint"), "minor": (2, "uint"), "patch": (3, "uint")},
    "Format": {"weights_encoding": (1, "uint"), "network_format": (2, "NetworkFormat")},
    "NetworkFormat": {"input": (1, "uint"), "output": (2, "uint"), "network": (3, "uint"),
                      "policy": (4, "uint"), "value": (5, "uint"), "moves_left": (6, "uint"),
                      "default_activation": (7, "uint"), "smolgen_activation": (8, "uint"),
                      "ffn_activation": (9, "uint"), "input_embedding": (10, "uint")},
    "Layer": {"min_val": (1, "float"), "max_val": (2, "float"), "params": (3, "bytes"),
              "encoding": (4, "uint"), "dims": (5, "*uint")},
    "ConvBlock": {"weights": (1, "Layer"), "biases": (2, "Layer"), "bn_means": (3, "Layer"),
                  "bn_stddivs": (4, "Layer"), "bn_gammas": (5, "Layer"), "bn_betas": (6, "Layer")},
    "SEunit": {"w1": (1, "Layer"), "b1": (2, "Layer"), "w2": (3, "Layer"), "b2": (4, "Layer")},
    "Residual": {"conv1": (1, "ConvBlock"), "conv2": (2, "ConvBlock"), "se": (3, "SEunit")},
    "Smolgen": {"compress": (1, "Layer"), "dense1_w": (2, "Layer"), "dense1_b": (3, "Layer"),
                "ln1_gammas": (4, "Layer"), "ln1_betas": (5, "Layer"), "dense2_w": (6, "Layer"),
                "dense2_b": (7, "Layer"), "ln2_gammas": (8, "Layer"), "ln2_betas": (9, "Layer")},
    "MHA": {"q_w": (1, "Layer"), "q_b": (2, "Layer"), "k_w": (3, "Layer"), "k_b": (4, "Layer"),
            "v_w": (5, "Layer"), "v_b": (6, "Layer"), "dense_w": (7, "Layer"),
            "dense_b": (8, "Layer"), "smolgen": (9, "Smolgen"), "rpe_q": (10, "Layer"),
            "rpe_k": (11, "Layer"), "rpe_v": (12, "Layer")},
    "FFN": {"dense1_w": (1, "Layer"), "dense1_b": (2, "Layer"), "dense2_w": (3, "Layer"),
            "dense2_b": (4, "Layer")},
    "EncoderLayer": {"mha": (1, "MHA"), "ln1_gammas": (2, "Layer"), "ln1_betas": (3, "Layer"),
                     "ffn": (4, "FFN"), "ln2_gammas": (5, "Layer"), "ln2_betas": (6, "Layer")},
    "PolicyHead": {"ip_pol_w": (1, "Layer"), "ip_pol_b": (2, "Layer"), "ip2_pol_w": (3, "Layer"),
                   "ip2_pol_b": (4, "Layer"), "ip3_pol_w": (5, "Layer"), "ip3_pol_b": (6, "Layer"),
                   "ip4_pol_w": (7, "Layer"), "pol_encoder": (8, "*EncoderLayer"),
                   "pol_headcount": (9, "uint"), "policy1": (10, "ConvBlock"),
                   "policy": (11, "ConvBlock")},
    "ValueHead": {"ip_val_w": (1, "Layer"), "ip_val_b": (2, "Layer"), "ip1_val_w": (3, "Layer"),
                  "ip1_val_b": (4, "Layer"), "ip2_val_w": (5, "Layer"), "ip2_val_b": (6, "Layer"),
                  "ip_val_err_w": (7, "Layer"), "ip_val_err_b": (8, "Layer"),
                  "value": (11, "ConvBlock")},
    "PolicyHeads": {"ip_pol_w": (1, "Layer"), "ip_pol_b": (2, "Layer"), "vanilla": (3, "PolicyHead"),
                    "optimistic_st": (4, "PolicyHead"), "soft": (5, "PolicyHead"),
                    "opponent": (6, "PolicyHead")},
    "ValueHeads": {"winner": (1, "ValueHead"), "q": (2, "ValueHead"), "st": (3, "ValueHead")},
    "Weights": {"input": (1, "ConvBlock"), "residual": (2, "*Residual"),
                "ip_emb_preproc_w": (37, "Layer"), "ip_emb_preproc_b": (38, "Layer"),
                "ip_emb_w": (25, "Layer"), "ip_emb_b": (26, "Layer"),
                "ip_emb_ln_gammas": (39, "Layer"), "ip_emb_ln_betas": (40, "Layer"),
                "ip_mult_gate": (33, "Layer"), "ip_add_gate": (34, "Layer"),
                "ip_emb_ffn": (41, "FFN"), "ip_emb_ffn_ln_gammas": (42, "Layer"),
                "ip_emb_ffn_ln_betas": (43, "Layer"),
                "encoder": (27, "*EncoderLayer"), "headcount": (28, "uint"),
                "pol_encoder": (21, "*EncoderLayer"), "pol_headcount": (24, "uint"),
                "policy1": (11, "ConvBlock"), "policy": (3, "ConvBlock"),
                "ip_pol_w": (4, "Layer"), "ip_pol_b": (5, "Layer"),
                "ip2_pol_w": (17, "Layer"), "ip2_pol_b": (18, "Layer"),
                "ip3_pol_w": (19, "Layer"), "ip3_pol_b": (20, "Layer"), "ip4_pol_w": (22, "Layer"),
                "value": (6, "ConvBlock"), "ip_val_w": (29, "Layer"), "ip_val_b": (30, "Layer"),
                "ip1_val_w": (7, "Layer"), "ip1_val_b": (8, "Layer"),
                "ip2_val_w": (9, "Layer"), "ip2_val_b": (10, "Layer"),
                "value_heads": (44, "ValueHeads"), "policy_heads": (45, "PolicyHeads"),
                "moves_left": (12, "ConvBlock"), "ip_mov_w": (31, "Layer"), "ip_mov_b": (32, "Layer"),
                "ip1_mov_w": (13, "Layer"), "ip1_mov_b": (14, "Layer"),
                "ip2_mov_w": (15, "Layer"), "ip2_mov_b": (16, "Layer"),
                "smolgen_w": (35, "Layer"), "smolgen_b": (36, "Layer")},
}


def _varint(v):
    out = bytearray()
    v &= (1 << 64) - 1
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _tag(number, wire_type):
    return _varint((number << 3) | wire_type)


def _f32_to_f16_bits(a):
    return a.astype(np.float16).view(np.uint16)


def _f32_to_bf16_bits(a):
    u = a.astype(np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16  # round to nearest even
    return u.astype(np.uint16)


def encode_layer(arr, encoding=FLOAT32):
    """numpy array -> serialized Weights.Layer body."""
    a = np.ascontiguousarray(arr, dtype=np.float32).reshape(-1)
    body = bytearray()
    if encoding == FLOAT32:
        params = a.astype("<f4").tobytes()
    elif encoding == FLOAT16:
        params = _f32_to_f16_bits(a).astype("<u2").tobytes()
    elif encoding == BFLOAT16:
        params = _f32_to_bf16_bits(a).astype("<u2").tobytes()
    elif encoding == LINEAR16:
        lo, hi = (float(a.min()), float(a.max())) if a.size else (0.0, 0.0)
        span = hi - lo if hi > lo else 1.0
        q = np.rint((a - lo) / span * 65535.0).clip(0, 65535).astype("<u2")
        params = q.tobytes()
        body += _tag(1, 5) + struct.pack("<f", lo)
        body += _tag(2, 5) + struct.pack("<f", hi)
    else:
        raise ValueError("unknown layer encoding %r" % (encoding,))
    body += _tag(3, 2) + _varint(len(params)) + params
    body += _tag(4, 0) + _varint(encoding)
    for d in np.shape(arr):
        body += _tag(5, 0) + _varint(int(d))
    return bytes(body)


def encode_message(msg_name, obj, layer_encoding=FLOAT32):
    """Serializes dict `obj` as message `msg_name` (fields in dict order)."""
    schema = SCHEMA[msg_name]
    out = bytearray()
    for key, val in obj.items():
        if val is None:
            continue
        number, kind = schema[key]
        repeated = kind.startswith("*")
        if repeated:
            kind = kind[1:]
        vals = val if repeated else [val]
        for v in vals:
            if kind == "uint":
                out += _tag(number, 0) + _varint(int(v))
            elif kind == "fixed32":
                out += _tag(number, 5) + struct.pack("<I", int(v))
            elif kind == "float":
                out += _tag(number, 5) + struct.pack("<f", float(v))
            elif kind in ("string", "bytes"):
                data = v.encode() if isinstance(v, str) else bytes(v)
                out += _tag(number, 2) + _varint(len(data)) + data
            elif kind == "Layer":
                if isinstance(v, tuple):  # (array, encoding) overrides the default
                    data = encode_layer(v[0], v[1])
                else:
                    data = encode_layer(v, layer_encoding)
                out += _tag(number, 2) + _varint(len(data)) + data
            else:
                data = encode_message(kind, v, layer_encoding)
                out += _tag(number, 2) + _varint(len(data)) + data
    return bytes(out)


def serialize_net(net, layer_encoding=FLOAT32):
    """dict with keys of message Net -> raw protobuf bytes."""
    full = {"magic": WEIGHT_MAGIC}
    full.update(net)
    return encode_message("Net", full, layer_encoding)


def write_pb_gz(path, net, layer_encoding=FLOAT32, compresslevel=0):
    data = serialize_net(net, layer_encoding)
    with gzip.GzipFile(path, "wb", compresslevel=compresslevel, mtime=0) as f:
        f.write(data)
    return len(data)
