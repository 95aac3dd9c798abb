"""Pins the numpy restatement of the blas backend (oracle/nn.py, oracle/netread.py)
against (a) the compiled self-contained reference translation units in
oracle/_ref when they are built, (b) library routines of torch/scipy and
closed forms, (c) the SHA-256 of the reference's policy tables."""
import ctypes
import hashlib
import os

import numpy as np
import pytest
import torch

from lc0_amd import netgen, netproto
from oracle import netread as nr
from oracle import nn as onn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libref_pieces.so")
f32 = np.float32


@pytest.fixture(scope="module")
def ref():
    if not os.path.exists(REF_SO):
        pytest.skip("oracle/_ref not built (needs the reference tree)")
    l = ctypes.CDLL(REF_SO)
    l.ref_activate.restype = ctypes.c_float
    l.ref_activate.argtypes = [ctypes.c_float, ctypes.c_int]
    l.ref_fast_exp.restype = ctypes.c_float
    l.ref_fast_exp.argtypes = [ctypes.c_float]
    l.ref_softmax.argtypes = [ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
    l.ref_layernorm_skip.argtypes = [ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_float,
                                     ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float]
    l.ref_winograd_filter_transform.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p]
    l.ref_bias_residual.argtypes = [ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p,
                                    ctypes.c_void_p, ctypes.c_int]
    l.ref_activate_se.argtypes = [ctypes.c_size_t, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p,
                                  ctypes.c_float, ctypes.c_void_p, ctypes.c_int]
    l.ref_attn_policy_map.restype = ctypes.POINTER(ctypes.c_short)
    l.ref_conv_policy_map.restype = ctypes.POINTER(ctypes.c_short)
    l.ref_pos_encoding.restype = ctypes.POINTER(ctypes.c_float)
    return l


# ---- tables ---------------------------------------------------------------
def test_policy_tables_match_reference_hashes():
    assert hashlib.sha256(onn.ATTN_POLICY_MAP.astype("<i2").tobytes()).hexdigest() == \
        "2cde8db6b669bd5c89646fab72e1572e440dfaaa41c0cab0beba151538398419"
    assert hashlib.sha256(onn.POS_ENCODING.astype("<f4").tobytes()).hexdigest() == \
        "a6461b73540fadaf6a0480f017077e302d25676521525e6a2f7b32fd5d7dc93d"
    cm = np.full(80 * 64, -1, np.int16)
    cm[:73 * 64] = onn.conv_policy_map()
    assert hashlib.sha256(onn.conv_policy_map().astype("<i2").tobytes()).hexdigest() == \
        "a65b9ce4b8cf3f99c8a98ad8da746ad09f3397b0ef7271a5dab8bee3cf01c94f"
    for m in (onn.ATTN_POLICY_MAP, onn.conv_policy_map()):
        used = m[m >= 0]
        assert len(used) == 1858 and len(set(used.tolist())) == 1858


def test_policy_tables_match_compiled_reference(ref):
    a = np.ctypeslib.as_array(ref.ref_attn_policy_map(), (4288,))
    c = np.ctypeslib.as_array(ref.ref_conv_policy_map(), (4672,))
    p = np.ctypeslib.as_array(ref.ref_pos_encoding(), (64, 64))
    assert (a == onn.ATTN_POLICY_MAP).all() and (c == onn.conv_policy_map()).all()
    assert (p == onn.POS_ENCODING).all()


# ---- activations ----------------------------------------------------------
ACTS = [nr.ACT_MISH, nr.ACT_RELU, nr.ACT_NONE, nr.ACT_TANH, nr.ACT_SIGMOID, nr.ACT_SELU,
        nr.ACT_SWISH, nr.ACT_RELU_2]


def test_activations_vs_compiled_reference(ref):
    x = np.concatenate([np.linspace(-12, 12, 4001), [-0.125, -0.1250001, 0.0, 30.0, -30.0]]).astype(f32)
    for act in ACTS:
        want = np.array([ref.ref_activate(float(v), act) for v in x], f32)
        got = onn.activate(x, act)
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=5e-7, err_msg="act %d" % act)


def test_activations_vs_torch_library():
    x = torch.linspace(-10, 10, 2001, dtype=torch.float64)
    xn = x.numpy().astype(f32)
    F = torch.nn.functional
    for act, fn in [(nr.ACT_MISH, F.mish), (nr.ACT_SWISH, F.silu), (nr.ACT_SELU, F.selu),
                    (nr.ACT_RELU, F.relu), (nr.ACT_SIGMOID, torch.sigmoid), (nr.ACT_TANH, torch.tanh)]:
        np.testing.assert_allclose(onn.activate(xn, act), fn(x).numpy(), rtol=1e-5, atol=2e-6)
    np.testing.assert_allclose(onn.activate(xn, nr.ACT_RELU_2), (F.relu(x) ** 2).numpy(), rtol=1e-6)


def test_softmax_and_layernorm(ref):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((7, 64)).astype(f32) * 5
    want = np.zeros_like(x)
    for i in range(7):
        ref.ref_softmax(64, x[i].ctypes.data, want[i].ctypes.data)
    np.testing.assert_allclose(onn.softmax_rows(x), want, rtol=1e-6, atol=1e-9)
    for skip in (None, rng.standard_normal((5, 48)).astype(f32)):
        d = rng.standard_normal((5, 48)).astype(f32)
        g = rng.standard_normal(48).astype(f32)
        b = rng.standard_normal(48).astype(f32)
        want = d.copy()
        ref.ref_layernorm_skip(5, 48, want.ctypes.data, 0.7, skip.ctypes.data if skip is not None else None,
                               g.ctypes.data, b.ctypes.data, 1e-3)
        got = onn.layer_norm_skip(d, 0.7, skip, g, b, 1e-3)
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_layernorm_vs_torch_library():
    rng = np.random.default_rng(1)
    d = rng.standard_normal((9, 32)).astype(f32)
    s = rng.standard_normal((9, 32)).astype(f32)
    g = rng.standard_normal(32).astype(f32)
    b = rng.standard_normal(32).astype(f32)
    t = torch.from_numpy(d).double() * 0.55 + torch.from_numpy(s).double()
    want = torch.nn.functional.layer_norm(t, (32,), torch.from_numpy(g).double(), torch.from_numpy(b).double(), 1e-6)
    np.testing.assert_allclose(onn.layer_norm_skip(d, 0.55, s, g, b, 1e-6), want.numpy(), rtol=1e-4, atol=1e-5)


def test_se_and_bias_residual_vs_compiled_reference(ref):
    rng = np.random.default_rng(2)
    B, C, K = 3, 8, 4
    x = rng.standard_normal((B, C, 64)).astype(f32)
    res = rng.standard_normal((B, C, 64)).astype(f32)
    bias = rng.standard_normal(C).astype(f32)
    w1, b1 = rng.standard_normal((K, C)).astype(f32), rng.standard_normal(K).astype(f32)
    w2, b2 = rng.standard_normal((2 * C, K)).astype(f32), rng.standard_normal(2 * C).astype(f32)
    got = onn.apply_se_unit(x, bias, res, w1, b1, w2, b2, nr.ACT_RELU)
    # textbook SE: pool -> fc -> relu -> fc -> sigmoid scale + shift; the
    # per-channel activation goes through the reference's own Activate().
    pool = x.astype(np.float64).mean(axis=2) + bias
    h = np.maximum(pool @ w1.T.astype(np.float64) + b1, 0)
    s = h @ w2.T.astype(np.float64) + b2
    gamma = 1 / (1 + np.exp(-s[:, :C]))
    beta = s[:, C:] + gamma * bias
    for b in range(B):
        for c in range(C):
            want = np.zeros(64, f32)
            ref.ref_activate_se(64, float(gamma[b, c]), x[b, c].ctypes.data, res[b, c].ctypes.data,
                                float(beta[b, c]), want.ctypes.data, nr.ACT_RELU)
            np.testing.assert_allclose(got[b, c], want, rtol=1e-4, atol=1e-5)
    data = x.copy()
    ref.ref_bias_residual(B, C, data.ctypes.data, bias.ctypes.data, res.ctypes.data, nr.ACT_MISH)
    np.testing.assert_allclose(onn.activate(res + x + bias[None, :, None], nr.ACT_MISH), data, rtol=1e-5, atol=1e-6)


# ---- winograd -------------------------------------------------------------
def test_winograd_filter_vs_compiled_reference(ref):
    rng = np.random.default_rng(3)
    f = rng.standard_normal((5, 3, 3, 3)).astype(f32)
    want = np.zeros(16 * 5 * 3, f32)
    ref.ref_winograd_filter_transform(f.ctypes.data, 5, 3, want.ctypes.data)
    np.testing.assert_allclose(onn.winograd_filter_transform(f, 5, 3), want, rtol=1e-6, atol=1e-7)


def test_winograd_conv_equals_direct_convolution():
    rng = np.random.default_rng(4)
    B, Cin, Cout = 2, 5, 7
    x = rng.standard_normal((B, Cin, 8, 8)).astype(f32)
    w = rng.standard_normal((Cout, Cin, 3, 3)).astype(f32)
    u = onn.winograd_filter_transform(w, Cout, Cin)
    got = onn.winograd_conv3(x, u, Cin, Cout)
    want = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), padding=1)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-4, atol=1e-4)


def test_conv1x1_and_fc_are_textbook_products():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 6, 64)).astype(f32)
    w = rng.standard_normal((4, 6)).astype(f32)
    want = torch.nn.functional.conv2d(torch.from_numpy(x.reshape(3, 6, 8, 8)), torch.from_numpy(w.reshape(4, 6, 1, 1)))
    np.testing.assert_allclose(onn.conv1x1(x, w, 6, 4).reshape(3, 4, 8, 8), want.numpy(), rtol=1e-5, atol=1e-5)
    xi = rng.standard_normal((5, 11)).astype(f32)
    wf = rng.standard_normal((7, 11)).astype(f32)
    bf = rng.standard_normal(7).astype(f32)
    want = torch.nn.functional.linear(torch.from_numpy(xi), torch.from_numpy(wf), torch.from_numpy(bf))
    np.testing.assert_allclose(onn.fc(xi, wf.reshape(-1), bf, nr.ACT_NONE), want.numpy(), rtol=1e-5, atol=1e-5)
    # no bias -> no activation either (fully_connected_layer.cc:103-105)
    np.testing.assert_allclose(onn.fc(xi, wf, None, nr.ACT_RELU), xi @ wf.T, rtol=1e-6)


def test_encode_planes_bits():
    masks = np.zeros((2, 112), np.uint64)
    vals = np.ones((2, 112), f32)
    masks[0, 3] = np.uint64(1) << np.uint64(63)
    masks[1, 109] = np.uint64(0xFFFFFFFFFFFFFFFF)
    vals[1, 109] = 37.0
    p = onn.encode_planes(masks, vals)
    assert p.shape == (2, 112, 64) and p[0, 3, 63] == 1.0 and p[0].sum() == 1.0
    assert (p[1, 109] == 37.0).all() and p[1].sum() == 37.0 * 64


# ---- weights file ---------------------------------------------------------
def test_writer_reader_round_trip(tmp_path):
    net = netgen.CONFIGS["tiny_attn"]()
    path = str(tmp_path / "t.pb.gz")
    netproto.write_pb_gz(path, net)
    got = nr.load(path)
    w = net["weights"]
    assert got.format.network == 6 and got.format.input_embedding == 1 and got.format.smolgen_activation == 7
    np.testing.assert_array_equal(got.weights.ip_emb_w, w["ip_emb_w"].reshape(-1))
    np.testing.assert_array_equal(got.weights.encoder[1].mha.smolgen.dense2_w,
                                  w["encoder"][1]["mha"]["smolgen"]["dense2_w"].reshape(-1))
    np.testing.assert_array_equal(got.weights.policy_heads["vanilla"].ip4_pol_w, w["ip4_pol_w"].reshape(-1))
    np.testing.assert_array_equal(got.weights.value_heads["winner"].ip2_val_b, w["ip2_val_b"])
    assert got.weights.encoder_head_count == 2 and got.weights.has_smolgen


def test_layer_encodings_and_bn_fold(tmp_path):
    rng = np.random.default_rng(6)
    a = rng.standard_normal(300).astype(f32)
    for enc, tol in [(netproto.FLOAT32, 0), (netproto.FLOAT16, 2e-3), (netproto.BFLOAT16, 1.6e-2),
                     (netproto.LINEAR16, 2e-4)]:
        tree = nr._walk(netproto.encode_message("SEunit", {"w1": (a, enc)}))
        got = nr._layer(tree, 1)
        np.testing.assert_allclose(got, a, rtol=tol, atol=tol)
    # LINEAR16 closed form: min*(1-t)+max*t with t=u16/65535.
    lay = netproto._tag(1, 5) + np.float32(-2).tobytes() + netproto._tag(2, 5) + np.float32(6).tobytes() + \
        netproto._tag(3, 2) + netproto._varint(4) + np.array([0, 65535], "<u2").tobytes()
    got = nr._layer({9: [lay]}, 9)
    np.testing.assert_allclose(got, [-2, 6])
    # BN fold == conv followed by batch norm (eps 1e-5).
    cout, cin = 4, 3
    w = rng.standard_normal((cout, cin, 3, 3)).astype(f32)
    b = rng.standard_normal(cout).astype(f32)
    mean, var = rng.standard_normal(cout).astype(f32), rng.random(cout).astype(f32) + 0.5
    gam, bet = rng.standard_normal(cout).astype(f32), rng.standard_normal(cout).astype(f32)
    blk = netproto.encode_message("Residual", {"conv1": {"weights": w, "biases": b, "bn_means": mean,
                                                         "bn_stddivs": var, "bn_gammas": gam, "bn_betas": bet}})
    cb = nr._conv_block(nr._walk(blk), 1)
    x = torch.randn(2, cin, 8, 8, dtype=torch.float64)
    y = torch.nn.functional.conv2d(x, torch.from_numpy(w).double(), torch.from_numpy(b).double(), padding=1)
    want = torch.nn.functional.batch_norm(y, torch.from_numpy(mean).double(), torch.from_numpy(var).double(),
                                          torch.from_numpy(gam).double(), torch.from_numpy(bet).double(), eps=1e-5)
    got = torch.nn.functional.conv2d(x, torch.from_numpy(cb.weights.reshape(cout, cin, 3, 3)).double(),
                                     torch.from_numpy(cb.biases).double(), padding=1)
    np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-4, atol=1e-4)


def test_loader_errors(tmp_path):
    net = netgen.CONFIGS["tiny_resnet"]()
    raw = bytearray(netproto.serialize_net(net))
    with pytest.raises(nr.WeightsError, match="bad header"):
        nr.parse_net(bytes(raw).replace(b"\xc0\x01\x00\x00", b"\xc1\x01\x00\x00", 1))
    bad = dict(net)
    bad["min_version"] = {"major": 0, "minor": 99, "patch": 0}
    with pytest.raises(nr.WeightsError, match="required"):
        nr.parse_net(netproto.serialize_net(bad))
    parsed = nr.parse_net(bytes(raw))
    with pytest.raises(nr.WeightsError, match="does not exist"):
        onn.BlasNetwork(parsed, policy_head="soft")


# ---- encoder layer and whole nets -----------------------------------------
def _tiny(name):
    return nr.parse_net(netproto.serialize_net(netgen.CONFIGS[name]()))


def test_encoder_layer_vs_torch_attention():
    """One smolgen encoder layer against torch's scaled_dot_product_attention
    (additive float mask = smolgen bias), linear and layer_norm in float64."""
    net = _tiny("tiny_attn")
    bn = onn.BlasNetwork(net)
    w = net.weights
    layer = w.encoder[0]
    emb, H = 64, 2
    rng = np.random.default_rng(7)
    B = 3
    x = rng.standard_normal((B * 64, emb)).astype(f32)
    alpha = 0.8
    got = bn.encoder_layer(x, layer, emb, H, nr.ACT_SWISH, nr.ACT_MISH, alpha, 1e-6)

    T = lambda a, *shape: torch.from_numpy(np.asarray(a)).double().reshape(*shape)
    F = torch.nn.functional
    xt = T(x, B * 64, emb)
    sg = layer.mha.smolgen
    hc, hs, gen = 8, 32, 64
    t = F.linear(xt, T(sg.compress, hc, emb)).reshape(B, 64 * hc)
    t = F.silu(F.linear(t, T(sg.dense1_w, hs, 64 * hc), T(sg.dense1_b, hs)))
    t = F.layer_norm(t, (hs,), T(sg.ln1_gammas, hs), T(sg.ln1_betas, hs), 1e-3)
    t = F.silu(F.linear(t, T(sg.dense2_w, gen, hs), T(sg.dense2_b, gen)))
    t = F.layer_norm(t, (gen,), T(sg.ln2_gammas, gen), T(sg.ln2_betas, gen), 1e-3)
    bias = F.linear(t.reshape(B, H, gen // H), T(w.smolgen_w, 4096, gen // H)).reshape(B, H, 64, 64)
    q = F.linear(xt, T(layer.mha.q_w, emb, emb), T(layer.mha.q_b, emb)).reshape(B, 64, H, emb // H).transpose(1, 2)
    k = F.linear(xt, T(layer.mha.k_w, emb, emb), T(layer.mha.k_b, emb)).reshape(B, 64, H, emb // H).transpose(1, 2)
    v = F.linear(xt, T(layer.mha.v_w, emb, emb), T(layer.mha.v_b, emb)).reshape(B, 64, H, emb // H).transpose(1, 2)
    a = F.scaled_dot_product_attention(q, k, v, attn_mask=bias)
    a = a.transpose(1, 2).reshape(B * 64, emb)
    o = F.linear(a, T(layer.mha.dense_w, emb, emb), T(layer.mha.dense_b, emb))
    x1 = F.layer_norm(o * alpha + xt, (emb,), T(layer.ln1_gammas, emb), T(layer.ln1_betas, emb), 1e-6)
    dff = layer.ffn.dense1_b.size
    h = F.mish(F.linear(x1, T(layer.ffn.dense1_w, dff, emb), T(layer.ffn.dense1_b, dff)))
    h = F.linear(h, T(layer.ffn.dense2_w, emb, dff), T(layer.ffn.dense2_b, emb))
    want = F.layer_norm(h * alpha + x1, (emb,), T(layer.ln2_gammas, emb), T(layer.ln2_betas, emb), 1e-6)
    np.testing.assert_allclose(got, want.numpy(), rtol=2e-4, atol=2e-4)


def _random_inputs(n, seed=11):
    from oracle import chess as oc
    pos = oc.random_positions(n, seed)
    return pos["masks"], pos["values"]


@pytest.mark.parametrize("name", ["tiny_attn", "tiny_attn_nosmolgen", "tiny_resnet"])
def test_whole_net_invariants(name):
    net = _tiny(name)
    bn = onn.BlasNetwork(net)
    masks, values = _random_inputs(6)
    out = bn.forward(masks, values)
    assert out["policy"].shape == (6, 1858) and np.isfinite(out["policy"]).all()
    np.testing.assert_allclose(out["wdl"].sum(axis=1), 1.0, rtol=1e-5)
    assert (out["m"] >= 0).all()
    # batch rows are independent: permuting inputs permutes outputs; chunking
    # by max batch size changes nothing.
    perm = np.array([3, 0, 5, 1, 4, 2])
    out_p = bn.forward(masks[perm], values[perm])
    np.testing.assert_allclose(out_p["policy"], out["policy"][perm], rtol=1e-4, atol=1e-5)
    bn2 = onn.BlasNetwork(net, batch_size=4)
    out_c = bn2.forward(masks, values)
    np.testing.assert_allclose(out_c["policy"], out["policy"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(out_c["wdl"], out["wdl"], rtol=1e-4, atol=1e-6)
    # mlh=false option zeroes the moves-left output (network_blas.cc:1000-1001)
    assert (onn.BlasNetwork(net, mlh=False).forward(masks, values)["m"] == 0).all()


def test_zero_smolgen_weights_equal_no_smolgen():
    g = netgen.CONFIGS["tiny_attn"]()
    g["weights"]["smolgen_w"] = np.zeros_like(g["weights"]["smolgen_w"])
    a = onn.BlasNetwork(nr.parse_net(netproto.serialize_net(g)))
    for layer in g["weights"]["encoder"]:
        del layer["mha"]["smolgen"]
    del g["weights"]["smolgen_w"]
    b = onn.BlasNetwork(nr.parse_net(netproto.serialize_net(g)))
    masks, values = _random_inputs(4)
    np.testing.assert_allclose(a.forward(masks, values)["policy"], b.forward(masks, values)["policy"],
                               rtol=1e-5, atol=1e-6)


def test_attention_policy_promotions_closed_form():
    """With a zero promotion matrix every promotion logit equals the plain
    from->to logit."""
    g = netgen.CONFIGS["tiny_attn_nosmolgen"]()
    g["weights"]["ip4_pol_w"] = np.zeros_like(g["weights"]["ip4_pol_w"])
    bn = onn.BlasNetwork(nr.parse_net(netproto.serialize_net(g)))
    masks, values = _random_inputs(2)
    pol = bn.forward(masks, values)["policy"]
    from oracle import chess as oc
    strs = oc.move_strs()
    idx = {s: i for i, s in enumerate(strs)}
    for s in strs[1792:]:
        np.testing.assert_allclose(pol[:, idx[s]], pol[:, idx[s[:4]]], rtol=1e-6)


def test_attention_policy_promotion_offsets_closed_form():
    """Non-zero promotion matrix (network_blas.cc:874-903). With Wk = 0 every key equals the bias vector c, so
    promotion_offsets[i][j] = c . ip4_pol_w[i] for every file j: the logit of promoting to piece p exceeds the
    plain from->to logit by exactly c . (row p + row 3). Rows chosen so that the three pieces get three
    different shifts: a wrong piece index (3j+p), a missing `+= offsets[3]` or a row mix-up changes them."""
    from oracle import chess as oc
    g = netgen.CONFIGS["tiny_attn_nosmolgen"]()
    w = g["weights"]
    pd = w["ip3_pol_b"].size
    rng = np.random.default_rng(11)
    c = rng.standard_normal(pd).astype(f32)
    w["ip3_pol_w"] = np.zeros_like(w["ip3_pol_w"])
    w["ip3_pol_b"] = c
    rows = rng.standard_normal((4, pd)).astype(f32)
    w["ip4_pol_w"] = rows
    pol = onn.BlasNetwork(nr.parse_net(netproto.serialize_net(g))).forward(*_random_inputs(3))["policy"]
    shift = rows.astype(np.float64) @ c.astype(np.float64)           # c . row_i
    strs = oc.move_strs()
    idx = {s: i for i, s in enumerate(strs)}
    seen = set()
    for s in strs[1792:]:
        piece = "qrb".index(s[4])
        want = shift[piece] + shift[3]
        got = pol[:, idx[s]].astype(np.float64) - pol[:, idx[s[:4]]]
        np.testing.assert_allclose(got, want, rtol=0, atol=2e-5 * max(1.0, abs(want)))
        seen.add(piece)
    assert seen == {0, 1, 2}
    assert min(abs(shift[a] - shift[b]) for a in range(3) for b in range(a)) > 1e-2   # the shifts tell pieces apart


def test_se_unit_split_special_cases():
    """ApplySEUnit (se_unit.cc:54-60): the first C outputs of the second dense layer are the sigmoid scale, the
    next C the shift. (1) shift rows zero: out = act(sigma * (x + bias) + residual), sigma from rows 0..C-1;
    (2) scale rows zero: sigma = 1/2 exactly, out = act(x/2 + residual + rows C..2C-1 + bias/2). Swapping the
    halves turns one case into the other."""
    rng = np.random.default_rng(4)
    B, C, K = 2, 6, 3
    x = rng.standard_normal((B, C, 64))
    res = rng.standard_normal((B, C, 64))
    bias = rng.standard_normal(C)
    w1, b1 = rng.standard_normal((K, C)), rng.standard_normal(K)
    w2, b2 = rng.standard_normal((2 * C, K)), rng.standard_normal(2 * C)
    h = np.maximum((x.mean(axis=2) + bias) @ w1.T + b1, 0)          # dense 1 with ReLU on pooled + bias
    call = lambda w2_, b2_: onn.apply_se_unit(x.astype(f32), bias.astype(f32), res.astype(f32), w1.astype(f32),
                                              b1.astype(f32), w2_.astype(f32), b2_.astype(f32), nr.ACT_RELU)
    w2a, b2a = w2.copy(), b2.copy()
    w2a[C:], b2a[C:] = 0, 0
    sigma = 1 / (1 + np.exp(-(h @ w2[:C].T + b2[:C])))
    np.testing.assert_allclose(call(w2a, b2a), np.maximum(sigma[:, :, None] * (x + bias[None, :, None]) + res, 0),
                               rtol=1e-4, atol=1e-5)
    w2b, b2b = w2.copy(), b2.copy()
    w2b[:C], b2b[:C] = 0, 0
    shift = h @ w2[C:].T + b2[C:]
    np.testing.assert_allclose(call(w2b, b2b),
                               np.maximum(0.5 * x + res + (shift + 0.5 * bias)[:, :, None], 0), rtol=1e-4, atol=1e-5)


def test_fast_exp_and_legal_softmax(ref):
    x = np.linspace(-30, 5, 701).astype(f32)
    want = np.array([ref.ref_fast_exp(float(v)) for v in x], f32)
    np.testing.assert_allclose(onn.fast_exp(x), want, rtol=1e-6)
    np.testing.assert_allclose(onn.fast_exp(x), np.exp(x.astype(np.float64)), rtol=4e-3)
    np.testing.assert_array_equal(onn.fast_exp(x), want)      # same float operations in the same order
    assert onn.fast_exp(np.array([-200.0, -np.inf], f32)).tolist() == [0.0, 0.0]
    rng = np.random.default_rng(8)
    logits = (rng.standard_normal(1858) * 3).astype(f32)
    for n, t in ((4, 1.359), (35, 1.0), (218, 2.2)):
        legal = rng.permutation(1858)[:n]
        p = onn.softmax_policy_legal(logits, legal, t)
        assert abs(p.sum() - 1) < 1e-5 and p.argmax() == logits[legal].argmax()
        # wrapper.cc:135-156 step by step on float scalars with the compiled FastExp
        inv_t = f32(1.0) / f32(t)
        mx = max(logits[i] for i in legal)
        vals = [f32(ref.ref_fast_exp(float(f32(f32(logits[i] - mx) * inv_t)))) for i in legal]
        total = f32(0)
        for v in vals:
            total = f32(total + v)
        scale = f32(1.0) / total
        np.testing.assert_array_equal(p, np.array([f32(v * scale) for v in vals], f32))
        # the polynomial exponential stays within a few 1e-3 of the exact softmax at this temperature
        exact = np.exp((logits[legal].astype(np.float64) - float(mx)) / t)
        np.testing.assert_allclose(p, exact / exact.sum(), rtol=8e-3)


def test_e4m3_codec_vs_compiled_reference(ref):
    """oracle/fp8.py against FP32toFP8E4M3FN / FP8E4M3FNtoFP32 (fp8_utils.h:111-155): all 256 codes,
    every fp16 value and random floats including exact ties and the saturation edge."""
    from oracle import fp8
    ref.ref_fp32_to_fp8e4m3.argtypes = [ctypes.c_float]
    ref.ref_fp32_to_fp8e4m3.restype = ctypes.c_uint8
    ref.ref_fp8e4m3_to_fp32.argtypes = [ctypes.c_uint8]
    ref.ref_fp8e4m3_to_fp32.restype = ctypes.c_float
    table = fp8.e4m3_table()
    for code in range(256):
        want = ref.ref_fp8e4m3_to_fp32(code)
        assert (np.isnan(want) and np.isnan(table[code])) or want == table[code]
    rng = np.random.default_rng(8)
    halves = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = (table[:126] + table[1:127]) / 2                       # exact ties between neighbours
    xs = np.concatenate([halves[~np.isnan(halves)], mids, -mids, [448, 463.9, 464, 465, 1e9, -1e9, np.inf, -np.inf],
                         rng.standard_normal(20000) * np.exp(rng.uniform(-8, 7, 20000))]).astype(np.float32)
    got = fp8.e4m3_encode(xs)
    want = np.array([ref.ref_fp32_to_fp8e4m3(float(v)) for v in xs], np.uint8)
    np.testing.assert_array_equal(got, want)


def test_e4m3_codec_is_nearest_even_by_brute_force():
    """Textbook definition: the nearest of the 254 finite codes, ties to the even mantissa, saturating."""
    from oracle import fp8
    table = fp8.e4m3_table().astype(np.float64)
    pos = table[:127]                                             # 0 .. 448, increasing
    rng = np.random.default_rng(9)
    xs = np.abs(rng.standard_normal(5000) * np.exp(rng.uniform(-8, 6.5, 5000))).astype(np.float32)
    xs = np.concatenate([xs, ((pos[:-1] + pos[1:]) / 2).astype(np.float32)])
    got = fp8.e4m3_encode(xs)
    for x, g in zip(xs.astype(np.float64), got):
        d = np.abs(pos - min(x, 448.0))
        best = np.flatnonzero(d == d.min())
        want = best[0] if len(best) == 1 else [c for c in best if c % 2 == 0][0]
        assert g == want, (x, g, want)
    np.testing.assert_array_equal(fp8.e4m3_encode(-xs), got | 0x80)
    codes, scale = fp8.quantize_rows(np.array([[1.0, -2.0, 0.5], [0, 0, 0]], np.float32))
    assert scale[0] == np.float32(2.0 / 448) and scale[1] == 1.0
    np.testing.assert_array_equal(fp8.e4m3_decode(codes[0]) * scale[0], [1.0, -2.0, 0.5])
