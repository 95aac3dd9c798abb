"""The product's weights loader (lc0_amd/csrc/weights.cc, through lc0mi_weights_list / lc0mi_weights_tensor of
the C ABI; host code only, no GPU) on what real lc0 files contain: the four Layer encodings
(src/utils/weights_adapter.cc:38-62), batch-norm statistics in their three historical forms
(src/neural/network_legacy.cc:62-131), the scalar value head and every branch of FixOlderWeightsFile
(src/neural/loader.cc:108-158).

Three checks per file: (1) every decoded tensor equals the oracle reader's (oracle/netread.py) to the last bit
or, where the two sum in different orders, to 1e-6; (2) the decoded values agree with the generator's float32
tensors within the encoding's resolution, and the batch-norm fold with torch's conv2d + batch_norm on the
unfolded tensors; (3) the upgraded format fields equal the decision table of loader.cc."""
import numpy as np
import pytest
import torch

from lc0_amd import backend, netgen, netproto
from oracle import netread as nr

ENCODINGS = ["float32", "linear16", "float16", "bfloat16"]
NETS = ["tiny_resnet_bn", "tiny_resnet_convpolicy_bn", "tiny_resnet_classical_value", "tiny_attn",
        "tiny_attn_dense", "tiny_attn_d64", "old_noformat", "old_classical", "old_se", "old_attn_as_se",
        "old_ab_legacy", "old_format6_with_heads"]


def _oracle_tensors(w):
    out = {}

    def put(name, v):
        v = np.asarray(v, np.float32).reshape(-1)
        if v.size:
            out[name] = v

    def conv(name, c):
        put(name + ".weights", c.weights)
        put(name + ".biases", c.biases)

    def enc(name, l):
        for k in ("q_w", "q_b", "k_w", "k_b", "v_w", "v_b", "dense_w", "dense_b"):
            put(name + ".mha." + k, getattr(l.mha, k))
        if l.mha.has_smolgen:
            for k, v in vars(l.mha.smolgen).items():
                put(name + ".mha.smolgen." + k, v)
        for k in ("ln1_gammas", "ln1_betas", "ln2_gammas", "ln2_betas"):
            put(name + "." + k, getattr(l, k))
        for k, v in vars(l.ffn).items():
            put(name + ".ffn." + k, v)

    conv("input", w.input)
    for i, r in enumerate(w.residual):
        conv("residual.%d.conv1" % i, r.conv1)
        conv("residual.%d.conv2" % i, r.conv2)
        if r.has_se:
            for k, v in vars(r.se).items():
                put("residual.%d.se.%s" % (i, k), v)
    for k in ("ip_emb_preproc_w", "ip_emb_preproc_b", "ip_emb_w", "ip_emb_b", "ip_emb_ln_gammas", "ip_emb_ln_betas",
              "ip_mult_gate", "ip_add_gate", "ip_emb_ffn_ln_gammas", "ip_emb_ffn_ln_betas", "ip_mov_w", "ip_mov_b",
              "ip1_mov_w", "ip1_mov_b", "ip2_mov_w", "ip2_mov_b", "smolgen_w"):
        put(k, getattr(w, k))
    for k, v in vars(w.ip_emb_ffn).items():
        put("ip_emb_ffn." + k, v)
    for i, l in enumerate(w.encoder):
        enc("encoder.%d" % i, l)
    conv("moves_left", w.moves_left)
    for hname, h in w.policy_heads.items():
        n = "policy_heads." + hname
        for k in ("ip_pol_w", "ip_pol_b", "ip2_pol_w", "ip2_pol_b", "ip3_pol_w", "ip3_pol_b", "ip4_pol_w"):
            put(n + "." + k, getattr(h, k))
        conv(n + ".policy1", h.policy1)
        conv(n + ".policy", h.policy)
        for i, l in enumerate(h.pol_encoder):
            enc(n + ".pol_encoder.%d" % i, l)
    for hname, h in w.value_heads.items():
        n = "value_heads." + hname
        conv(n + ".value", h.value)
        for k in ("ip_val_w", "ip_val_b", "ip1_val_w", "ip1_val_b", "ip2_val_w", "ip2_val_b"):
            put(n + "." + k, getattr(h, k))
    return out


@pytest.mark.parametrize("encoding", ENCODINGS)
@pytest.mark.parametrize("name", NETS)
def test_loader_equals_oracle_reader(name, encoding):
    raw = netproto.serialize_net(netgen.CONFIGS[name](), netgen.ENCODINGS[encoding])
    fmt, got = backend.decoded_weights(raw)
    ref = nr.parse_net(raw)
    want = _oracle_tensors(ref.weights)
    assert sorted(got) == sorted(want)
    for key in ("input", "output", "network", "policy", "value", "moves_left", "default_activation",
                "smolgen_activation", "ffn_activation", "input_embedding"):
        assert fmt[key] == getattr(ref.format, key), key
    assert fmt["headcount"] == ref.weights.encoder_head_count
    for k in want:
        assert got[k].shape == want[k].shape, k
        np.testing.assert_allclose(got[k], want[k], rtol=1e-6, atol=1e-7, err_msg=k)


# resolution of each encoding relative to a tensor's range / magnitude
_TOL = {"float32": (0.0, 0.0), "linear16": (1.0 / 65535, 0.0), "float16": (0.0, 2.0 ** -11), "bfloat16": (0.0, 2.0 ** -8)}


@pytest.mark.parametrize("encoding", ENCODINGS)
def test_decoded_layers_agree_with_the_generator(encoding):
    net = netgen.CONFIGS["tiny_attn_dense"]()
    _, got = backend.decoded_weights(netproto.serialize_net(net, netgen.ENCODINGS[encoding]))
    w = net["weights"]
    range_tol, rel_tol = _TOL[encoding]
    pairs = [("ip_emb_w", w["ip_emb_w"]), ("encoder.1.mha.smolgen.dense2_w", w["encoder"][1]["mha"]["smolgen"]["dense2_w"]),
             ("encoder.0.ffn.dense1_b", w["encoder"][0]["ffn"]["dense1_b"]), ("smolgen_w", w["smolgen_w"]),
             ("ip_mult_gate", w["ip_mult_gate"]), ("policy_heads.vanilla.ip_pol_w", w["policy_heads"]["ip_pol_w"]),
             ("policy_heads.soft.ip4_pol_w", w["policy_heads"]["soft"]["ip4_pol_w"]),
             ("policy_heads.optimistic.ip2_pol_w", w["policy_heads"]["optimistic_st"]["ip2_pol_w"]),
             ("value_heads.st.ip1_val_w", w["value_heads"]["st"]["ip1_val_w"])]
    for name, src in pairs:
        src = np.asarray(src, np.float32).reshape(-1)
        # round to nearest: half a step of the 16-bit grid, or half an ulp (at most 2^-11 resp. 2^-8 of the value)
        # (binary16 subnormals below 2^-14 are 2^-24 apart)
        tol = 0.51 * range_tol * float(src.max() - src.min()) + rel_tol * np.abs(src) + (2.0 ** -25 if encoding == "float16" else 1e-12)
        assert np.all(np.abs(got[name] - src) <= tol), name


@pytest.mark.parametrize("name", ["tiny_resnet_bn", "old_se"])
def test_batch_norm_fold_equals_convolution_then_batch_norm(name):
    """All three historical forms: with gammas/betas, without them, and without biases either."""
    net = netgen.CONFIGS[name]()
    _, got = backend.decoded_weights(netproto.serialize_net(net))
    rng = np.random.default_rng(8)
    blocks = [("input", net["weights"]["input"])]
    for i, r in enumerate(net["weights"]["residual"]):
        blocks += [("residual.%d.conv1" % i, r["conv1"]), ("residual.%d.conv2" % i, r["conv2"])]
    forms = set()
    for key, blk in blocks:
        wt = torch.from_numpy(np.asarray(blk["weights"], np.float64))
        cout, cin = wt.shape[:2]
        x = torch.from_numpy(rng.standard_normal((2, cin, 8, 8)))
        bias = torch.from_numpy(np.asarray(blk["biases"], np.float64)) if "biases" in blk else None
        gam = torch.from_numpy(np.asarray(blk["bn_gammas"], np.float64)) if "bn_gammas" in blk else None
        bet = torch.from_numpy(np.asarray(blk["bn_betas"], np.float64)) if "bn_betas" in blk else None
        forms.add((bias is not None, gam is not None))
        y = torch.nn.functional.conv2d(x, wt, bias, padding=1)
        want = torch.nn.functional.batch_norm(y, torch.from_numpy(np.asarray(blk["bn_means"], np.float64)),
                                              torch.from_numpy(np.asarray(blk["bn_stddivs"], np.float64)), gam, bet, eps=1e-5)
        fw = torch.from_numpy(got[key + ".weights"].astype(np.float64).reshape(cout, cin, 3, 3))
        fb = torch.from_numpy(got[key + ".biases"].astype(np.float64))
        np.testing.assert_allclose(torch.nn.functional.conv2d(x, fw, fb, padding=1).numpy(), want.numpy(),
                                   rtol=1e-4, atol=1e-4, err_msg=key)
    if name == "tiny_resnet_bn":
        assert forms == {(True, True), (True, False), (False, False)}


# loader.cc:108-158, one row per branch: stored (network, fields present) -> format after the fix
UPGRADES = {
    "old_noformat": dict(input=1, output=1, network=3, policy=1, value=1),
    "old_classical": dict(network=3, policy=1, value=1),
    "old_se": dict(network=4, policy=1, value=1),
    "old_attn_as_se": dict(network=6, ffn_activation=8, smolgen_activation=7, input_embedding=1),
    "old_ab_legacy": dict(network=7, input_embedding=2),
    "old_format6_with_heads": dict(network=7, input_embedding=2),
    "tiny_attn": dict(network=6, input_embedding=1, ffn_activation=0),
    "tiny_attn_nosmolgen": dict(network=6, input_embedding=1),
}


@pytest.mark.parametrize("name", sorted(UPGRADES))
def test_older_file_formats_are_upgraded(name):
    fmt, _ = backend.decoded_weights(netproto.serialize_net(netgen.CONFIGS[name]()))
    for key, want in UPGRADES[name].items():
        assert fmt[key] == want, (name, key, fmt)


def test_attention_body_without_smolgen_stored_as_se_keeps_default_activations():
    """loader.cc:137-141: the squared-ReLU / swish override applies only when smolgen_w is present."""
    net = netgen._old_format(netgen.attention_body(64, 2, 2, 96, seed=5, perturb_ln=True, std=0.1), network=4,
                             drop=("smolgen_activation", "ffn_activation", "input_embedding"))
    fmt, _ = backend.decoded_weights(netproto.serialize_net(net))
    assert (fmt["network"], fmt["ffn_activation"], fmt["smolgen_activation"], fmt["input_embedding"]) == (6, 0, 0, 1)


def test_non_linear16_file_encoding_needs_a_recent_min_version():
    """loader.cc:181-185."""
    net = netgen.CONFIGS["tiny_resnet"]()
    net["format"]["weights_encoding"] = netproto.FLOAT16
    with pytest.raises(backend.BackendError, match="unsupported encoding"):
        backend.decoded_weights(netproto.serialize_net(net))
    net["min_version"] = {"major": 0, "minor": 33, "patch": 0}
    backend.decoded_weights(netproto.serialize_net(net))
