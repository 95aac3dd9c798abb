"""Whole-net fixture tests/golden/tiny_net_outputs.npz (written by tests/golden/make_tiny_net_outputs.py):
oracle outputs of the seeded tiny nets on 8 positions stored as UCI move lists.

CPU: the positions replay to the stored planes bit-exactly and the oracle reproduces the stored
outputs. GPU: the backend, through the C ABI, matches them within the fp32 / fp16 tolerances."""
import os

import numpy as np
import pytest

from lc0_amd import netgen
from oracle import chess as oc
from oracle import netread as nr
from oracle import nn as onn

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_net_outputs.npz")
NETS = ["tiny_resnet", "tiny_resnet_convpolicy", "tiny_attn", "tiny_attn_dense"]


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN, allow_pickle=False)


def test_positions_replay_to_the_stored_planes(golden):
    for i, line in enumerate(golden["uci"]):
        h = oc.History()
        for mv in str(line).split():
            h.append_uci(mv)
        masks, values, _ = h.encode()
        np.testing.assert_array_equal(masks, golden["masks"][i])
        np.testing.assert_array_equal(values, golden["values"][i])


@pytest.mark.parametrize("name", NETS)
def test_oracle_reproduces_the_fixture(name, golden):
    res = onn.BlasNetwork(nr.load(netgen.cached_config(name))).forward(golden["masks"], golden["values"])
    # same code, possibly another BLAS build underneath: summation order only
    np.testing.assert_allclose(res["policy"], golden[name + ".policy"], rtol=0, atol=2e-5)
    np.testing.assert_allclose(res["wdl"], golden[name + ".wdl"], rtol=0, atol=2e-5)
    np.testing.assert_allclose(res["m"], golden[name + ".m"], rtol=1e-4, atol=2e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("name,options,tol", [("tiny_resnet", "precision=fp32", 1e-3), ("tiny_resnet", "", 5e-3),
                                              ("tiny_resnet_convpolicy", "precision=fp32", 1e-3),
                                              ("tiny_attn", "", 5e-3), ("tiny_attn_dense", "", 5e-3)])
def test_gpu_matches_the_fixture(name, options, tol, golden):
    from lc0_amd import Network
    net = Network(netgen.cached_config(name), options)
    comp = net.NewComputation()
    comp.AddInputs(golden["masks"], golden["values"])
    comp.ComputeBlocking()
    res = comp.results()
    want_p, want_wdl, want_m = golden[name + ".policy"], golden[name + ".wdl"], golden[name + ".m"]
    assert np.abs(onn.softmax_rows(res["policy"]) - onn.softmax_rows(want_p)).max() <= tol
    assert np.abs(res["policy"] - want_p).max() <= 6 * tol * max(1.0, float(np.abs(want_p).max()))
    assert np.abs(res["q"] - (want_wdl[:, 0] - want_wdl[:, 2])).max() <= tol
    assert np.abs(res["d"] - want_wdl[:, 1]).max() <= tol
    assert (np.abs(res["m"] - want_m) / np.maximum(np.abs(want_m), 1.0)).max() <= 2e-2


def test_writer_schema_matches_reference_net_proto():
    """Field numbers, nesting and repetition of lc0_amd.netproto.SCHEMA against proto/net.proto of the reference
    (tests/golden/net_proto_fields.json, extracted from its text by tests/golden/make_net_proto_fields.py). The
    oracle's reader and the product's reader are checked against files this writer produces, so this pins all
    three views of the format."""
    import json

    from lc0_amd import netproto

    golden = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "net_proto_fields.json")))
    scalar = {"uint": ("uint32", "Encoding", "InputFormat", "OutputFormat", "NetworkStructure", "PolicyFormat",
                       "ValueFormat", "MovesLeftFormat", "ActivationFunction", "DefaultActivation",
                       "InputEmbeddingFormat"),
              "float": ("float",), "bytes": ("bytes",), "string": ("string",), "fixed32": ("fixed32",)}
    checked = 0
    for message, fields in netproto.SCHEMA.items():
        assert message in golden, message
        for name, (number, kind) in fields.items():
            ref = golden[message][name]
            assert ref["number"] == number, (message, name)
            repeated = kind.startswith("*")
            assert (ref["label"] == "repeated") == repeated, (message, name)
            kind = kind.lstrip("*")
            if kind in scalar:
                assert ref["type"] in scalar[kind], (message, name, ref["type"])
            else:
                assert ref["type"].split(".")[-1] == kind, (message, name, ref["type"])
            checked += 1
    assert checked >= 140
    # the writer knows every field of the messages a weights file is made of
    for message in ("Weights", "ConvBlock", "SEunit", "Residual", "Smolgen", "MHA", "FFN", "EncoderLayer",
                    "PolicyHead", "PolicyHeads", "ValueHeads", "Layer", "NetworkFormat", "Format"):
        # (the head maps are read by no backend: src/neural/network_legacy.cc:236-306)
        missing = set(golden[message]) - set(netproto.SCHEMA[message]) - {"policy_head_map", "value_head_map"}
        assert not missing, (message, missing)
