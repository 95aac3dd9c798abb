"""Pins the whole-net wiring of oracle/nn.py (flatten orders of the heads, attention-policy Q.K^T and promotion
offsets, PE_DENSE preprocessing, gating layout, SE split, smolgen flatten, residual-tower order) against an
independent float64 model (tests/blas_model_f64.py: torch conv2d / scaled_dot_product_attention / layer_norm on
the generator's weight dictionary, reference tables parsed from the reference's header text when present).

For every layout decision there is a `perturb` switch in the model that takes a plausible wrong alternative;
`test_perturbed_layout_is_detected` shows the comparison fails under each of them."""
import numpy as np
import pytest

from lc0_amd import netgen
from oracle import chess as oc
from oracle import netread as nr
from oracle import nn as onn

from blas_model_f64 import BlasModelF64

NETS = ["tiny_resnet", "tiny_resnet_convpolicy", "tiny_resnet_nose", "tiny_resnet_40se", "tiny_attn",
        "tiny_attn_nosmolgen", "tiny_attn_dense", "tiny_attn_d64", "tiny_resnet_attnpolicy"]
TOL = 1e-4


def _outputs(name, perturb=None, n=6):
    pos = oc.random_positions(n, seed=321)
    oracle = onn.BlasNetwork(nr.load(netgen.cached_config(name))).forward(pos["masks"], pos["values"])
    model = BlasModelF64(netgen.CONFIGS[name](), perturb=perturb).forward(pos["masks"], pos["values"])
    return oracle, model


def _max_errors(oracle, model):
    errs = {"policy": float(np.abs(oracle["policy"] - model["policy"]).max()),
            "m": float(np.abs(oracle["m"] - model["m"]).max())}
    key = "wdl" if "wdl" in oracle else "q"
    errs["value"] = float(np.abs(oracle[key] - model[key]).max())
    return errs


@pytest.mark.parametrize("name", NETS)
def test_oracle_equals_independent_float64_model(name):
    oracle, model = _outputs(name)
    errs = _max_errors(oracle, model)
    scale = max(1.0, float(np.abs(model["policy"]).max()))
    assert errs["policy"] <= TOL * scale, errs
    assert errs["value"] <= TOL, errs
    assert errs["m"] <= TOL * max(1.0, float(np.abs(model["m"]).max())), errs
    # the policy must not be trivially flat, or the comparison would pin nothing
    assert float(model["policy"].std()) > 1e-3


PERTURBATIONS = [("tiny_attn", "value_flatten", "value"), ("tiny_attn", "mlh_flatten", "m"),
                 ("tiny_attn", "policy_qk_transpose", "policy"), ("tiny_attn", "promotion_index", "policy"),
                 ("tiny_attn", "smolgen_flatten", "policy"), ("tiny_attn_dense", "gating_transpose", "policy"),
                 ("tiny_attn_dense", "pe_dense_order", "policy"), ("tiny_resnet", "se_split", "policy")]


@pytest.mark.parametrize("name,perturb,output", PERTURBATIONS)
def test_perturbed_layout_is_detected(name, perturb, output):
    oracle, model = _outputs(name, perturb=perturb)
    errs = _max_errors(oracle, model)
    assert errs[output] > 20 * TOL, (perturb, errs)
