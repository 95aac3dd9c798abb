"""What pins oracle/fp8_net.py, the numpy emulation of the fp8 configuration that the GPU's e4m3 pass is held to:
  * with quantisation and half rounding switched off it is the fp32 oracle, bit for bit;
  * on operands that e4m3 represents exactly the quantised dense layer is the plain dense layer;
  * its quantisation error has the size the format predicts, and a mis-wired activation scale moves the result by
    far more than the bound the GPU comparison uses (so that comparison can tell the two apart)."""
import numpy as np
import pytest

from lc0_amd import netgen
from oracle import chess as oc
from oracle import fp8
from oracle import fp8_net
from oracle import netread as nr
from oracle import nn as onn

f32 = np.float32


@pytest.fixture(scope="module")
def positions():
    return oc.random_positions(24, seed=4242)


@pytest.mark.parametrize("name", ["tiny_attn_f8", "tiny_attn_f8_sg", "tiny_attn_dense_f8", "tiny_attn_d64"])
def test_emulation_switched_off_is_the_fp32_oracle_bit_for_bit(name, positions):
    net = nr.load(netgen.cached_config(name))
    want = onn.BlasNetwork(net).forward(positions["masks"], positions["values"])
    got = fp8_net.Fp8BlasNetwork(net, quantize=False, half_points=False).forward(positions["masks"], positions["values"])
    for key in want:
        np.testing.assert_array_equal(got[key].view(np.uint32), want[key].view(np.uint32), err_msg=key)


def test_quantised_dense_layer_on_exactly_representable_operands():
    """Weights and activations taken from the e4m3 grid (rows scaled so that their largest magnitude is 448, as the
    per-row rule assumes): quantisation changes nothing and the layer equals the oracle's Forward1D."""
    rng = np.random.default_rng(5)
    table = fp8.e4m3_table()
    grid = table[np.isfinite(table)]
    w = rng.choice(grid, (48, 128)).astype(f32)
    w[:, 0] = 448.0                          # absmax / 448 is then a power of two: the codes are the grid values
    w *= f32(2.0 ** -12)
    x = rng.choice(grid[np.abs(grid) <= 16], (20, 128)).astype(f32)
    b = rng.standard_normal(48).astype(f32)
    lin = fp8_net._QuantLinear(w.reshape(-1), 128)
    np.testing.assert_array_equal(lin.scale, np.full(48, 2.0 ** -12, f32))
    got = lin(fp8_net.quantize_activation(x * f32(0.25), 0.25), 0.25, b, nr.ACT_MISH)
    want = onn.fc(x * f32(0.25), w.reshape(-1), b, nr.ACT_MISH)
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-6)


def test_activation_quantisation_saturates_and_uses_the_reciprocal():
    codes = fp8_net.quantize_activation(np.array([1e6, -1e6, 0.0, 3.0], f32), 0.5)
    np.testing.assert_array_equal(fp8.e4m3_decode(codes), np.array([448.0, -448.0, 0.0, 6.0], f32))


def test_quantisation_noise_and_miswired_scales(positions):
    """On the smallest fp8-capable net: the emulated fp8 pass stays within the noise e4m3 predicts of the fp32 oracle
    (a few per cent of the logit spread). Rounding to half on top of it moves the result by a good part of that noise
    again, although a half carries eight more mantissa bits: a perturbation of relative size d flips a code with
    probability ~ d / step and then moves the value by a whole step, so its variance is d x step against step^2 / 12
    for the quantisation itself. Two faithful evaluations of an fp8 net therefore differ by a fixed fraction of the
    format's noise, and a comparison between them resolves a wiring fault only when the fault is larger than that.
    The faults below are: FFN1 and Q/K/V scaled back with each other's activation scale (the scales made to differ by
    1.5, as layer-norm gains of a trained net would), and Q/K/V and the attention-output layer likewise (there the
    factor on V cancels against the one on the output layer and only the softmax temperature changes)."""
    net = nr.load(netgen.cached_config("tiny_attn_f8_sg"))
    m, v = positions["masks"], positions["values"]
    want = onn.BlasNetwork(net).forward(m, v)["policy"]
    spread = float(want.std())
    emu = fp8_net.Fp8BlasNetwork(net, gemms=("qkv", "dense", "ffn1", "ffn2", "smolgen"))
    scales, sg_scales = emu.calibrate(m, v)
    assert scales.shape == (2, 4) and sg_scales.shape == (2, 3) and (scales > 0).all() and (sg_scales > 0).all()
    got = emu.forward(m, v)["policy"]
    rms = lambda a: float(np.sqrt(np.mean(a * a)))
    assert 1e-4 * spread < rms(got - want) < 0.1 * spread
    no_half = fp8_net.Fp8BlasNetwork(net, scales=scales, smolgen_scales=sg_scales, half_points=False,
                                     gemms=("qkv", "dense", "ffn1", "ffn2", "smolgen")).forward(m, v)["policy"]
    noise = rms(got - want)
    assert 0.05 * noise < rms(no_half - got) < noise
    for fault in ("swap_x_x1", "swap_x_att"):
        # (make the two scales of the swap differ as they do on a trained net: layer norm gains are not all one)
        s2 = scales.copy()
        s2[:, 2] *= 1.5
        ref = fp8_net.Fp8BlasNetwork(net, scales=s2, smolgen_scales=sg_scales).forward(m, v)["policy"]
        bad = fp8_net.Fp8BlasNetwork(net, scales=s2, smolgen_scales=sg_scales, perturb=fault).forward(m, v)["policy"]
        assert rms(bad - ref) > 1.5 * noise, fault


def test_generator_on_half_operands_is_the_chain_minus_one_quantisation(positions):
    """gemms "smolgen_chain" (the generator layer on the half-precision output of the last row norm, the other three
    smolgen layers on e4m3 operands) against "smolgen" (all four) and against no smolgen layer in e4m3: it differs from
    both, by less than e4m3 noise, and it is the closer of the two to the fp32 oracle's attention bias path when only
    the generator's quantisation is at stake (same scales, same everything else)."""
    net = nr.load(netgen.cached_config("tiny_attn_f8_sg"))
    m, v = positions["masks"], positions["values"]
    big = ("qkv", "dense", "ffn1", "ffn2")
    scales, sg_scales = fp8_net.Fp8BlasNetwork(net, gemms=big + ("smolgen",)).calibrate(m, v)
    run = lambda gemms: fp8_net.Fp8BlasNetwork(net, scales=scales, smolgen_scales=sg_scales, gemms=gemms).forward(m, v)["policy"]
    want = onn.BlasNetwork(net).forward(m, v)["policy"]
    all4, chain3, none = run(big + ("smolgen",)), run(big + ("smolgen_chain",)), run(big)
    rms = lambda a: float(np.sqrt(np.mean(a * a)))
    noise = rms(all4 - want)
    assert 0 < rms(chain3 - all4) < noise
    assert 0 < rms(chain3 - none) < noise
    # with nothing else quantised, taking the generator out of e4m3 can only bring the result closer to fp32
    only4 = fp8_net.Fp8BlasNetwork(net, scales=scales, smolgen_scales=sg_scales, gemms=("smolgen",)).forward(m, v)["policy"]
    only3 = fp8_net.Fp8BlasNetwork(net, scales=scales, smolgen_scales=sg_scales, gemms=("smolgen_chain",)).forward(m, v)["policy"]
    assert rms(only3 - want) < rms(only4 - want)
