"""TEST ORACLE, not product code: the blas-backend restatement (oracle/nn.py) with the arithmetic of the
fp8 configuration emulated in numpy, so that a GPU result in e4m3 can be held to a tight bound instead of
to the noise level of the format.

What is emulated (the reference has no fp8 arithmetic of its own: it hands the graph to MIGraphX,
src/neural/backends/onnx/network_onnx.cc:757, and owns only the codec, src/utils/fp8_utils.h:111-155):
  * weights of the encoder's Q/K/V, attention-output and FFN layers (and, on request, of the smolgen
    layers) are e4m3 codes with one scale per output row, absmax / 448 (oracle/fp8.py: quantize_rows);
  * the operand of each of those layers is quantised with one scale per tensor and layer,
    code = e4m3(value * (1 / scale)), saturating; products of decoded codes are summed exactly (float64)
    and multiplied by (activation scale x row scale) in float32 before bias and activation;
  * with `half_points` the values the GPU backend stores as halves between kernels (layer outputs, the
    residual stream, un-normalised softmax weights) are rounded to half at the same points, so that the
    two differ only by summation order inside a kernel.
The activation scales are inputs (what the backend's calibration produced, or `calibrate()` below, which
applies the same rule to this model's own activations: largest magnitude -> 224).

Pins: with `quantize=False, half_points=False` every overridden step runs the parent's statements in the
parent's order and the result equals oracle/nn.py bit for bit (tests/test_oracle_fp8_net.py); the codec
and the per-row weight quantisation are pinned in tests/test_oracle_nn.py against the compiled reference
functions; the switch `perturb` mis-wires one scale on purpose so that tests can show the comparison
notices it.
"""
import numpy as np

from . import fp8
from . import netread as nr
from .nn import BlasNetwork, activate, f32, fc, layer_norm_skip, softmax_rows

SCALES_PER_LAYER = 4          # x (Q/K/V operand), attention output, x1 (FFN1 operand), FFN hidden
SMOLGEN_SCALES_PER_LAYER = 3  # compression output, first and second layer-norm output of the chain


def _half(a):
    return np.asarray(a, np.float16).astype(f32)


class _QuantLinear:
    """One dense layer with e4m3 weights: codes, decoded values, per-row scale."""

    def __init__(self, w, in_size):
        w = np.asarray(w, f32).reshape(-1, in_size)
        self.codes, self.scale = fp8.quantize_rows(w)
        self.values = fp8.e4m3_decode(self.codes).astype(np.float64)

    def __call__(self, x_codes, act_scale, bias, act):
        """act(col_scale * sum_k dec(x)[m][k] dec(w)[n][k] + bias), col_scale = act_scale * row scale (float32)."""
        acc = (fp8.e4m3_decode(x_codes).astype(np.float64) @ self.values.T).astype(f32)
        y = acc * (f32(act_scale) * self.scale)[None, :]
        if bias is not None:
            y = activate(y + np.asarray(bias, f32), act)
        return y.astype(f32)


def quantize_activation(x, scale):
    """e4m3 codes of x / scale as the kernels form them: multiply by the float32 reciprocal, saturate."""
    return fp8.e4m3_encode(np.asarray(x, f32) * (f32(1.0) / f32(scale)))


class Fp8BlasNetwork(BlasNetwork):
    """BlasNetwork whose body encoder layers run the fp8 configuration.

    scales: float array [layers][4] (x, attention output, x1, FFN hidden), value = code x scale.
    gemms: which layers use e4m3 operands, subset of {"qkv", "dense", "ffn1", "ffn2", "smolgen", "smolgen_chain"}
        ("smolgen": compression, both dense layers and the shared generator layer; "smolgen_chain": the first three,
        with the generator on the half-precision output of the last row norm, as the backend computes it when the
        generator runs inside its attention kernel).
    smolgen_scales: [layers][3], needed when "smolgen" is listed.
    perturb: None, "swap_x_x1" (the Q/K/V and FFN1 products are scaled back with each other's activation
      scale), "swap_x_att" (the same for Q/K/V and the attention-output layer) or "stale_layer" (every layer
      scales back with the activation scales of the layer before it).
    """

    def __init__(self, net, scales=None, gemms=("qkv", "dense", "ffn1", "ffn2"), quantize=True, half_points=True,
                 smolgen_scales=None, perturb=None, **kw):
        super().__init__(net, **kw)
        self.quantize = quantize
        self.half_points = half_points
        self.gemms = set(gemms)
        self.perturb = perturb
        self.scales = None if scales is None else np.asarray(scales, f32).reshape(len(self.w.encoder), SCALES_PER_LAYER)
        self.smolgen_scales = (None if smolgen_scales is None else
                               np.asarray(smolgen_scales, f32).reshape(len(self.w.encoder), SMOLGEN_SCALES_PER_LAYER))
        self.absmax = None       # filled by calibrate()
        self._carry = None       # float32 layer-norm output of the previous layer, before rounding to half
        self._qw = {}
        if quantize:
            emb = self.w.ip_emb_b.size
            for li, layer in enumerate(self.w.encoder):
                mha, ffn = layer.mha, layer.ffn
                d_model = mha.q_b.size
                q = {}
                if "qkv" in self.gemms:
                    q["q"], q["k"], q["v"] = (_QuantLinear(w, emb) for w in (mha.q_w, mha.k_w, mha.v_w))
                if "dense" in self.gemms:
                    q["dense"] = _QuantLinear(mha.dense_w, d_model)
                if "ffn1" in self.gemms:
                    q["ffn1"] = _QuantLinear(ffn.dense1_w, emb)
                if "ffn2" in self.gemms:
                    q["ffn2"] = _QuantLinear(ffn.dense2_w, ffn.dense1_b.size)
                if ("smolgen" in self.gemms or "smolgen_chain" in self.gemms) and mha.has_smolgen:
                    sg = mha.smolgen
                    hc = sg.compress.size // emb
                    q["sg_compress"] = _QuantLinear(sg.compress, emb)
                    q["sg_dense1"] = _QuantLinear(sg.dense1_w, 64 * hc)
                    q["sg_dense2"] = _QuantLinear(sg.dense2_w, sg.dense1_b.size)
                    q["sg_global"] = _QuantLinear(self.w.smolgen_w, sg.dense2_b.size // self.w.encoder_head_count)
                self._qw[li] = q

    # -- helpers -------------------------------------------------------------------------------------
    def _h(self, a):
        return _half(a) if self.half_points else a

    def _layer_index(self, layer):
        for i, l in enumerate(self.w.encoder):
            if l is layer:
                return i
        return -1

    def _scale(self, li, which):
        if self.perturb == "stale_layer":
            li = max(li - 1, 0)
        return self.scales[li][which]

    def _note(self, li, slot, a):
        if self.absmax is not None:
            self.absmax[li][slot] = max(self.absmax[li][slot], float(np.abs(a).max()))

    def _note_sg(self, li, slot, a):
        if self.absmax is not None:
            self.absmax_smolgen[li][slot] = max(self.absmax_smolgen[li][slot], float(np.abs(a).max()))

    def calibrate(self, masks, values):
        """Activation scales by the backend's rule on this model's own (unquantised) activations: the largest
        magnitude of each tensor over the given positions maps to 224. Returns (scales, smolgen_scales)."""
        n = len(self.w.encoder)
        saved = self.quantize
        self.quantize = False
        self.absmax = np.zeros((n, SCALES_PER_LAYER))
        self.absmax_smolgen = np.zeros((n, SMOLGEN_SCALES_PER_LAYER))
        try:
            self.forward(masks, values)
            amax, amax_sg = self.absmax, self.absmax_smolgen
        finally:
            self.absmax = None
            self.quantize = saved
        to_scale = lambda a: np.where(a > 0, a / 224.0, 1.0).astype(f32)
        self.scales, self.smolgen_scales = to_scale(amax), to_scale(amax_sg)
        return self.scales, self.smolgen_scales

    # -- forward -------------------------------------------------------------------------------------
    def _forward_chunk(self, masks, values):
        self._carry = None
        return super()._forward_chunk(masks, values)

    def encoder_layer(self, x, layer, emb, heads, smolgen_act, ffn_act, alpha, eps):
        li = self._layer_index(layer)
        if li < 0:                       # policy-head encoder layers stay in the parent's arithmetic
            return super().encoder_layer(x, layer, emb, heads, smolgen_act, ffn_act, alpha, eps)
        qz = self.quantize
        qw = self._qw.get(li, {})
        bsz = x.shape[0] // 64
        mha = layer.mha
        d_model = mha.q_b.size
        depth = d_model // heads
        # x: the residual stream as stored (halves); xf: the same values before that rounding, which is
        # what the layer norm quantises from. The first layer's input exists as halves only.
        xf = x if self._carry is None else self._carry
        x = self._h(x)
        if self._carry is None:
            xf = x
        self._note(li, 0, x)
        s_x = self._scale(li, 0) if qz else None
        sg_q = "smolgen" in self.gemms or "smolgen_chain" in self.gemms
        xq = quantize_activation(xf, self.scales[li][0]) if qz and ("qkv" in self.gemms or sg_q) else None
        qk_bias = None
        if mha.has_smolgen:
            sg = mha.smolgen
            hc = sg.compress.size // emb
            gen = sg.dense2_b.size
            if qz and sg_q:
                ss = self.smolgen_scales[li]
                t = qw["sg_compress"](xq, s_x, None, nr.ACT_NONE)
                tq = quantize_activation(t, ss[0]).reshape(bsz, 64 * hc)
                t = self._h(qw["sg_dense1"](tq, ss[0], sg.dense1_b, smolgen_act))
                # (the two row norms write their e4m3 copies from the float values, like the body's norms)
                t = layer_norm_skip(t, 1.0, None, sg.ln1_gammas, sg.ln1_betas, 1e-3)
                tq = quantize_activation(t, ss[1])
                t = self._h(qw["sg_dense2"](tq, ss[1], sg.dense2_b, smolgen_act))
                t = layer_norm_skip(t, 1.0, None, sg.ln2_gammas, sg.ln2_betas, 1e-3)
                if "smolgen" in self.gemms:
                    tq = quantize_activation(t, ss[2]).reshape(bsz * heads, gen // heads)
                    qk_bias = self._h(qw["sg_global"](tq, ss[2], None, nr.ACT_NONE))
                else:
                    qk_bias = self._h(fc(self._h(t).reshape(bsz * heads, gen // heads), self.w.smolgen_w, None,
                                         nr.ACT_NONE))
            else:
                t = self._h(fc(x, sg.compress, None, nr.ACT_NONE))
                self._note_sg(li, 0, t)
                t = self._h(fc(t.reshape(bsz, 64 * hc), sg.dense1_w, sg.dense1_b, smolgen_act))
                t = self._h(layer_norm_skip(t, 1.0, None, sg.ln1_gammas, sg.ln1_betas, 1e-3))
                self._note_sg(li, 1, t)
                t = self._h(fc(t, sg.dense2_w, sg.dense2_b, smolgen_act))
                t = self._h(layer_norm_skip(t, 1.0, None, sg.ln2_gammas, sg.ln2_betas, 1e-3))
                self._note_sg(li, 2, t)
                qk_bias = self._h(fc(t.reshape(bsz * heads, gen // heads), self.w.smolgen_w, None, nr.ACT_NONE))
            qk_bias = qk_bias.reshape(bsz, heads, 64, 64)
        if qz and "qkv" in self.gemms:
            s_back = (self._scale(li, 2) if self.perturb == "swap_x_x1" else
                      self._scale(li, 1) if self.perturb == "swap_x_att" else s_x)
            q, k, v = (self._h(qw[n](xq, s_back, b, nr.ACT_NONE)) for n, b in (("q", mha.q_b), ("k", mha.k_b), ("v", mha.v_b)))
            q = q.reshape(bsz, 64, heads, depth)
            k = k.reshape(bsz, 64, heads, depth)
        else:
            q = self._h(fc(x, mha.q_w, mha.q_b, nr.ACT_NONE)).reshape(bsz, 64, heads, depth)
            k = self._h(fc(x, mha.k_w, mha.k_b, nr.ACT_NONE)).reshape(bsz, 64, heads, depth)
            v = None
        scaling = f32(1.0) / np.sqrt(f32(depth))
        qk = np.matmul(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 3, 1)) * scaling
        if qk_bias is not None:
            qk = qk_bias + qk
        if v is None:
            v = self._h(fc(x, mha.v_w, mha.v_b, nr.ACT_NONE))
        v = v.reshape(bsz, 64, heads, depth)
        if self.half_points:
            # the kernels multiply V by the un-normalised softmax weights, rounded to half, and divide by
            # the float sum of the unrounded ones afterwards
            qk = qk.astype(f32)
            e = np.exp(qk - qk.max(axis=-1, keepdims=True))
            a = np.matmul(_half(e), v.transpose(0, 2, 1, 3)) / e.sum(axis=-1, keepdims=True, dtype=f32)
        else:
            p = softmax_rows(qk.astype(f32))
            a = np.matmul(p, v.transpose(0, 2, 1, 3))
        a = np.ascontiguousarray(a.transpose(0, 2, 1, 3)).reshape(bsz * 64, d_model)
        self._note(li, 1, a)
        if qz and "dense" in self.gemms:
            s_att = self._scale(li, 0) if self.perturb == "swap_x_att" else self._scale(li, 1)
            o = qw["dense"](quantize_activation(a, self.scales[li][1]), s_att, mha.dense_b, nr.ACT_NONE)
        else:
            o = fc(self._h(a), mha.dense_w, mha.dense_b, nr.ACT_NONE)
        o = self._h(o)
        x1f = layer_norm_skip(o, alpha, x, layer.ln1_gammas, layer.ln1_betas, eps)
        x1 = self._h(x1f)
        self._note(li, 2, x1)
        if qz and "ffn1" in self.gemms:
            s_back = self._scale(li, 0) if self.perturb == "swap_x_x1" else self._scale(li, 2)
            h = qw["ffn1"](quantize_activation(x1f, self.scales[li][2]), s_back, layer.ffn.dense1_b, ffn_act)
        else:
            h = fc(x1, layer.ffn.dense1_w, layer.ffn.dense1_b, ffn_act)
        self._note(li, 3, self._h(h))
        if qz and "ffn2" in self.gemms:
            # (an FFN1 with e4m3 operands quantises its float result; a half FFN1 output is quantised from the halves)
            src = h if "ffn1" in self.gemms else self._h(h)
            h = qw["ffn2"](quantize_activation(src, self.scales[li][3]), self._scale(li, 3), layer.ffn.dense2_b, nr.ACT_NONE)
        else:
            h = fc(self._h(h), layer.ffn.dense2_w, layer.ffn.dense2_b, nr.ACT_NONE)
        h = self._h(h)
        out = layer_norm_skip(h, alpha, x1, layer.ln2_gammas, layer.ln2_betas, eps)
        self._carry = out
        return out
