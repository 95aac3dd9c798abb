"""TEST INFRASTRUCTURE -- CPU restatement (numpy, float32) of lc0's `blas`
network backend: the parity checker and the timed CPU baseline.  Matrix
products go through numpy's BLAS sgemm exactly where the reference calls
cblas_sgemm; everything else is elementwise float32.  Never imported by the
shipped package.

Follows (reference file:line):
  BlasComputation::ComputeBlocking      src/neural/backends/blas/network_blas.cc:473-971
  ForwardEncoderLayer                   src/neural/backends/blas/network_blas.cc:271-471
  EncodePlanes                          src/neural/backends/blas/network_blas.cc:973-981
  BlasNetwork ctor / MakeBlasNetwork    src/neural/backends/blas/network_blas.cc:983-1182
  FullyConnectedLayer::Forward1D        src/neural/backends/blas/fully_connected_layer.cc:49-106
  Convolution1::Forward                 src/neural/backends/blas/convolution1.cc:30-70
  WinogradConvolution3 (F(2x2,3x3))     src/neural/backends/blas/winograd_convolution3.cc:47-324
  WinogradFilterTransformF              src/neural/backends/shared/winograd_filter.cc:54-90
  ApplySEUnit                           src/neural/backends/blas/se_unit.cc:31-91
  LayerNorm2DWithSkipConnection         src/neural/backends/blas/encoder.h:29-78
  activations / softmax                 src/neural/backends/shared/activation.cc:37-267
  policy tables (closed form)           src/neural/tables/attention_policy_map.h, policy_map.h
  legal-move softmax of the caller      src/neural/wrapper.cc:135-156, src/utils/fastmath.h:59-86
  check-backend comparison              src/neural/backends/network_check.cc:121-186

Pins: activations, softmax, LayerNorm and the winograd filter transform against
the compiled reference translation units (oracle/_ref) and against torch/scipy
library routines; winograd convolution against direct zero-padded 3x3
correlation; the policy tables against SHA-256 of the reference's tables and
against oracle/_ref; one encoder layer against torch's
scaled_dot_product_attention + layer_norm; promotion offsets and the SE
gamma/beta split by closed-form special cases (tests/test_oracle_nn.py).
The whole-net wiring (flatten orders of the heads, policy Q.K^T, PE_DENSE
preprocessing, gating layout, smolgen flatten, residual-tower order, SE split)
is pinned against an independent float64 model written from the reference's
C++ (tests/blas_model_f64.py, tests/test_oracle_wholenet.py), which also shows
that each of these layout decisions, perturbed, fails the comparison.
The reference ships no whole-net output vectors and its backend cannot be
built here, so no reference-produced number enters these checks.
"""
import numpy as np

from . import netread as nr

f32 = np.float32
K_INPUT_PLANES = 112
K_SQUARES = 64
K_POLICY_OUTPUTS = 1858
K_POLICY_USED_PLANES = 73


# ---------------------------------------------------------------- tables ----
def _move_index_table():
    """(from,to) -> index for the 1792 queen/knight moves, then 66 promotions."""
    plain = {}
    idx = 0
    for frm in range(64):
        for to in range(64):
            if frm == to:
                continue
            dr, df = abs(to // 8 - frm // 8), abs(to % 8 - frm % 8)
            if dr == 0 or df == 0 or dr == df or (dr, df) in ((1, 2), (2, 1)):
                plain[(frm, to)] = idx
                idx += 1
    promo = {}
    for ff in range(8):
        for tf in (ff - 1, ff, ff + 1):
            if 0 <= tf < 8:
                for p in range(3):  # q, r, b
                    promo[(ff, tf, p)] = idx
                    idx += 1
    assert idx == K_POLICY_OUTPUTS
    return plain, promo


def attn_policy_map():
    """kAttnPolicyMap: 64*64 from-to logits then 8x24 promotion logits."""
    plain, promo = _move_index_table()
    m = np.full(64 * 64 + 8 * 24, -1, np.int16)
    for (frm, to), i in plain.items():
        m[frm * 64 + to] = i
    for (ff, tf, p), i in promo.items():
        m[4096 + 24 * ff + 3 * tf + p] = i
    return m


def pos_encoding():
    """kPosEncoding[64][64]: -1 on the diagonal, 1 where a move exists."""
    m = attn_policy_map()[:4096].reshape(64, 64)
    pe = (m >= 0).astype(f32)
    pe[np.arange(64), np.arange(64)] = -1.0
    return pe


def conv_policy_map():
    """kConvPolicyMap[73*64]: plane-major (plane*64 + from-square)."""
    plain, promo = _move_index_table()
    m = np.full(K_POLICY_USED_PLANES * 64, -1, np.int16)
    dirs = [(1, 0), (1, 1), (0, 1), (-1, 1), (-1, 0), (-1, -1), (0, -1), (1, -1)]  # (drank, dfile): N NE E SE S SW W NW
    knight = [(2, 1), (1, 2), (-1, 2), (-2, 1), (-2, -1), (-1, -2), (1, -2), (2, -1)]
    for sq in range(64):
        r, f = sq // 8, sq % 8
        for d, (dr, dfl) in enumerate(dirs):
            for dist in range(1, 8):
                rr, ff = r + dr * dist, f + dfl * dist
                if 0 <= rr < 8 and 0 <= ff < 8:
                    m[(d * 7 + dist - 1) * 64 + sq] = plain[(sq, rr * 8 + ff)]
        for k, (dr, dfl) in enumerate(knight):
            rr, ff = r + dr, f + dfl
            if 0 <= rr < 8 and 0 <= ff < 8:
                m[(56 + k) * 64 + sq] = plain[(sq, rr * 8 + ff)]
        if r == 6:
            for di, dfl in enumerate((-1, 0, 1)):      # NW, N, NE
                ff = f + dfl
                if 0 <= ff < 8:
                    for pi, p in enumerate((1, 2, 0)):  # r, b, q  (table ids: q0 r1 b2)
                        m[(64 + di * 3 + pi) * 64 + sq] = promo[(f, ff, p)]
    return m


ATTN_POLICY_MAP = attn_policy_map()
POS_ENCODING = pos_encoding()


# ----------------------------------------------------------- activations ----
def _mish(x):
    e = np.exp(x)
    n = e * e + f32(2.0) * e
    with np.errstate(invalid="ignore", over="ignore"):
        d = x / (n + f32(2.0))
        return np.where(x <= f32(-0.125), n * d, x - f32(2.0) * d).astype(f32)


def activate(x, act):
    """Activate() of shared/activation.cc:74-100 on float32 arrays."""
    x = np.asarray(x, f32)
    if act == nr.ACT_RELU:
        return np.where(x > 0, x, f32(0)).astype(f32)
    if act == nr.ACT_RELU_2:
        return np.where(x > 0, x * x, f32(0)).astype(f32)
    if act == nr.ACT_MISH:
        return _mish(x)
    if act == nr.ACT_TANH:
        return np.tanh(x).astype(f32)
    if act == nr.ACT_SIGMOID:
        return (f32(1.0) / (f32(1.0) + np.exp(-x))).astype(f32)
    if act == nr.ACT_SELU:
        alpha, scale = f32(1.67326324), f32(1.05070098)
        return np.where(x > 0, scale * x, scale * alpha * (np.exp(np.minimum(x, 0)) - f32(1.0))).astype(f32)
    if act == nr.ACT_SWISH:
        return (x / (f32(1.0) + np.exp(-x))).astype(f32)
    if act == nr.ACT_NONE:
        return x
    raise ValueError("unsupported activation function")


def softmax_rows(x):
    """SoftmaxActivation (activation.cc:37-49) over the last axis."""
    x = np.asarray(x, f32)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return (e / e.sum(axis=-1, keepdims=True, dtype=f32)).astype(f32)


def layer_norm_skip(data, alpha, skip, gammas, betas, eps):
    """LayerNorm2DWithSkipConnection (encoder.h:29-66): rows of `data`."""
    t = data * f32(alpha)
    if skip is not None:
        t = t + skip
    t = t.astype(f32)
    mean = t.mean(axis=-1, keepdims=True, dtype=f32)
    diff = t - mean
    var = (diff * diff).mean(axis=-1, keepdims=True, dtype=f32)
    den = f32(1.0) / np.sqrt(var + f32(eps))
    return (betas + gammas * diff * den).astype(f32)


def fc(x, w, b, act, out_size=None):
    """Forward1D: out = act(x . w^T + b); w is [out][in] row-major.  Bias and
    activation are applied only when a bias is given (fully_connected_layer.cc:103-105)."""
    x = np.asarray(x, f32)
    in_size = x.shape[-1]
    w = np.asarray(w, f32).reshape(-1, in_size)
    y = x @ w.T
    if b is not None:
        y = activate(y + np.asarray(b, f32), act)
    return y.astype(f32)


# -------------------------------------------------------------- winograd ----
_G = np.array([[1, 0, 0], [.5, .5, .5], [.5, -.5, .5], [0, 0, 1]], f32)
_BT = np.array([[1, 0, -1, 0], [0, 1, 1, 0], [0, -1, 1, 0], [0, 1, 0, -1]], f32)
_AT = np.array([[1, 1, 1, 0], [0, 1, -1, -1]], f32)


def winograd_filter_transform(f, outputs, channels):
    """U[xi][nu][c][o] = (G g G^T)[xi][nu] (winograd_filter.cc:54-90)."""
    g = np.asarray(f, f32).reshape(outputs, channels, 3, 3)
    u = np.einsum("ik,ockl,jl->ijco", _G, g, _G, optimize=True)
    return np.ascontiguousarray(u, f32).reshape(-1)


def winograd_conv3(x, u, cin, cout):
    """3x3 same-padded convolution of x[B,cin,8,8] with transformed filter u
    (TransformIn / Sgemm / TransformOut, winograd_convolution3.cc:59-324)."""
    b = x.shape[0]
    xp = np.zeros((b, cin, 10, 10), f32)
    xp[:, :, 1:9, 1:9] = x
    # tiles[b, c, by, bx, i, j] = xp[b, c, 2by+i, 2bx+j]
    tiles = np.lib.stride_tricks.sliding_window_view(xp, (4, 4), axis=(2, 3))[:, :, ::2, ::2]
    v = np.einsum("ik,bcyxkl,jl->ijbyxc", _BT, tiles, _BT, optimize=True).astype(f32)
    v = v.reshape(16, b * 16, cin)
    uu = np.asarray(u, f32).reshape(16, cin, cout)
    m = np.matmul(v, uu)  # [16, B*16, cout]
    m = m.reshape(4, 4, b, 4, 4, cout)
    y = np.einsum("ik,klbyxo,jl->boyixj", _AT, m, _AT, optimize=True).astype(f32)
    return np.ascontiguousarray(y.reshape(b, cout, 8, 8))


def conv1x1(x, w, cin, cout):
    """Convolution1::Forward: per sample W[cout,cin] . x[cin,64]."""
    w = np.asarray(w, f32).reshape(cout, cin)
    return np.einsum("oc,bcs->bos", w, x.reshape(x.shape[0], cin, 64), optimize=True).astype(f32)


def bias_activate(x, biases, act):
    return activate(x + np.asarray(biases, f32)[None, :, None], act)


def apply_se_unit(x, ch_bias, residual, w1, b1, w2, b2, act):
    """ApplySEUnit (se_unit.cc:31-91) on [B,C,64] tensors."""
    bsz, c, _ = x.shape
    pool = (x.sum(axis=2, dtype=f32) / f32(64) + ch_bias).astype(f32)
    h = fc(pool, w1, b1, act)
    s = fc(h, w2, b2, nr.ACT_NONE)
    gamma = (f32(1.0) / (f32(1.0) + np.exp(-s[:, :c]))).astype(f32)
    beta = (s[:, c:] + gamma * ch_bias).astype(f32)
    return activate(gamma[:, :, None] * x + residual + beta[:, :, None], act)


# ---------------------------------------------------------------- network ----
def encode_planes(masks, values):
    """EncodePlanes: [B,112] (mask,value) -> [B,112,64] float32."""
    masks = np.asarray(masks, np.uint64)
    bits = (masks[:, :, None] >> np.arange(64, dtype=np.uint64)[None, None, :]) & np.uint64(1)
    return (bits.astype(f32) * np.asarray(values, f32)[:, :, None]).astype(f32)


class BlasNetwork:
    """Mirror of BlasNetwork + BlasComputation for whole batches."""

    def __init__(self, net, policy_head="vanilla", value_head="winner", mlh=True, batch_size=256):
        nf = net.format
        if nf.network not in (nr.NETWORK_CLASSICAL_WITH_HEADFORMAT, nr.NETWORK_SE_WITH_HEADFORMAT,
                              nr.NETWORK_ATTENTIONBODY_WITH_HEADFORMAT,
                              nr.NETWORK_ATTENTIONBODY_WITH_MULTIHEADFORMAT):
            raise nr.WeightsError("Network format %d is not supported by the BLAS backend." % nf.network)
        if nf.policy not in (nr.POLICY_CLASSICAL, nr.POLICY_CONVOLUTION, nr.POLICY_ATTENTION):
            raise nr.WeightsError("Policy format %d is not supported by the BLAS backend." % nf.policy)
        if nf.value not in (nr.VALUE_CLASSICAL, nr.VALUE_WDL):
            raise nr.WeightsError("Value format %d is not supported by the BLAS backend." % nf.value)
        if nf.moves_left not in (0, nr.MOVES_LEFT_V1):
            raise nr.WeightsError("Moves left head format %d is not supported by the BLAS backend." % nf.moves_left)
        if nf.default_activation not in (0, 1):
            raise nr.WeightsError("Default activation %d is not supported by the BLAS backend." % nf.default_activation)
        if nf.input_embedding not in (0, 1, 2):
            raise nr.WeightsError("Input embedding %d is not supported by the BLAS backend." % nf.input_embedding)
        self.nf = nf
        self.w = w = net.weights
        self.max_batch_size = min(batch_size, 2048)
        self.wdl = nf.value == nr.VALUE_WDL
        self.moves_left = nf.moves_left == nr.MOVES_LEFT_V1 and mlh
        self.conv_policy = nf.policy == nr.POLICY_CONVOLUTION
        self.attn_policy = nf.policy == nr.POLICY_ATTENTION
        self.attn_body = nf.network in (nr.NETWORK_ATTENTIONBODY_WITH_HEADFORMAT,
                                        nr.NETWORK_ATTENTIONBODY_WITH_MULTIHEADFORMAT)
        self.default_act = nr.ACT_MISH if nf.default_activation == 1 else nr.ACT_RELU
        self.pe_dense = nf.input_embedding == nr.INPUT_EMBEDDING_PE_DENSE
        self.smolgen_act = self.ffn_act = nr.ACT_NONE
        if self.attn_body:
            self.smolgen_act = self.default_act if nf.smolgen_activation == nr.ACT_DEFAULT else nf.smolgen_activation
            self.ffn_act = self.default_act if nf.ffn_activation == nr.ACT_DEFAULT else nf.ffn_activation
        if policy_head not in w.policy_heads:
            raise nr.WeightsError("The policy head you specified '%s' does not exist in this net." % policy_head)
        if value_head not in w.value_heads:
            raise nr.WeightsError("The value head you specified '%s' does not exist in this net." % value_head)
        self.ph = w.policy_heads[policy_head]
        self.vh = w.value_heads[value_head]
        # Filter transforms done once at construction (network_blas.cc:1038-1072).
        ch = w.input.biases.size
        self.channels = ch
        self.u_input = winograd_filter_transform(w.input.weights, ch, K_INPUT_PLANES) if ch else None
        self.u_res = [(winograd_filter_transform(r.conv1.weights, ch, ch),
                       winograd_filter_transform(r.conv2.weights, ch, ch)) for r in w.residual]
        if self.conv_policy:
            v = w.policy_heads["vanilla"]
            self.u_pol1 = winograd_filter_transform(v.policy1.weights, ch, ch)
            self.u_pol = winograd_filter_transform(v.policy.weights, v.policy.biases.size, ch)
        self.conv_map = conv_policy_map() if self.conv_policy else None

    # ForwardEncoderLayer (network_blas.cc:271-471); x is [B*64, emb].
    def encoder_layer(self, x, layer, emb, heads, smolgen_act, ffn_act, alpha, eps):
        bsz = x.shape[0] // 64
        mha = layer.mha
        d_model = mha.q_b.size
        depth = d_model // heads
        qk_bias = None
        if mha.has_smolgen:
            sg = mha.smolgen
            hc = sg.compress.size // emb
            hs = sg.dense1_b.size
            gen = sg.dense2_b.size
            t = fc(x, sg.compress, None, nr.ACT_NONE)                       # [B*64, hc]
            t = fc(t.reshape(bsz, 64 * hc), sg.dense1_w, sg.dense1_b, smolgen_act)
            t = layer_norm_skip(t, 1.0, None, sg.ln1_gammas, sg.ln1_betas, 1e-3)
            t = fc(t, sg.dense2_w, sg.dense2_b, smolgen_act)                # [B, H*g]
            t = layer_norm_skip(t, 1.0, None, sg.ln2_gammas, sg.ln2_betas, 1e-3)
            qk_bias = fc(t.reshape(bsz * heads, gen // heads), self.w.smolgen_w, None, nr.ACT_NONE)
            qk_bias = qk_bias.reshape(bsz, heads, 64, 64)
        q = fc(x, mha.q_w, mha.q_b, nr.ACT_NONE).reshape(bsz, 64, heads, depth)
        k = fc(x, mha.k_w, mha.k_b, nr.ACT_NONE).reshape(bsz, 64, heads, depth)
        scaling = f32(1.0) / np.sqrt(f32(depth))
        qk = np.matmul(q.transpose(0, 2, 1, 3), k.transpose(0, 2, 3, 1)) * scaling  # [B,H,64,64]
        if qk_bias is not None:
            qk = qk_bias + qk
        p = softmax_rows(qk.astype(f32))
        v = fc(x, mha.v_w, mha.v_b, nr.ACT_NONE).reshape(bsz, 64, heads, depth)
        a = np.matmul(p, v.transpose(0, 2, 1, 3))                           # [B,H,64,depth]
        a = np.ascontiguousarray(a.transpose(0, 2, 1, 3)).reshape(bsz * 64, d_model)
        o = fc(a, mha.dense_w, mha.dense_b, nr.ACT_NONE)
        x = layer_norm_skip(o, alpha, x, layer.ln1_gammas, layer.ln1_betas, eps)
        h = fc(x, layer.ffn.dense1_w, layer.ffn.dense1_b, ffn_act)
        h = fc(h, layer.ffn.dense2_w, layer.ffn.dense2_b, nr.ACT_NONE)
        return layer_norm_skip(h, alpha, x, layer.ln2_gammas, layer.ln2_betas, eps)

    def forward(self, masks, values, return_intermediates=False):
        """Returns dict(policy [B,1858] raw logits, wdl [B,3] (or q [B]), m [B])."""
        masks = np.asarray(masks, np.uint64)
        values = np.asarray(values, f32)
        outs = []
        for s in range(0, masks.shape[0], self.max_batch_size):
            outs.append(self._forward_chunk(masks[s:s + self.max_batch_size],
                                            values[s:s + self.max_batch_size]))
        res = {k: np.concatenate([o[k] for o in outs], axis=0) for k in outs[0]}
        return res

    def _forward_chunk(self, masks, values):
        w = self.w
        bsz = masks.shape[0]
        act = self.default_act
        planes = encode_planes(masks, values)          # [B,112,64] NCHW
        flow = None                                     # NCHW tower output [B,C,64]
        if w.residual:
            ch = self.channels
            y = winograd_conv3(planes.reshape(bsz, 112, 8, 8), self.u_input, 112, ch).reshape(bsz, ch, 64)
            flow = bias_activate(y, w.input.biases, act)
            for r, (u1, u2) in zip(w.residual, self.u_res):
                t = winograd_conv3(flow.reshape(bsz, ch, 8, 8), u1, ch, ch).reshape(bsz, ch, 64)
                t = bias_activate(t, r.conv1.biases, act)
                t = winograd_conv3(t.reshape(bsz, ch, 8, 8), u2, ch, ch).reshape(bsz, ch, 64)
                if r.has_se:
                    flow = apply_se_unit(t, r.conv2.biases, flow, r.se.w1, r.se.b1, r.se.w2, r.se.b2, act)
                else:
                    flow = activate(flow + t + r.conv2.biases[None, :, None], act)  # BiasResidual
        x = None                                        # token-major [B*64, emb]
        if self.attn_body:
            emb = w.ip_emb_b.size
            if not w.residual:
                nhwc = planes.transpose(0, 2, 1)        # [B,64,112]
                if self.pe_dense:
                    enc_ch = w.ip_emb_preproc_b.size // 64
                    pre = np.ascontiguousarray(nhwc[:, :, :12]).reshape(bsz, 64 * 12)
                    pe = fc(pre, w.ip_emb_preproc_w, w.ip_emb_preproc_b, nr.ACT_NONE).reshape(bsz, 64, enc_ch)
                else:
                    pe = np.broadcast_to(POS_ENCODING[None], (bsz, 64, 64))
                inp = np.concatenate([nhwc, pe], axis=2).astype(f32)
                inp = inp.reshape(bsz * 64, -1)
            else:
                # As the reference: buffer3 is not rewritten in this branch, the
                # embedding reads whatever it holds; not a supported net shape.
                raise nr.WeightsError("attention body on top of a residual tower is not restated")
            x = fc(inp, w.ip_emb_w, w.ip_emb_b, act)
            if self.pe_dense:
                x = layer_norm_skip(x, 1.0, None, w.ip_emb_ln_gammas, w.ip_emb_ln_betas, 1e-3)
            if w.ip_mult_gate.size > 0 and w.ip_add_gate.size > 0:
                mult = w.ip_mult_gate.reshape(emb, 64).T
                add = w.ip_add_gate.reshape(emb, 64).T
                x = (x.reshape(bsz, 64, emb) * mult[None] + add[None]).astype(f32).reshape(bsz * 64, emb)
            alpha = f32(np.power(2.0 * len(w.encoder), -0.25))
            if self.pe_dense:
                h = fc(x, w.ip_emb_ffn.dense1_w, w.ip_emb_ffn.dense1_b, self.ffn_act)
                h = fc(h, w.ip_emb_ffn.dense2_w, w.ip_emb_ffn.dense2_b, nr.ACT_NONE)
                x = layer_norm_skip(h, alpha, x, w.ip_emb_ffn_ln_gammas, w.ip_emb_ffn_ln_betas, 1e-3)
            eps = 1e-3 if self.pe_dense else 1e-6
            for layer in w.encoder:
                x = self.encoder_layer(x, layer, emb, w.encoder_head_count, self.smolgen_act,
                                       self.ffn_act, alpha, eps)
        out = {}
        vh = self.vh
        # Value head (network_blas.cc:725-772).
        if self.attn_body:
            hv = fc(x, vh.ip_val_w, vh.ip_val_b, act).reshape(bsz, -1)
        else:
            cv = vh.value.biases.size
            hv = bias_activate(conv1x1(flow, vh.value.weights, self.channels, cv), vh.value.biases, act).reshape(bsz, -1)
        hv = fc(hv, vh.ip1_val_w, vh.ip1_val_b, act)
        if self.wdl:
            out["wdl"] = softmax_rows(fc(hv, vh.ip2_val_w, vh.ip2_val_b, nr.ACT_NONE))
        else:
            out["q"] = np.tanh((hv @ vh.ip2_val_w.reshape(-1) + vh.ip2_val_b[0]).astype(np.float64)).astype(f32)
        # Moves-left head (:775-803).
        if self.moves_left:
            if self.attn_body:
                hm = fc(x, w.ip_mov_w, w.ip_mov_b, act).reshape(bsz, -1)
            else:
                cm = w.moves_left.biases.size
                hm = bias_activate(conv1x1(flow, w.moves_left.weights, self.channels, cm),
                                   w.moves_left.biases, act).reshape(bsz, -1)
            hm = fc(hm, w.ip1_mov_w, w.ip1_mov_b, act)
            out["m"] = fc(hm, w.ip2_mov_w, w.ip2_mov_b, nr.ACT_RELU).reshape(bsz)
        else:
            out["m"] = np.zeros(bsz, f32)
        # Policy head (:806-968).
        ph = self.ph
        if self.attn_policy:
            if not self.attn_body:
                x = np.ascontiguousarray(flow.transpose(0, 2, 1)).reshape(bsz * 64, self.channels)
            pe_size = ph.ip_pol_b.size
            t = fc(x, ph.ip_pol_w, ph.ip_pol_b, act if self.attn_body else nr.ACT_SELU)
            for layer in ph.pol_encoder:
                t = self.encoder_layer(t, layer, pe_size, ph.pol_encoder_head_count,
                                       self.smolgen_act if self.attn_body else nr.ACT_NONE,
                                       self.ffn_act if self.attn_body else nr.ACT_SELU, 1.0, 1e-6)
            pd = ph.ip2_pol_b.size
            q = fc(t, ph.ip2_pol_w, ph.ip2_pol_b, nr.ACT_NONE).reshape(bsz, 64, pd)
            k = fc(t, ph.ip3_pol_w, ph.ip3_pol_b, nr.ACT_NONE).reshape(bsz, 64, pd)
            scaling = f32(1.0) / np.sqrt(f32(pd))
            logits = (np.matmul(q, k.transpose(0, 2, 1)) * scaling).astype(f32)   # [B,64,64]
            ppo = ph.ip4_pol_w.reshape(4, pd)
            off = np.einsum("bjk,ik->bij", k[:, 56:64, :], ppo, optimize=True).astype(f32)  # [B,4,8]
            off3 = off[:, :3, :] + off[:, 3:4, :]
            # promo[b, k, j, i] = logits[b, 48+k, 56+j] + off3[b, i, j]
            promo = logits[:, 48:56, 56:64][:, :, :, None] + off3.transpose(0, 2, 1)[:, None, :, :]
            buf = np.concatenate([logits.reshape(bsz, 4096), promo.reshape(bsz, 192)], axis=1)
            policy = np.zeros((bsz, K_POLICY_OUTPUTS), f32)
            sel = ATTN_POLICY_MAP >= 0
            policy[:, ATTN_POLICY_MAP[sel]] = buf[:, sel]
        elif self.conv_policy:
            ch = self.channels
            pch = ph.policy.biases.size
            t = winograd_conv3(flow.reshape(bsz, ch, 8, 8), self.u_pol1, ch, ch).reshape(bsz, ch, 64)
            t = bias_activate(t, ph.policy1.biases, act)
            t = winograd_conv3(t.reshape(bsz, ch, 8, 8), self.u_pol, ch, pch).reshape(bsz, pch, 64)
            t = bias_activate(t, ph.policy.biases, nr.ACT_NONE).reshape(bsz, pch * 64)
            policy = np.zeros((bsz, K_POLICY_OUTPUTS), f32)
            sel = self.conv_map >= 0
            policy[:, self.conv_map[sel]] = t[:, :K_POLICY_USED_PLANES * 64][:, sel]
        else:
            cp = ph.policy.biases.size
            t = bias_activate(conv1x1(flow, ph.policy.weights, self.channels, cp), ph.policy.biases, act)
            policy = fc(t.reshape(bsz, cp * 64), ph.ip_pol_w, ph.ip_pol_b, nr.ACT_NONE)
        out["policy"] = policy
        return out

    # NetworkComputation getters over a forward() result.
    @staticmethod
    def q_val(out, s):
        return out["wdl"][s, 0] - out["wdl"][s, 2] if "wdl" in out else out["q"][s]

    @staticmethod
    def d_val(out, s):
        return out["wdl"][s, 1] if "wdl" in out else f32(0)


# ---------------------------------------------------- caller-side helpers ----
def fast_exp(a):
    """FastExp (fastmath.h:59-86) on a float32 array."""
    with np.errstate(all="ignore"):   # arguments below -126 (down to -inf) take the early return, as in the reference
        a = (np.asarray(a, f32) * f32(1.442695040)).astype(f32)
        safe = np.where(a < -126, f32(0), a)
        exp = np.where(safe < 0, (safe - f32(1)).astype(np.int32), safe.astype(np.int32)).astype(np.int32)
        out = (safe - exp.astype(f32)).astype(f32)
        out = (f32(1.0) + out * (f32(0.6602339) + f32(0.33976606) * out)).astype(f32)
        bits = out.view(np.int32) + (exp.astype(np.int64) << 23).astype(np.int32)
        res = bits.view(f32).copy()
        res[a < -126] = 0.0
    return res


def softmax_policy_legal(logits, legal_idx, temperature=1.359):
    """NetworkAsBackendComputation::SoftmaxPolicy (wrapper.cc:135-156): every step in float, the
    reciprocal temperature formed once (wrapper.cc:81-82), the total accumulated move by move
    (std::accumulate) and applied as a multiplication by 1/total (1 when the total is 0)."""
    legal_idx = np.asarray(legal_idx, np.int64)
    if legal_idx.size == 0:
        return np.zeros(0, f32)
    l = np.asarray(logits, f32)[legal_idx]
    inv_t = f32(1.0) / f32(temperature)
    with np.errstate(over="ignore"):
        p = fast_exp(((l - l.max()).astype(f32) * inv_t).astype(f32))
    total = np.add.accumulate(p, dtype=f32)[-1]          # sequential, left to right
    scale = f32(1.0) / total if total > 0 else f32(1.0)
    return (p * scale).astype(f32)


def check_softmax_legal(logits, legal_idx):
    """Exact-exp softmax over legal moves as the check backend does
    (network_check.cc:121-141)."""
    l = np.asarray(logits, np.float64)[legal_idx]
    e = np.exp(l - l.max())
    return (e / e.sum()).astype(f32)
