"""Independent float64 model of the reference blas backend's forward pass, for pinning oracle/nn.py.

Written from the reference's C++ (file:line below), not from the oracle:
  * it consumes the weight dictionary of lc0_amd.netgen directly (no weight-file reader involved),
  * 3x3 convolutions are torch's direct `conv2d` (no winograd),
  * attention, layer norm, softmax and the activations are torch library routines in float64,
  * every reshape carries the flat-buffer index expression of the C++ loop it stands for.

`perturb` switches one layout decision to a plausible wrong alternative; the tests use it to show that the
comparison with the oracle fails under that mistake.

Reference: src/neural/backends/blas/network_blas.cc:271-471 (encoder layer), :473-971 (ComputeBlocking),
src/neural/backends/blas/se_unit.cc:31-91, src/neural/backends/blas/encoder.h:29-66,
src/neural/network_legacy.cc:196-306 (which weights make up the heads).
"""
import os
import re

import numpy as np
import torch
import torch.nn.functional as F

REF_TABLES = "/root/reference/src/neural/tables"
T = torch.float64


def _parse_table(path, name):
    text = open(path).read()
    body = text[text.index(name):]
    body = body[body.index("{") + 1:body.index("};")]
    return np.array([int(v) for v in re.findall(r"-?\d+", body)], np.int64)


def policy_tables():
    """kAttnPolicyMap / kConvPolicyMap as the reference headers spell them (parsed from their text) when the
    reference tree is present, else the oracle's closed forms (pinned to the same tables by SHA-256)."""
    if os.path.isdir(REF_TABLES):
        attn = _parse_table(os.path.join(REF_TABLES, "attention_policy_map.h"), "kAttnPolicyMap[]")
        conv = _parse_table(os.path.join(REF_TABLES, "policy_map.h"), "kConvPolicyMap[]")
        return attn, conv
    from oracle import nn as onn
    return onn.ATTN_POLICY_MAP.astype(np.int64), onn.conv_policy_map().astype(np.int64)


def pos_encoding_table():
    if os.path.isdir(REF_TABLES):
        text = open(os.path.join(REF_TABLES, "attention_policy_map.h")).read()
        body = text[text.index("kPosEncoding[64]"):]
        body = body[body.index("=") + 1:body.index("};")]
        vals = [float(v) for v in re.findall(r"-?\d+\.?\d*f?", body.replace("f", ""))]
        return np.array(vals, np.float64).reshape(64, 64)
    from oracle import nn as onn
    return onn.POS_ENCODING.astype(np.float64)


def _t(a):
    return torch.as_tensor(np.asarray(a, np.float64), dtype=T)


def _act(x, name):
    if name == "relu":
        return torch.relu(x)
    if name == "mish":
        return F.mish(x)
    if name == "swish":
        return F.silu(x)
    if name == "selu":
        return F.selu(x)
    if name == "none":
        return x
    raise ValueError(name)


def _fc(x, w, b, act="none"):
    """Forward1D (fully_connected_layer.cc:49-106): rows of x times w[out][in]; bias and activation only
    when a bias is given."""
    w = _t(w).reshape(-1, x.shape[-1])
    y = x @ w.T
    if b is not None:
        y = _act(y + _t(b), act)
    return y


def _ln(data, alpha, skip, gammas, betas, eps):
    """LayerNorm2DWithSkipConnection (encoder.h:29-66): normalise data * alpha + skip over the channels."""
    v = data * alpha
    if skip is not None:
        v = v + skip
    return F.layer_norm(v, (v.shape[-1],), _t(gammas), _t(betas), eps)


class BlasModelF64:
    def __init__(self, net, perturb=None):
        self.nf = net["format"]["network_format"]
        self.w = net["weights"]
        self.perturb = perturb
        self.attn_body = self.nf["network"] in (6, 7)
        self.default_act = "mish" if self.nf.get("default_activation", 0) == 1 else "relu"
        sa, fa = self.nf.get("smolgen_activation", 0), self.nf.get("ffn_activation", 0)
        names = {0: self.default_act, 1: "mish", 2: "relu", 3: "none", 6: "selu", 7: "swish"}
        self.smolgen_act, self.ffn_act = names[sa], names[fa]
        self.pe_dense = self.nf.get("input_embedding", 0) == 2
        self.attn_map, self.conv_map = policy_tables()

    # ---- heads' weights: network_legacy.cc:236-306 ----
    def _policy_head(self):
        w = self.w
        if "policy_heads" in w:
            ph = w["policy_heads"]
            head = dict(ph["vanilla"])
            head["ip_pol_w"], head["ip_pol_b"] = ph["ip_pol_w"], ph["ip_pol_b"]
            return head
        return w

    def _value_head(self):
        return self.w["value_heads"]["winner"] if "value_heads" in self.w else self.w

    # ---- ForwardEncoderLayer, network_blas.cc:271-471; x is [B, 64, emb] ----
    def _encoder_layer(self, x, layer, heads, smolgen_act, ffn_act, alpha, eps):
        b, _, emb = x.shape
        mha = layer["mha"]
        d_model = len(mha["q_b"])
        depth = d_model // heads
        bias = None
        if "smolgen" in mha:
            sg = mha["smolgen"]
            hc = np.asarray(sg["compress"]).size // emb
            t = _fc(x, sg["compress"], None)                          # [B,64,hc]; buffer index (b*64+sq)*hc + c
            if self.perturb == "smolgen_flatten":
                t = t.transpose(1, 2)
            t = t.reshape(b, 64 * hc)                                  # Forward1D(batch, 64*hc, ...): index sq*hc + c
            t = _fc(t, sg["dense1_w"], sg["dense1_b"], smolgen_act)
            t = _ln(t, 1.0, None, sg["ln1_gammas"], sg["ln1_betas"], 1e-3)
            t = _fc(t, sg["dense2_w"], sg["dense2_b"], smolgen_act)
            t = _ln(t, 1.0, None, sg["ln2_gammas"], sg["ln2_betas"], 1e-3)
            gen = t.shape[1] // heads
            # Forward1D(batch*heads, gen, 64*64): row b*heads + h reads t[b][h*gen .. (h+1)*gen)
            bias = _fc(t.reshape(b * heads, gen), self.w["smolgen_w"], None).reshape(b, heads, 64, 64)
        q = _fc(x, mha["q_w"], mha["q_b"])
        k = _fc(x, mha["k_w"], mha["k_b"])
        v = _fc(x, mha["v_w"], mha["v_b"])
        # head h owns columns h*depth .. (h+1)*depth (A = &Q[h*depth], lda = heads*depth)
        split = lambda m: m.reshape(b, 64, heads, depth).permute(0, 2, 1, 3)
        attn = F.scaled_dot_product_attention(split(q), split(k), split(v), attn_mask=bias,
                                              scale=1.0 / float(np.sqrt(np.float32(depth))))
        attn = attn.permute(0, 2, 1, 3).reshape(b, 64, d_model)
        o = _fc(attn, mha["dense_w"], mha["dense_b"])
        x = _ln(o, alpha, x, layer["ln1_gammas"], layer["ln1_betas"], eps)
        h = _fc(x, layer["ffn"]["dense1_w"], layer["ffn"]["dense1_b"], ffn_act)
        h = _fc(h, layer["ffn"]["dense2_w"], layer["ffn"]["dense2_b"])
        return _ln(h, alpha, x, layer["ln2_gammas"], layer["ln2_betas"], eps)

    def _conv3(self, x, block, act):
        """convolve3.Forward + BiasActivate: NCHW correlation with [out][in][3][3] filters."""
        y = F.conv2d(x, _t(block["weights"]), padding=1)
        return y if act is None else _act(y + _t(block["biases"])[None, :, None, None], act)

    def _conv1(self, x, block, act):
        y = F.conv2d(x, _t(block["weights"]).reshape(len(block["biases"]), -1, 1, 1))
        return _act(y + _t(block["biases"])[None, :, None, None], act)

    def forward(self, masks, values):
        w, act = self.w, self.default_act
        masks = np.asarray(masks, np.uint64)
        b = masks.shape[0]
        # EncodePlanes (network_blas.cc:973-981): buffer[plane*64 + i] = mask bit i ? value : 0
        planes = np.zeros((b, 112, 64))
        for i in range(64):
            planes[:, :, i] = ((masks >> np.uint64(i)) & np.uint64(1)).astype(np.float64) * np.asarray(values, np.float64)
        planes = _t(planes)
        flow = None
        if w.get("residual"):
            flow = self._conv3(planes.reshape(b, 112, 8, 8), w["input"], act)
            for r in w["residual"]:
                t = self._conv3(flow, r["conv1"], act)
                t = self._conv3(t, r["conv2"], None)
                bias = _t(r["conv2"]["biases"])
                if "se" in r:
                    # se_unit.cc:37-73: pool = mean + bias; fc1 with activation; fc2; first C outputs -> sigmoid
                    # scale, next C -> shift (+ scale * bias); out = act(scale * x + residual + shift)
                    se = r["se"]
                    c = bias.numel()
                    pool = t.mean(dim=(2, 3)) + bias
                    s = _fc(_fc(pool, se["w1"], se["b1"], act), se["w2"], se["b2"])
                    first, second = (s[:, c:], s[:, :c]) if self.perturb == "se_split" else (s[:, :c], s[:, c:])
                    gamma = torch.sigmoid(first)
                    beta = second + gamma * bias
                    flow = _act(gamma[:, :, None, None] * t + flow + beta[:, :, None, None], act)
                else:
                    flow = _act(flow + t + bias[None, :, None, None], act)      # BiasResidual
        x = None
        if self.attn_body:
            emb = len(w["ip_emb_b"])
            nhwc = planes.transpose(1, 2)                       # buffer3[b][i*input_size + j] = buffer1[b][j*64 + i]
            if self.pe_dense:
                enc = len(w["ip_emb_preproc_b"]) // 64
                pre = nhwc[:, :, :12]                           # buffer3[b][i*12 + j], network_blas.cc:616-624
                if self.perturb == "pe_dense_order":
                    pre = pre.transpose(1, 2)
                pe = _fc(pre.reshape(b, 64 * 12), w["ip_emb_preproc_w"], w["ip_emb_preproc_b"])
                pe = pe.reshape(b, 64, enc)                     # buffer2[b][i*enc + (j-112)], :645-650
            else:
                pe = _t(pos_encoding_table())[None].expand(b, 64, 64)
            x = _fc(torch.cat([nhwc, pe], dim=2), w["ip_emb_w"], w["ip_emb_b"], act)
            if self.pe_dense:
                x = _ln(x, 1.0, None, w["ip_emb_ln_gammas"], w["ip_emb_ln_betas"], 1e-3)
            if "ip_mult_gate" in w and "ip_add_gate" in w:
                # buffer1[b][i][j] * ip_mult_gate[j*64 + i] + ip_add_gate[j*64 + i], :670-682
                mult, add = _t(w["ip_mult_gate"]).reshape(emb, 64), _t(w["ip_add_gate"]).reshape(emb, 64)
                if self.perturb == "gating_transpose":
                    mult, add = _t(w["ip_mult_gate"]).reshape(64, emb).T, _t(w["ip_add_gate"]).reshape(64, emb).T
                x = x * mult.T[None] + add.T[None]
            alpha = float(np.float32(pow(2.0 * len(w["encoder"]), -0.25)))
            if self.pe_dense:
                ffn = w["ip_emb_ffn"]
                h = _fc(_fc(x, ffn["dense1_w"], ffn["dense1_b"], self.ffn_act), ffn["dense2_w"], ffn["dense2_b"])
                x = _ln(h, alpha, x, w["ip_emb_ffn_ln_gammas"], w["ip_emb_ffn_ln_betas"], 1e-3)
            eps = 1e-3 if self.pe_dense else 1e-6
            for layer in w["encoder"]:
                x = self._encoder_layer(x, layer, w["headcount"], self.smolgen_act, self.ffn_act, alpha, eps)
        out = {}
        vh = self._value_head()
        # Value head, network_blas.cc:725-772. Attention body: head_buffer[(b*64+sq)*planes + c], consumed by
        # Forward1D(batch, planes*64, ...) -> input index sq*planes + c. Tower: NCHW, index c*64 + sq.
        if self.attn_body:
            hv = _fc(x, vh["ip_val_w"], vh["ip_val_b"], act)
            if self.perturb == "value_flatten":
                hv = hv.transpose(1, 2)
            hv = hv.reshape(b, -1)
        else:
            hv = self._conv1(flow, vh["value"], act).reshape(b, -1)
        hv = _fc(hv, vh["ip1_val_w"], vh["ip1_val_b"], act)
        if self.nf["value"] == 2:
            out["wdl"] = torch.softmax(_fc(hv, vh["ip2_val_w"], vh["ip2_val_b"]), dim=1).numpy()
        else:
            out["q"] = torch.tanh(hv @ _t(vh["ip2_val_w"]).reshape(-1) + float(np.asarray(vh["ip2_val_b"])[0])).numpy()
        # Moves-left head, :775-803.
        if self.nf.get("moves_left", 0) == 1:
            if self.attn_body:
                hm = _fc(x, w["ip_mov_w"], w["ip_mov_b"], act)
                if self.perturb == "mlh_flatten":
                    hm = hm.transpose(1, 2)
                hm = hm.reshape(b, -1)
            else:
                hm = self._conv1(flow, w["moves_left"], act).reshape(b, -1)
            hm = _fc(hm, w["ip1_mov_w"], w["ip1_mov_b"], act)
            out["m"] = _fc(hm, w["ip2_mov_w"], w["ip2_mov_b"], "relu").reshape(b).numpy()
        else:
            out["m"] = np.zeros(b)
        # Policy head, :806-968.
        ph = self._policy_head()
        policy = np.zeros((b, 1858))
        if self.nf["policy"] == 3:
            if not self.attn_body:
                x = flow.reshape(b, -1, 64).transpose(1, 2)      # buffer1[b][i*C + j] = buffer2[b][j*64 + i]
            t = _fc(x, ph["ip_pol_w"], ph["ip_pol_b"], act if self.attn_body else "selu")
            for layer in ph.get("pol_encoder", []):
                t = self._encoder_layer(t, layer, ph["pol_headcount"],
                                        self.smolgen_act if self.attn_body else "none",
                                        self.ffn_act if self.attn_body else "selu", 1.0, 1e-6)
            pd = len(ph["ip2_pol_b"])
            q = _fc(t, ph["ip2_pol_w"], ph["ip2_pol_b"])         # A
            k = _fc(t, ph["ip3_pol_w"], ph["ip3_pol_b"])         # B
            scaling = 1.0 / float(np.sqrt(np.float32(pd)))
            # C[from][to] = scaling * sum_d A[from][d] * B[to][d]  (cblas_sgemm NoTrans, Trans, :864-866)
            logits = scaling * (k @ q.transpose(1, 2) if self.perturb == "policy_qk_transpose" else q @ k.transpose(1, 2))
            ppo = _t(ph["ip4_pol_w"]).reshape(4, pd)
            off = torch.einsum("bjd,id->bij", k[:, 56:64, :], ppo)      # promotion_offsets[i][j], :876-887
            off = off[:, :3, :] + off[:, 3:4, :]                         # :888-892
            buf = torch.zeros(b, 64 * 64 + 8 * 24, dtype=T)
            buf[:, :4096] = logits.reshape(b, 4096)
            for kk in range(8):
                for j in range(8):
                    for i in range(3):
                        idx = 4096 + (8 * i + 24 * kk + j if self.perturb == "promotion_index" else 24 * kk + 3 * j + i)
                        buf[:, idx] = logits[:, 48 + kk, 56 + j] + off[:, i, j]   # :893-903
            buf = buf.numpy()
            for i, j in enumerate(self.attn_map):                        # :905-915
                if j >= 0:
                    policy[:, j] = buf[:, i]
        elif self.nf["policy"] == 2:
            t = self._conv3(flow, ph["policy1"], act)
            t = self._conv3(t, ph["policy"], "none").reshape(b, -1).numpy()   # head_buffer[b][plane*64 + sq]
            for i, j in enumerate(self.conv_map):                        # :934-945
                if j >= 0:
                    policy[:, j] = t[:, i]
        else:
            t = self._conv1(flow, ph["policy"], act).reshape(b, -1)
            policy = _fc(t, ph["ip_pol_w"], ph["ip_pol_b"]).numpy()
        out["policy"] = policy
        return out
