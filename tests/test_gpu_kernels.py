"""Per-kernel parity on the GPU: each hand-written kernel, called through the C
ABI (include/lc0mi_kernels.h), against the oracle function it replaces on the
same seeded tensors. fp16 tolerances are stated per test."""
import numpy as np
import pytest

from oracle import netread as nr
from oracle import nn as onn

pytestmark = pytest.mark.gpu
f32 = np.float32


def _h(a):
    """Round to fp16 and back: what the kernel actually sees."""
    return np.asarray(a, np.float16).astype(f32)


@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (128, 128, 128), (192, 96, 176), (300, 3, 128), (7, 1858 // 2, 72),
                                   (1024, 256, 1024), (5, 8, 16)])
@pytest.mark.parametrize("act", [nr.ACT_NONE, nr.ACT_MISH, nr.ACT_SWISH, nr.ACT_RELU])
def test_gemm_vs_oracle_fc(m, n, k, act):
    from lc0_amd import kernels as K
    rng = np.random.default_rng(m * 7 + n * 3 + k + act)
    a = _h(rng.standard_normal((m, k)) * 0.5)
    w = _h(rng.standard_normal((n, k)) * 0.2)
    b = rng.standard_normal(n).astype(f32)
    want = onn.fc(a, w.reshape(-1), b, act)
    got = K.gemm(a, w, b, act=act, out_f32=True)
    # fp16 operands, fp32 accumulation, fp32 output: only summation order differs.
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)
    got16 = K.gemm(a, w, b, act=act).astype(f32)
    np.testing.assert_allclose(got16, want, rtol=2e-3, atol=2e-3)  # + one fp16 rounding of the output


def test_gemm_no_bias_scale_and_batched():
    from lc0_amd import kernels as K
    rng = np.random.default_rng(1)
    a = _h(rng.standard_normal((5, 64, 96)))
    w = _h(rng.standard_normal((5, 64, 96)))
    got = K.gemm(a, w, None, scale=0.125, out_f32=True)
    want = np.matmul(a, w.transpose(0, 2, 1)) * 0.125
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("m,n,k,split", [(256, 256, 2048, 8), (37, 130, 520, 3), (64, 64, 64, 4), (300, 8, 4096, 16)])
def test_gemm_splitk_vs_oracle_fc(m, n, k, split):
    from lc0_amd import kernels as K
    rng = np.random.default_rng(m + n + k)
    a = _h(rng.standard_normal((m, k)) * 0.5)
    w = _h(rng.standard_normal((n, k)) * 0.1)
    b = rng.standard_normal(n).astype(f32)
    got = K.gemm_splitk(a, w, b, split_k=split)
    np.testing.assert_allclose(got, onn.fc(a, w.reshape(-1), b, nr.ACT_NONE), rtol=3e-4, atol=3e-4)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7, 9, 10])
@pytest.mark.parametrize("m,n,k", [(2048, 1024, 256), (777, 200, 128), (300, 1858, 64), (64, 64, 192), (1000, 32, 256)])
def test_every_gemm_variant_vs_oracle_fc(variant, m, n, k):
    """Every tile variant (the three direct-to-LDS kernels and the two
    register-staged ones) on full and ragged M / N."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(m + n)
    a = _h(rng.standard_normal((m, k)) * 0.5)
    w = _h(rng.standard_normal((n, k)) * 0.1)
    b = rng.standard_normal(n).astype(f32)
    K.set_gemm_variant(variant)
    try:
        got = K.gemm(a, w, b, act=nr.ACT_MISH).astype(f32)
    finally:
        K.set_gemm_variant(-1)
    np.testing.assert_allclose(got, onn.fc(a, w.reshape(-1), b, nr.ACT_MISH), rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("m,n,k", [
    (1, 256, 2048),      # 16x16 panels, eight steps of 32 per wave in one round
    (64, 1024, 1536),    # 16x16 panels, six steps
    (64, 1536, 1024),    # 32x16 panels
    (7, 8192, 264),      # 16x32 panels, a last step of 8 values
    (64, 3072, 1024),    # 32x32 panels
    (512, 1024, 528),    # 64x32 panels, a last step of 16 values
    (100, 700, 4096),    # sixteen steps per wave: two rounds of eight
    (130, 600, 3392),    # fourteen steps per wave, a last wave with fewer
    (33, 50, 40),        # a single full step and a last step of 8 values
    (16, 16, 8),         # nothing but the last step
    (20000, 40, 512)])   # more panels than CUs: the largest panel shape
def test_row_panel_gemm_panel_shapes_and_reduction_tails(m, n, k):
    """The row-panel kernel (variant 6) picks its panel by problem size and its load depth by K: every panel shape,
    every depth, reductions that are not multiples of 32, half and float output, with activation and without bias,
    against FullyConnectedLayer::Forward1D (blas/fully_connected_layer.cc:49-106)."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(m * 5 + n * 3 + k)
    a = _h(rng.standard_normal((m, k)) * 0.5)
    w = _h(rng.standard_normal((n, k)) * 0.1)
    b = rng.standard_normal(n).astype(f32)
    K.set_gemm_variant(6)
    try:
        got32 = K.gemm(a, w, b, act=nr.ACT_MISH, out_f32=True)
        got16 = K.gemm(a, w, None, act=nr.ACT_NONE).astype(f32)
    finally:
        K.set_gemm_variant(-1)
    np.testing.assert_allclose(got32, onn.fc(a, w.reshape(-1), b, nr.ACT_MISH), rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(got16, onn.fc(a, w.reshape(-1), np.zeros(n, f32), nr.ACT_NONE), rtol=2e-3, atol=2e-3)


def test_gemm_automatic_choice_over_random_shapes():
    """The launcher picks the kernel by shape (row panels of five sizes, direct-to-LDS tiles of seven with two to four
    stages, register-staged tiles): sixty seeded shapes between 1x1x8 and 6000x4000x4096, ragged in every dimension,
    against FullyConnectedLayer::Forward1D (blas/fully_connected_layer.cc:49-106)."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(2718)
    for case in range(60):
        m = int(rng.choice([1, 3, 16, 17, 64, 100, 192, 256, 500, 1024, 3000, 6000]))
        n = int(rng.choice([1, 8, 31, 32, 64, 130, 256, 1000, 1024, 1858, 3072, 4000]))
        k = int(rng.choice([8, 24, 64, 128, 200, 256, 512, 1000, 1024, 1536, 4096]))
        if m * n * k > 6000 * 1024 * 1536:
            continue
        a = _h(rng.standard_normal((m, k)) * 0.5)
        w = _h(rng.standard_normal((n, k)) * (2.0 / np.sqrt(k)))
        b = rng.standard_normal(n).astype(f32)
        act = [nr.ACT_NONE, nr.ACT_MISH, nr.ACT_RELU][case % 3]
        want = onn.fc(a, w.reshape(-1), b, act)
        got = K.gemm(a, w, b, act=act).astype(f32)
        np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3, err_msg="shape %dx%dx%d" % (m, n, k))


def test_row_panel_gemm_batched_with_scale():
    from lc0_amd import kernels as K
    rng = np.random.default_rng(11)
    a = _h(rng.standard_normal((3, 40, 288)))
    w = _h(rng.standard_normal((3, 70, 288)))
    K.set_gemm_variant(6)
    try:
        got = K.gemm(a, w, None, scale=0.125, out_f32=True)
    finally:
        K.set_gemm_variant(-1)
    np.testing.assert_allclose(got, np.matmul(a, w.transpose(0, 2, 1)) * 0.125, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("rows,c,f32_in,act", [(256, 256, True, nr.ACT_SWISH), (256, 8192, False, nr.ACT_NONE),
                                               (3, 32, True, nr.ACT_MISH), (17, 1024, False, nr.ACT_RELU)])
def test_layer_norm_rows_vs_oracle(rows, c, f32_in, act):
    from lc0_amd import kernels as K
    rng = np.random.default_rng(rows * 3 + c)
    x = rng.standard_normal((rows, c)).astype(f32)
    if not f32_in:
        x = _h(x)
    s = _h(rng.standard_normal((rows, c)))
    g = (1 + 0.1 * rng.standard_normal(c)).astype(f32)
    b = (0.1 * rng.standard_normal(c)).astype(f32)
    want = onn.layer_norm_skip(onn.activate(x, act), 0.7, s, g, b, 1e-3)
    got = K.layer_norm_rows(x, s, g, b, 0.7, 1e-3, pre_act=act, x_is_f32=f32_in).astype(f32)
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)


def test_gemm_f32_vs_oracle_fc():
    from lc0_amd import kernels as K
    rng = np.random.default_rng(2)
    for m, n, k in [(64, 64, 64), (70, 33, 20), (513, 130, 256)]:
        a = rng.standard_normal((m, k)).astype(f32)
        w = rng.standard_normal((n, k)).astype(f32)
        b = rng.standard_normal(n).astype(f32)
        np.testing.assert_allclose(K.gemm_f32(a, w, b, act=nr.ACT_MISH), onn.fc(a, w, b, nr.ACT_MISH),
                                   rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("rows,c", [(64, 64), (300, 256), (128, 1024), (9, 8192), (5, 32)])
@pytest.mark.parametrize("with_skip", [True, False])
def test_layer_norm_vs_oracle(rows, c, with_skip):
    from lc0_amd import kernels as K
    rng = np.random.default_rng(rows + c)
    x = _h(rng.standard_normal((rows, c)))
    s = _h(rng.standard_normal((rows, c))) if with_skip else None
    g = (1 + 0.1 * rng.standard_normal(c)).astype(f32)
    b = (0.1 * rng.standard_normal(c)).astype(f32)
    want = onn.layer_norm_skip(x, 0.427, s, g, b, 1e-6)
    got = K.layer_norm(x, s, g, b, 0.427, 1e-6).astype(f32)
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)  # fp16 output rounding


@pytest.mark.parametrize("batch,heads", [(1, 1), (3, 2), (5, 8), (2, 32)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_attention_vs_oracle(batch, heads, with_bias):
    from lc0_amd import kernels as K
    rng = np.random.default_rng(batch * 100 + heads)
    d = heads * 32
    qkv = _h(rng.standard_normal((batch * 64, 3 * d)))
    bias = _h(rng.standard_normal((batch, heads, 64, 64)) * 2) if with_bias else None
    scale = 1.0 / np.sqrt(32.0)
    got = K.attention(qkv, bias, batch, heads, scale).astype(f32)
    q = qkv[:, :d].reshape(batch, 64, heads, 32).transpose(0, 2, 1, 3)
    k = qkv[:, d:2 * d].reshape(batch, 64, heads, 32).transpose(0, 2, 1, 3)
    v = qkv[:, 2 * d:].reshape(batch, 64, heads, 32).transpose(0, 2, 1, 3)
    s = np.matmul(q, k.transpose(0, 1, 3, 2)) * f32(scale)
    if bias is not None:
        s = bias + s
    p = onn.softmax_rows(s)
    want = np.matmul(p, v).transpose(0, 2, 1, 3).reshape(batch * 64, d)
    # probabilities are rounded to fp16 before P.V and the output is fp16.
    np.testing.assert_allclose(got, want, rtol=4e-3, atol=4e-3)


def test_expand_planes_bit_exact():
    from lc0_amd import kernels as K
    from oracle import chess as oc
    pos = oc.random_positions(33, seed=5)
    want = onn.encode_planes(pos["masks"], pos["values"])           # [B,112,64]
    got_nchw = K.expand_planes_nchw(pos["masks"], pos["values"])
    assert np.array_equal(got_nchw, want)
    got = K.expand_planes_attn(pos["masks"], pos["values"], 176).astype(f32).reshape(33, 64, 176)
    assert np.array_equal(got[:, :, :112], want.transpose(0, 2, 1))  # values <= 99 are exact in fp16
    assert np.array_equal(got[:, :, 112:176], np.broadcast_to(onn.POS_ENCODING, (33, 64, 64)))
    got_pad = K.expand_planes_attn(pos["masks"], pos["values"], 192).astype(f32).reshape(33, 64, 192)
    assert np.array_equal(got_pad[:, :, :176], got) and (got_pad[:, :, 176:] == 0).all()


def test_attn_policy_gather_vs_oracle():
    from lc0_amd import kernels as K
    rng = np.random.default_rng(3)
    B, pd = 4, 64
    logits = rng.standard_normal((B, 64, 64)).astype(f32)
    keys = _h(rng.standard_normal((B * 64, pd)))
    ppo = rng.standard_normal((4, pd)).astype(f32)
    got = K.attn_policy_gather(logits, keys, ppo)
    k3 = keys.reshape(B, 64, pd)
    off = np.einsum("bjk,ik->bij", k3[:, 56:64], ppo)
    off3 = off[:, :3] + off[:, 3:4]
    promo = logits[:, 48:56, 56:64][:, :, :, None] + off3.transpose(0, 2, 1)[:, None]
    buf = np.concatenate([logits.reshape(B, 4096), promo.reshape(B, 192)], axis=1)
    want = np.zeros((B, 1858), f32)
    sel = onn.ATTN_POLICY_MAP >= 0
    want[:, onn.ATTN_POLICY_MAP[sel]] = buf[:, sel]
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    # plain from->to logits are moved bit-exactly
    plain = onn.ATTN_POLICY_MAP[:4096]
    ps = plain >= 0
    assert np.array_equal(got[:, plain[ps]], logits.reshape(B, 4096)[:, ps])


@pytest.mark.parametrize("fp16", [False, True])
@pytest.mark.parametrize("batch,cin,cout,se_k,with_skip", [(3, 112, 32, 0, False), (2, 32, 32, 8, True),
                                                            (5, 64, 64, 16, True), (2, 16, 80, 0, False),
                                                            (1, 24, 24, 0, True)])
def test_winograd_conv_vs_oracle(batch, cin, cout, se_k, with_skip, fp16):
    """F(4x4,3x3) convolution with its fused tail against the oracle's convolution
    (itself checked against direct 3x3 correlation) and ApplySEUnit."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(batch + cin + cout + se_k)
    rnd = (lambda a: _h(a)) if fp16 else (lambda a: np.asarray(a, f32))
    x = rnd(rng.standard_normal((batch, cin, 8, 8)))                 # NCHW for the oracle
    filt = rnd(rng.standard_normal((cout, cin, 3, 3)) * (cin * 9) ** -0.5)
    bias = (0.1 * rng.standard_normal(cout)).astype(f32)
    skip = rnd(rng.standard_normal((batch, cout, 64))) if with_skip else None
    u = onn.winograd_filter_transform(filt, cout, cin)
    y = onn.winograd_conv3(x, u, cin, cout).reshape(batch, cout, 64)
    if se_k:
        se = (rng.standard_normal((se_k, cout)).astype(f32) * 0.3, rng.standard_normal(se_k).astype(f32) * 0.1,
              rng.standard_normal((2 * cout, se_k)).astype(f32) * 0.3, rng.standard_normal(2 * cout).astype(f32) * 0.1)
        want = onn.apply_se_unit(y, bias, skip if with_skip else np.zeros_like(y), *se, nr.ACT_RELU)
    else:
        se = None
        t = y + bias[None, :, None]
        if with_skip:
            t = t + skip
        want = onn.activate(t, nr.ACT_RELU)
    got = K.winograd_conv(x.reshape(batch, cin, 64).transpose(0, 2, 1), filt, bias,
                          skip.transpose(0, 2, 1) if with_skip else None, se, act=nr.ACT_RELU, fp16=fp16)
    got = got.transpose(0, 2, 1)
    if fp16:
        # Transformed inputs, filters and the winograd-domain products are all rounded to 11 bits, and
        # the inverse transform A^T (entries up to 8, i.e. 64 in two dimensions) amplifies the rounding of
        # the products: a few per cent of the output scale at the corner outputs of a tile, ~0.3 % rms.
        np.testing.assert_allclose(got, want, rtol=5e-2, atol=5e-2)
        assert np.sqrt(np.mean((got - want) ** 2)) <= 6e-3 * max(1.0, float(np.abs(want).max()))
    else:
        np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-4)


def test_expand_planes_nhwc_bit_exact():
    from lc0_amd import kernels as K
    from oracle import chess as oc
    pos = oc.random_positions(9, seed=6)
    want = onn.encode_planes(pos["masks"], pos["values"]).transpose(0, 2, 1)
    assert np.array_equal(K.expand_planes_nhwc(pos["masks"], pos["values"]), want)


# ---- e4m3 (fp8) kernels -----------------------------------------------------
def _f8_close(got_codes, want_values, mul, tol=2e-3):
    """Quantised outputs: the kernel quantises its own fp32 value, which differs from the oracle's by
    up to tol (absolute and relative, the bound of the unquantised tests); so the decoded code must
    lie within half an e4m3 step plus that of the oracle value, and nearly all codes must be equal."""
    from oracle import fp8
    got = fp8.e4m3_decode(got_codes).astype(np.float64)
    want = np.clip(np.asarray(want_values, np.float64) * mul, -448, 448)
    step = np.maximum(2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -6))) - 3), 2.0 ** -9)
    excess = np.abs(got - want) - (0.5 * step + tol * mul + tol * np.abs(want))
    assert excess.max() <= 0, excess.max()
    exact = fp8.e4m3_encode(want.astype(f32))
    assert (exact == got_codes).mean() > 0.97


def test_quantize_f8_bit_exact():
    """Every fp16 value (x scale) -> e4m3: bit-exact against the oracle codec (NaN inputs excluded:
    the reference maps them to 0x7f, the kernel's clamp to +-448)."""
    from lc0_amd import kernels as K
    from oracle import fp8
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    halves = halves[~np.isnan(halves)]
    halves = np.concatenate([halves, np.zeros((-len(halves)) % 8, np.float16)])
    for mul in (1.0, 0.37, 16.0):
        got = K.quantize_f8(halves, mul)
        want = fp8.e4m3_encode(halves.astype(f32) * f32(mul))
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("variant", [-1, 0, 1, 2, 5, 6, 7, 10])
@pytest.mark.parametrize("m,n,k", [(512, 512, 128), (300, 200, 256), (2048, 1536, 1024), (64, 3072, 1024), (1, 17, 128),
                                   (64, 1024, 1536), (64, 1536, 1024), (5, 8192, 256), (700, 40, 4096)])
def test_gemm_f8_vs_exact_product(variant, m, n, k):
    """e4m3 operands are exact inputs, so the product is pinned by float64 arithmetic on the decoded
    values; tolerance covers fp32 accumulation and the fp16 output rounding. Variant 6 is the row-panel kernel
    (the last four shapes and (64, 3072, 1024) take one panel shape each; one, two and four 128-wide k-steps per
    wave)."""
    from lc0_amd import kernels as K
    from oracle import fp8
    rng = np.random.default_rng(m + n + k)
    a = fp8.e4m3_encode(rng.standard_normal((m, k)) * 2)
    w, wscale = fp8.quantize_rows(rng.standard_normal((n, k)) * 0.05)
    b = rng.standard_normal(n).astype(f32)
    sa = f32(0.031)
    exact = (fp8.e4m3_decode(a).astype(np.float64) @ fp8.e4m3_decode(w).astype(np.float64).T) * (sa * wscale) + b
    K.set_gemm_variant(variant)
    try:
        got = K.gemm_f8(a, w, sa * wscale, b).astype(np.float64)
        np.testing.assert_allclose(got, exact, rtol=2e-3, atol=2e-3)
        want_act = onn.activate(exact.astype(f32), nr.ACT_MISH)
        got8 = K.gemm_f8(a, w, sa * wscale, b, act=nr.ACT_MISH, out_f8=True, out_mul=20.0)
        _f8_close(got8, want_act, 20.0)
    finally:
        K.set_gemm_variant(-1)


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("stores", ["cached", "stream", "write_through", "auto_keep"])
def test_output_store_kinds_give_the_same_result(stores, variant):
    """The 256-row tiles write a large output with ordinary, streaming or written-through stores, and the layer norm
    reads and writes through: every kind must give the bits of the default (here: streaming by the size rule for
    the GEMMs, ordinary loads and stores for the layer norm), which is held to the oracle on some rows. Variants:
    the 256x256, 256x192 and 256x128 tiles."""
    from lc0_amd import kernels as K
    from oracle import fp8
    kind = {"cached": K.STORES_CACHED, "stream": K.STORES_STREAM, "write_through": K.STORES_WRITE_THROUGH,
            "auto_keep": K.STORES_AUTO_KEEP}[stores]
    rng = np.random.default_rng(11)
    m, n, k = 16384, 1024, 128                       # 32 MiB of half output from 16384 rows: the size rule's edge
    a = _h(rng.standard_normal((m, k)) * 0.5)
    w = _h(rng.standard_normal((n, k)) * 0.2)
    b = rng.standard_normal(n).astype(f32)
    a8 = fp8.e4m3_encode(rng.standard_normal((m, k)) * 2)
    w8, wscale = fp8.quantize_rows(rng.standard_normal((n, k)) * 0.05)
    x = _h(rng.standard_normal((4096, 1024)))
    g, be = rng.standard_normal(1024).astype(f32), rng.standard_normal(1024).astype(f32)
    K.set_gemm_variant(variant)
    try:
        want = K.gemm(a, w, b)
        want8 = K.gemm_f8(a8, w8, f32(0.031) * wscale, b)
        want_ln = K.layer_norm(x, x, g, be, 0.5, 1e-6)
        K.set_out_stores(kind)
        got = K.gemm(a, w, b)
        got8 = K.gemm_f8(a8, w8, f32(0.031) * wscale, b)
        got_ln = K.layer_norm(x, x, g, be, 0.5, 1e-6)
    finally:
        K.set_out_stores(K.STORES_AUTO)
        K.set_gemm_variant(-1)
    np.testing.assert_allclose(want.astype(f32)[-512:], onn.fc(a[-512:], w.reshape(-1), b, nr.ACT_NONE), rtol=2e-3,
                               atol=2e-3)
    assert np.array_equal(got, want)
    assert np.array_equal(got8, want8)
    assert np.array_equal(got_ln, want_ln)


@pytest.mark.parametrize("m,n,k", [(20480, 1024, 1536), (20481, 1024, 1024), (24576, 1000, 1024)])
def test_product_cut_along_its_rows_equals_one_launch(m, n, k):
    """A product whose tiles leave a partial round is cut into whole rounds of large tiles and a rest on another tile
    shape. The first part carries the bits of one launch of the large tiles; in the rest a few outputs per million
    that sit on a half-precision tie fall the other way (the compiler rounds scale * acc + bias once, straight to
    half, in some places of one kernel instance and twice, through float, in another): at most one half-precision
    step, in at most 2e-5 of the outputs. Rows of both parts and of
    the seam against the oracle's layer."""
    from lc0_amd import kernels as K
    m1 = K.gemm_row_split(m, n, k)
    assert 0 < m1 < m, "this shape is meant to be cut"
    rng = np.random.default_rng(m + n)
    a = _h(rng.standard_normal((m, k)) * 0.5)
    w = _h(rng.standard_normal((n, k)) * 0.1)
    b = rng.standard_normal(n).astype(f32)
    got = K.gemm(a, w, b, 0.5, nr.ACT_MISH)
    K.set_gemm_variant(0)
    try:
        want = K.gemm(a, w, b, 0.5, nr.ACT_MISH)
    finally:
        K.set_gemm_variant(-1)
    assert np.array_equal(got[:m1], want[:m1])
    differ = got[m1:] != want[m1:]
    assert differ.mean() <= 2e-5, differ.sum()
    steps = np.abs(got[m1:].view(np.int16).astype(np.int32) - want[m1:].view(np.int16).astype(np.int32))
    assert steps.max() <= 1   # neighbouring half values (same sign: a tie near zero does not occur with this bias)
    rows = np.r_[0:64, m1 - 64:m1 + 64, m - 64:m]
    np.testing.assert_allclose(got[rows].astype(f32), _fc_scaled(a[rows], w, b, 0.5, nr.ACT_MISH), rtol=3e-3, atol=3e-3)


def _fc_scaled(a, w, b, scale, act):
    """act(scale * a w^T + b) in float64 through the oracle's activation."""
    z = scale * (a.astype(np.float64) @ w.astype(np.float64).T) + b
    return onn.activate(z.astype(f32), act)


def test_cold_cache_timing_hook_leaves_results_alone():
    """The profiling hook times launches one by one behind a cache-flushing copy: same output, a positive time."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(5)
    x = rng.standard_normal((512, 256), dtype=np.float32).astype(np.float16)
    g, b = np.ones(256, np.float32), np.zeros(256, np.float32)
    warm, ms_warm = K.layer_norm(x, x, g, b, 0.5, 1e-6, time_iters=3)
    K.set_cold_cache(64)
    try:
        cold, ms_cold = K.layer_norm(x, x, g, b, 0.5, 1e-6, time_iters=3)
    finally:
        K.set_cold_cache(0)
    assert np.array_equal(warm, cold)
    assert ms_warm > 0 and ms_cold > 0


def test_layer_norm_f8_output():
    from lc0_amd import kernels as K
    rng = np.random.default_rng(77)
    x = _h(rng.standard_normal((200, 1024)))
    s = _h(rng.standard_normal((200, 1024)))
    g = (1 + 0.1 * rng.standard_normal(1024)).astype(f32)
    b = (0.1 * rng.standard_normal(1024)).astype(f32)
    want = onn.layer_norm_skip(x, 0.427, s, g, b, 1e-6)
    y, yq = K.layer_norm_f8(x, s, g, b, 0.427, 1e-6, 50.0)
    np.testing.assert_allclose(y.astype(f32), want, rtol=2e-3, atol=2e-3)
    _f8_close(yq, want, 50.0)
    np.testing.assert_array_equal(y, K.layer_norm(x, s, g, b, 0.427, 1e-6))   # the fp16 output is unchanged


def test_attention_f8_output_matches_half_output():
    from lc0_amd import kernels as K
    from oracle import fp8
    rng = np.random.default_rng(78)
    batch, heads = 3, 4
    qkv = _h(rng.standard_normal((batch * 64, 3 * heads * 32)))
    bias = _h(rng.standard_normal((batch, heads, 64, 64)))
    half_out = K.attention(qkv, bias, batch, heads, 32 ** -0.5).astype(f32)
    got = K.attention_f8(qkv, bias, batch, heads, 32 ** -0.5, 100.0)
    _f8_close(got, half_out, 100.0)   # same fp32 result, rounded to e4m3 instead of fp16 (fp16 error << e4m3 step)


def _smolgen_attention_reference(qkv, gen, w, batch, heads, scale):
    """float32 numpy: the generator layer (logits as halves, as the separate GEMM stores them), then the attention."""
    d = heads * 32
    logits = (gen.astype(f32).reshape(batch * heads, -1) @ w.astype(f32).T).astype(np.float16).astype(f32)
    logits = logits.reshape(batch, heads, 64, 64)
    q = qkv[:, :d].astype(f32).reshape(batch, 64, heads, 32).transpose(0, 2, 1, 3)
    k = qkv[:, d:2 * d].astype(f32).reshape(batch, 64, heads, 32).transpose(0, 2, 1, 3)
    v = qkv[:, 2 * d:].astype(f32).reshape(batch, 64, heads, 32).transpose(0, 2, 1, 3)
    p = onn.softmax_rows(np.matmul(q, k.transpose(0, 1, 3, 2)) * f32(scale) + logits)
    return np.matmul(p, v).transpose(0, 2, 1, 3).reshape(batch * 64, d), logits


@pytest.mark.parametrize("batch,heads,gen_sz", [(1, 2, 32), (2, 4, 32), (5, 8, 128), (4, 32, 256), (7, 32, 256),
                                                (19, 24, 256), (3, 1, 32), (6, 3, 128), (9, 31, 256)])
def test_smolgen_attention_vs_oracle(batch, heads, gen_sz):
    """The generator layer inside the attention kernel (network_blas.cc:332-347 + :352-439): odd batches (a sample
    pair with one sample), fewer than 32 heads (unused matrix columns), odd head counts (a last head without a
    neighbour in its 128-byte rows) and every generator width; also against the two separate kernels, whose logits
    make the same round trip through halves."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(batch * 1000 + heads * 10 + gen_sz)
    d = heads * 32
    qkv = _h(rng.standard_normal((batch * 64, 3 * d)))
    gen = _h(rng.standard_normal((batch, heads, gen_sz)))
    w = _h(rng.standard_normal((4096, gen_sz)) * (2.0 / np.sqrt(gen_sz)))
    scale = 1.0 / np.sqrt(32.0)
    want, logits = _smolgen_attention_reference(qkv, gen, w, batch, heads, scale)
    got = K.smolgen_attention(qkv, gen, w, batch, heads, scale).astype(f32)
    np.testing.assert_allclose(got, want, rtol=4e-3, atol=4e-3)   # probabilities and output are rounded to fp16
    separate = K.attention(qkv, _h(logits), batch, heads, scale).astype(f32)
    np.testing.assert_allclose(got, separate, rtol=0, atol=4e-3)


def test_smolgen_attention_f8_output():
    from lc0_amd import kernels as K
    rng = np.random.default_rng(79)
    batch, heads, gen_sz = 3, 4, 32
    qkv = _h(rng.standard_normal((batch * 64, 3 * heads * 32)))
    gen = _h(rng.standard_normal((batch, heads, gen_sz)))
    w = _h(rng.standard_normal((4096, gen_sz)) * 0.3)
    half_out = K.smolgen_attention(qkv, gen, w, batch, heads, 32 ** -0.5).astype(f32)
    got = K.smolgen_attention(qkv, gen, w, batch, heads, 32 ** -0.5, f8_out=True, out_mul=100.0)
    _f8_close(got, half_out, 100.0)


@pytest.mark.parametrize("depth", [64, 128])
def test_attention_head_depths(depth):
    from lc0_amd import kernels as K
    rng = np.random.default_rng(depth)
    batch, heads = 3, 3
    d = heads * depth
    qkv = _h(rng.standard_normal((batch * 64, 3 * d)))
    bias = _h(rng.standard_normal((batch, heads, 64, 64)))
    scale = 1.0 / np.sqrt(float(depth))
    got = K.attention(qkv, bias, batch, heads, scale, depth=depth).astype(f32)
    q = qkv[:, :d].reshape(batch, 64, heads, depth).transpose(0, 2, 1, 3)
    k = qkv[:, d:2 * d].reshape(batch, 64, heads, depth).transpose(0, 2, 1, 3)
    v = qkv[:, 2 * d:].reshape(batch, 64, heads, depth).transpose(0, 2, 1, 3)
    p = onn.softmax_rows(bias + np.matmul(q, k.transpose(0, 1, 3, 2)) * f32(scale))
    want = np.matmul(p, v).transpose(0, 2, 1, 3).reshape(batch * 64, d)
    np.testing.assert_allclose(got, want, rtol=4e-3, atol=4e-3)


@pytest.mark.parametrize("fp16", [True, False])
@pytest.mark.parametrize("batch,c,se_k,with_skip", [(3, 32, 8, True), (2, 64, 0, False), (5, 256, 64, True)])
def test_fused_output_input_transform_equals_separate_kernels(batch, c, se_k, with_skip, fp16):
    """The output transform that also produces the next convolution's transformed input must give
    exactly what the stand-alone input transform gives on the stored activations (fp32 at 256
    channels does not fit the fused kernel's LDS budget and is refused)."""
    from lc0_amd import BackendError, kernels as K
    rng = np.random.default_rng(batch + c)
    x = rng.standard_normal((batch, 64, c)).astype(f32)
    filt = (rng.standard_normal((c, c, 3, 3)) * (c * 9) ** -0.5).astype(f32)
    bias = (0.1 * rng.standard_normal(c)).astype(f32)
    skip = rng.standard_normal((batch, 64, c)).astype(f32) if with_skip else None
    se = None
    if se_k:
        se = (rng.standard_normal((se_k, c)).astype(f32) * 0.3, rng.standard_normal(se_k).astype(f32) * 0.1,
              rng.standard_normal((2 * c, se_k)).astype(f32) * 0.3, rng.standard_normal(2 * c).astype(f32) * 0.1)
    if not fp16 and c == 256:
        with pytest.raises(BackendError, match="cannot be fused"):
            K.winograd_conv(x, filt, bias, skip, se, fp16=fp16, fused_next=True)
        return
    out, vf, vs = K.winograd_conv(x, filt, bias, skip, se, fp16=fp16, fused_next=True)
    np.testing.assert_array_equal(vf, vs)
    np.testing.assert_array_equal(out, K.winograd_conv(x, filt, bias, skip, se, fp16=fp16))
    assert np.abs(vf).max() > 0.1


def test_legal_softmax_bit_exact_vs_oracle():
    """legal_softmax_kernel against SoftmaxPolicy's restatement (oracle/nn.py: FastExp pinned on the
    compiled reference header): list lengths around the wave size and the 256 limit, an empty list,
    equal logits, logits so far below the maximum that FastExp returns 0, and several temperatures."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(11)
    lens = [0, 1, 2, 35, 63, 64, 65, 128, 218, 255, 256, 20, 31]
    policy = (rng.standard_normal((len(lens), 1858)) * 3).astype(f32)
    policy[3, :] = 0.25                              # all equal
    policy[4, ::2] = -1.0e4                          # FastExp underflow branch (a < -126)
    policy[5, :] = -3.0e38
    policy[5, 17] = 3.0e38                           # difference overflows to -inf
    lists = [rng.permutation(1858)[:n] for n in lens]
    lists[5][0] = 17
    for t in (1.359, 1.0, 0.37, 2.2, 10.0):
        got = K.legal_softmax(policy, lists, t)
        for i, ids in enumerate(lists):
            want = onn.softmax_policy_legal(policy[i], ids, t)
            np.testing.assert_array_equal(got[i].view(np.uint32), want.view(np.uint32), err_msg="row %d T %g" % (i, t))


def _fold_norm_into_layer(w, b, gamma, beta):
    """Host-side preparation of a layer that follows a layer norm: weights times gamma (as halves), their row sums
    as stored, and the bias plus the beta term."""
    wg = np.asarray(w.astype(np.float64) * gamma[None, :], np.float16)
    c = wg.astype(np.float64).sum(axis=1).astype(f32)
    d = (b.astype(np.float64) + w.astype(np.float64) @ beta.astype(np.float64)).astype(f32)
    return wg, c, d


@pytest.mark.parametrize("m,n,k,n2,act,skip_is_sum", [
    (16384, 1024, 1024, 1536, nr.ACT_MISH, True),    # 256x256 producer, 256x192 consumer (the BT4 shapes)
    (2048, 1024, 1536, 3072, nr.ACT_NONE, True),
    (2100, 512, 256, 32, nr.ACT_NONE, False),        # ragged rows; the consumer is a single 32-column panel
    (4096, 256, 128, 256, nr.ACT_RELU, True),        # 128x64 tiles: four lanes per row in the producer
    (4096, 768, 768, 64, nr.ACT_SWISH, False),
    (4096, 320, 256, 128, nr.ACT_NONE, True),        # row length no multiple of any column tile: the last tile's
    (4200, 200, 128, 64, nr.ACT_MISH, False),        # columns past N must stay out of the row statistics
])
def test_layer_norm_folded_into_the_gemms_around_it(m, n, k, n2, act, skip_is_sum):
    """x1 = LN(alpha * (a . w1 + b1) + s) followed by act(x1 . w2 + b2), against the oracle's dense layer and
    layer norm (LayerNorm2DWithSkipConnection), with the norm computed inside the two GEMMs: the first leaves the
    un-normalised sum and its row sums, the second normalises its product. s is either given, or itself the layer
    norm of an un-normalised sum s0 whose statistics and gamma / beta the first GEMM receives."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(m + 3 * n + 5 * k + n2)
    eps, alpha = 1e-6, 0.43
    a = _h(rng.standard_normal((m, k)) * 0.5)
    w1 = _h(rng.standard_normal((n, k)) * (1.0 / np.sqrt(k)))
    b1 = (rng.standard_normal(n) * 0.1).astype(f32)
    g1 = (1.0 + 0.2 * rng.standard_normal(n)).astype(f32)
    be1 = (0.1 * rng.standard_normal(n)).astype(f32)
    w2 = _h(rng.standard_normal((n2, n)) * (1.0 / np.sqrt(n)))
    b2 = (rng.standard_normal(n2) * 0.1).astype(f32)
    s0 = _h(rng.standard_normal((m, n)) * 1.5 + 0.7 * rng.standard_normal((m, 1)))   # rows with a mean of their own
    g0 = (1.0 + 0.2 * rng.standard_normal(n)).astype(f32)
    be0 = (0.1 * rng.standard_normal(n)).astype(f32)
    if skip_is_sum:
        s0_stats = np.stack([s0.sum(axis=1), (s0.astype(np.float64) ** 2).sum(axis=1)], axis=1).astype(f32)
        # as three partial sums per row, the last two empty, to exercise the addition of parts
        s0_stats = np.concatenate([s0_stats[:, None, :], np.zeros((m, 2, 2), f32)], axis=1)
        s = onn.layer_norm_skip(s0, 1.0, None, g0, be0, eps)
        u, stats = K.gemm_norm_producer(a, w1, b1 * alpha, s0, scale=alpha, skip_stats=s0_stats, skip_gamma=g0,
                                        skip_beta=be0, eps=eps)
    else:
        s = s0
        u, stats = K.gemm_norm_producer(a, w1, b1 * alpha, s0, scale=alpha, eps=eps)
    t = onn.fc(a, w1.reshape(-1), b1, nr.ACT_NONE)
    want_u = alpha * t + s
    u32 = u.astype(f32)
    # two roundings to half on the way (the product, then the sum)
    np.testing.assert_allclose(u32, want_u, rtol=3e-3, atol=3e-3)
    # the row sums describe U as stored, up to the rounding of its n elements to half (2^-11 relative each, taken
    # before the rounding: six standard deviations of the accumulated rounding errors are about 0.1 for the sums)
    np.testing.assert_allclose(stats[:, :, 0].sum(axis=1), u32.astype(np.float64).sum(axis=1), rtol=1e-4, atol=0.1)
    np.testing.assert_allclose(stats[:, :, 1].sum(axis=1), (u32.astype(np.float64) ** 2).sum(axis=1), rtol=1e-3)
    # consumer: against the oracle's layer norm of the stored U followed by its dense layer
    wg, c, d = _fold_norm_into_layer(w2, b2, g1, be1)
    got = K.gemm_norm_consumer(u, wg, c, d, stats, eps=eps, act=act, latency_first=(n2 <= 32)).astype(f32)
    x1 = onn.layer_norm_skip(u32, 1.0, None, g1, be1, eps)
    want = onn.fc(x1, w2.reshape(-1), b2, act)
    # fp16 output, gamma-scaled weights rounded to half once more: 3e-3 of the output scale (about 1)
    np.testing.assert_allclose(got, want, rtol=4e-3, atol=4e-3)
    # and the pair against the unfused pair of kernels on the same inputs
    t16 = K.gemm(a, w1, b1)
    x1_k = K.layer_norm(t16, s.astype(np.float16), g1, be1, alpha, eps)
    ref_pair = K.gemm(x1_k, w2, b2, act=act).astype(f32)
    assert np.abs(got - want).max() <= 2.0 * np.abs(ref_pair - want).max() + 2e-3


@pytest.mark.parametrize("producer_variant,consumer_variant", [(0, 1), (2, 2), (5, 5), (7, 7), (0, 3), (7, 4), (2, 0)])
def test_layer_norm_folding_in_every_gemm_variant_that_has_it(producer_variant, consumer_variant):
    """The same pair as above on one shape with the kernel variants forced: every direct-to-LDS tile shape as
    producer (except 256x192, which the choice never takes for one) and every variant as consumer."""
    from lc0_amd import kernels as K
    m, n, k, n2 = 2100, 512, 256, 384
    rng = np.random.default_rng(producer_variant * 16 + consumer_variant)
    eps, alpha = 1e-6, 0.5
    a = _h(rng.standard_normal((m, k)) * 0.5)
    w1 = _h(rng.standard_normal((n, k)) * (1.0 / np.sqrt(k)))
    b1 = (rng.standard_normal(n) * 0.1).astype(f32)
    g1 = (1.0 + 0.2 * rng.standard_normal(n)).astype(f32)
    be1 = (0.1 * rng.standard_normal(n)).astype(f32)
    w2 = _h(rng.standard_normal((n2, n)) * (1.0 / np.sqrt(n)))
    b2 = (rng.standard_normal(n2) * 0.1).astype(f32)
    s = _h(rng.standard_normal((m, n)) + 0.5 * rng.standard_normal((m, 1)))
    wg, c, d = _fold_norm_into_layer(w2, b2, g1, be1)
    try:
        K.set_gemm_variant(producer_variant)
        u, stats = K.gemm_norm_producer(a, w1, b1 * alpha, s, scale=alpha, eps=eps)
        K.set_gemm_variant(consumer_variant)
        got = K.gemm_norm_consumer(u, wg, c, d, stats, eps=eps, act=nr.ACT_MISH).astype(f32)
    finally:
        K.set_gemm_variant(-1)
    assert stats.shape[1] == -(-n // {0: 256, 2: 128, 5: 128, 7: 64}[producer_variant])
    u32 = u.astype(f32)
    np.testing.assert_allclose(u32, alpha * onn.fc(a, w1.reshape(-1), b1, nr.ACT_NONE) + s, rtol=3e-3, atol=3e-3)
    want = onn.fc(onn.layer_norm_skip(u32, 1.0, None, g1, be1, eps), w2.reshape(-1), b2, nr.ACT_MISH)
    np.testing.assert_allclose(got, want, rtol=4e-3, atol=4e-3)


# ---- bfloat16 instances of the 16-bit kernels, and the general (any type, any shape) kernels ----------------------
def _bf(a):
    """Values rounded to bfloat16, as float32."""
    from lc0_amd import kernels as K
    return K.from_bf16(K.to_bf16(a))


@pytest.mark.parametrize("variant", [-1, 0, 1, 2, 3, 4, 5, 7, 9, 10])
@pytest.mark.parametrize("m,n,k", [(2048, 1024, 256), (777, 200, 128), (300, 1858, 64), (1000, 32, 256)])
def test_every_gemm_variant_in_bf16_vs_oracle_fc(variant, m, n, k):
    """Every tile shape of the dense-layer kernels with bfloat16 operands (v_mfma_f32_32x32x16_bf16, fp32
    accumulation, bfloat16 output) against the oracle's Forward1D on the same bfloat16-rounded inputs. The only
    difference allowed is the rounding of the output to 8 significant bits and the summation order."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(variant * 7 + m + n + k)
    a = _bf(rng.standard_normal((m, k)) * 0.5)
    w = _bf(rng.standard_normal((n, k)) * 0.1)
    b = rng.standard_normal(n).astype(f32)
    want = onn.fc(a, w.reshape(-1), b, nr.ACT_MISH)
    try:
        K.set_gemm_variant(variant)
        with K.bf16():
            got = K.gemm(a, w, b, act=nr.ACT_MISH)
            got_f32 = K.gemm(a, w, b, act=nr.ACT_NONE, out_f32=True)
    finally:
        K.set_gemm_variant(-1)
    np.testing.assert_allclose(got, want, rtol=2.0 ** -7, atol=2e-3)          # one rounding to bfloat16 (2^-9) and slack
    np.testing.assert_allclose(got_f32, onn.fc(a, w.reshape(-1), b, nr.ACT_NONE), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("rows,c", [(300, 256), (128, 1024), (9, 8192)])
def test_layer_norms_in_bf16_vs_oracle(rows, c):
    from lc0_amd import kernels as K
    rng = np.random.default_rng(rows + c)
    x, s = _bf(rng.standard_normal((rows, c))), _bf(rng.standard_normal((rows, c)) * 0.5)
    g, b = (1 + 0.1 * rng.standard_normal(c)).astype(f32), (0.1 * rng.standard_normal(c)).astype(f32)
    want = onn.layer_norm_skip(x, 0.7, s, g, b, 1e-6)
    with K.bf16():
        got = K.layer_norm(x, s, g, b, 0.7, 1e-6)
        got_rows = K.layer_norm_rows(x, s, g, b, 0.7, 1e-6)
    np.testing.assert_allclose(got, want, rtol=2.0 ** -7, atol=2.0 ** -8)
    np.testing.assert_allclose(got_rows, want, rtol=2.0 ** -7, atol=2.0 ** -8)


@pytest.mark.parametrize("batch,heads,depth", [(3, 2, 32), (2, 4, 64), (2, 2, 128)])
def test_attention_in_bf16_vs_oracle(batch, heads, depth):
    from lc0_amd import kernels as K
    rng = np.random.default_rng(batch * 100 + heads + depth)
    d = heads * depth
    qkv = _bf(rng.standard_normal((batch * 64, 3 * d)))
    bias = _bf(rng.standard_normal((batch, heads, 64, 64)) * 2)
    scale = 1.0 / np.sqrt(float(depth))
    q, k, v = (qkv[:, i * d:(i + 1) * d].reshape(batch, 64, heads, depth).transpose(0, 2, 1, 3) for i in range(3))
    p = onn.softmax_rows(np.matmul(q, k.transpose(0, 1, 3, 2)) * f32(scale) + bias)
    want = np.matmul(p, v).transpose(0, 2, 1, 3).reshape(batch * 64, d)
    with K.bf16():
        got = K.attention(qkv, bias, batch, heads, scale, depth=depth)
    # probabilities and the output are rounded to bfloat16 (2^-9 each)
    np.testing.assert_allclose(got, want, rtol=2.0 ** -6, atol=2.0 ** -6)


def test_smolgen_attention_in_bf16_vs_reference():
    from lc0_amd import kernels as K
    batch, heads, gen_sz = 6, 32, 256
    rng = np.random.default_rng(77)
    d = heads * 32
    qkv = _bf(rng.standard_normal((batch * 64, 3 * d)))
    gen = _bf(rng.standard_normal((batch, heads, gen_sz)))
    w = _bf(rng.standard_normal((4096, gen_sz)) * (2.0 / np.sqrt(gen_sz)))
    scale = 1.0 / np.sqrt(32.0)
    logits = _bf(gen.reshape(batch * heads, -1) @ w.T).reshape(batch, heads, 64, 64)   # kept as bfloat16 in LDS
    q, k, v = (qkv[:, i * d:(i + 1) * d].reshape(batch, 64, heads, 32).transpose(0, 2, 1, 3) for i in range(3))
    p = onn.softmax_rows(np.matmul(q, k.transpose(0, 1, 3, 2)) * f32(scale) + logits)
    want = np.matmul(p, v).transpose(0, 2, 1, 3).reshape(batch * 64, d)
    with K.bf16():
        got = K.smolgen_attention(qkv, gen, w, batch, heads, scale)
    np.testing.assert_allclose(got, want, rtol=2.0 ** -5, atol=2.0 ** -5)


@pytest.mark.parametrize("dtype,tol", [("float", 2e-6), ("half", 2e-3), ("bf16", 2.0 ** -7)])
@pytest.mark.parametrize("batch,heads,depth,with_bias", [(2, 3, 48, True), (1, 2, 20, False), (2, 2, 128, True),
                                                         (3, 4, 32, True)])
def test_general_attention_kernel_vs_oracle(dtype, tol, batch, heads, depth, with_bias):
    """attention_generic_kernel: head depths the matrix-core kernel does not take, every element type (float:
    the reference's arithmetic, agreement to rounding)."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(batch + 10 * heads + depth)
    rnd = {"float": lambda a: a.astype(f32), "half": lambda a: _h(a).astype(f32), "bf16": _bf}[dtype]
    d = heads * depth
    qkv = rnd(rng.standard_normal((batch * 64, 3 * d)))
    bias = rnd(rng.standard_normal((batch, heads, 64, 64)) * 2) if with_bias else None
    scale = 1.0 / np.sqrt(float(depth))
    q, k, v = (qkv[:, i * d:(i + 1) * d].reshape(batch, 64, heads, depth).transpose(0, 2, 1, 3) for i in range(3))
    s = np.matmul(q, k.transpose(0, 1, 3, 2)) * f32(scale)
    p = onn.softmax_rows(s + bias if with_bias else s)
    want = np.matmul(p, v).transpose(0, 2, 1, 3).reshape(batch * 64, d)
    got = K.attention_generic(qkv, bias, batch, heads, depth, scale, dtype=dtype)
    np.testing.assert_allclose(got, want, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype,tol", [("float", 2e-6), ("half", 2e-3), ("bf16", 2.0 ** -7)])
@pytest.mark.parametrize("rows,c,act", [(37, 100, nr.ACT_NONE), (5, 8200, nr.ACT_SWISH), (64, 36, nr.ACT_MISH)])
def test_general_layer_norm_kernel_vs_oracle(dtype, tol, rows, c, act):
    """layer_norm_generic_kernel: row lengths that are no multiple of 8 or exceed 8192, an activation applied first."""
    from lc0_amd import kernels as K
    rng = np.random.default_rng(rows + c)
    rnd = {"float": lambda a: a.astype(f32), "half": lambda a: _h(a).astype(f32), "bf16": _bf}[dtype]
    x, s = rnd(rng.standard_normal((rows, c))), rnd(rng.standard_normal((rows, c)) * 0.5)
    g, b = (1 + 0.1 * rng.standard_normal(c)).astype(f32), (0.1 * rng.standard_normal(c)).astype(f32)
    want = onn.layer_norm_skip(onn.activate(x, act), 0.6, s, g, b, 1e-3)
    got = K.layer_norm_generic(x, s, g, b, 0.6, 1e-3, pre_act=act, dtype=dtype)
    np.testing.assert_allclose(got, want, rtol=tol, atol=2 * tol)
