"""numpy front end of the single-kernel entry points (include/lc0mi_kernels.h).

Each function runs exactly one gfx950 kernel of the forward pass on host
arrays; used by the per-kernel parity tests and micro-benchmarks.
"""
import ctypes as C

import numpy as np

from .backend import BackendError, load_library

ACT_MISH, ACT_RELU, ACT_NONE, ACT_TANH, ACT_SIGMOID, ACT_SELU, ACT_SWISH, ACT_RELU_2 = 1, 2, 3, 4, 5, 6, 7, 8


def _lib():
    lib = load_library()
    if not getattr(lib, "_k_ready", False):
        vp, ci, ll, cf, cd = C.c_void_p, C.c_int, C.c_longlong, C.c_float, C.POINTER(C.c_double)
        lib.lc0mi_k_gemm.argtypes = [vp, ci, ll, vp, ci, ll, vp, ci, ci, ci, ci, cf, ci, ci, vp, ci, ll, ci, cd]
        lib.lc0mi_k_gemm_splitk.argtypes = [vp, ci, vp, ci, vp, ci, ci, ci, ci, cf, vp, ci]
        lib.lc0mi_k_gemm_variant_name.argtypes = [ci, ci, ci, ci, ci]
        lib.lc0mi_k_gemm_variant_name.restype = C.c_char_p
        lib.lc0mi_k_gemm_row_split.argtypes = [ci, ci, ci]
        lib.lc0mi_k_set_gemm_row_split.argtypes = [ci]
        lib.lc0mi_k_set_gemm_row_split.restype = None
        lib.lc0mi_k_gemm_norm_producer.argtypes = [vp, ci, vp, ci, vp, ci, ci, ci, cf, vp, vp, ci, vp, vp, cf, vp, vp, ci,
                                                   C.POINTER(C.c_int), ci, cd]
        lib.lc0mi_k_gemm_norm_consumer.argtypes = [vp, ci, vp, ci, vp, vp, ci, ci, ci, vp, ci, cf, ci, ci, vp, ci, ci, cd]
        lib.lc0mi_k_layer_norm_rows.argtypes = [vp, vp, ci, vp, vp, vp, ci, ci, cf, cf, vp]
        lib.lc0mi_k_winograd_conv.argtypes = [vp] * 8 + [ci] * 6 + [vp] * 3
        lib.lc0mi_k_expand_planes_nhwc.argtypes = [vp, vp, ci, vp]
        lib.lc0mi_k_gemm_f32.argtypes = [vp, ci, vp, ci, vp, ci, ci, ci, cf, ci, vp, ci]
        lib.lc0mi_k_layer_norm.argtypes = [vp, vp, vp, vp, ci, ci, cf, cf, vp, ci, cd]
        lib.lc0mi_k_attention.argtypes = [vp, vp, ci, ci, ci, cf, vp, ci, cd]
        lib.lc0mi_k_expand_planes_attn.argtypes = [vp, vp, ci, ci, vp, ci, cd]
        lib.lc0mi_k_expand_planes_nchw.argtypes = [vp, vp, ci, vp]
        lib.lc0mi_k_attn_policy_gather.argtypes = [vp, vp, vp, ci, ci, vp]
        lib.lc0mi_k_gemm_f8.argtypes = [vp, ci, vp, ci, vp, vp, ci, ci, ci, ci, ci, cf, vp, ci, ci, cd]
        lib.lc0mi_k_quantize_f8.argtypes = [vp, ll, cf, vp]
        lib.lc0mi_k_layer_norm_f8.argtypes = [vp, vp, vp, vp, ci, ci, cf, cf, cf, vp, vp]
        lib.lc0mi_k_attention_f8.argtypes = [vp, vp, ci, ci, cf, cf, vp]
        lib.lc0mi_k_smolgen_attention.argtypes = [vp, vp, vp, ci, ci, ci, cf, ci, cf, vp, ci, cd]
        lib.lc0mi_k_legal_softmax.argtypes = [vp, vp, vp, cf, ci, vp]
        lib.lc0mi_k_attention_generic.argtypes = [ci, vp, vp, ci, ci, ci, cf, vp]
        lib.lc0mi_k_layer_norm_generic.argtypes = [ci, vp, vp, vp, vp, ci, ci, cf, cf, ci, vp]
        lib._k_ready = True
    return lib


def _check(rc):
    if rc:
        raise BackendError(load_library().lc0mi_last_error().decode(errors="replace"))


_BF16 = False


def to_bf16(a):
    """float array -> uint16 bfloat16 bits, round to nearest even."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def from_bf16(bits):
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


class bf16:
    """with kernels.bf16(): the 16-bit operands of gemm, layer_norm, layer_norm_rows, attention and
    smolgen_attention are bfloat16 (inputs rounded to it, results returned as float32) and the kernels run their
    bf16 instances."""

    def __enter__(self):
        global _BF16
        _BF16 = True
        _lib().lc0mi_k_set_bf16(1)

    def __exit__(self, *exc):
        global _BF16
        _BF16 = False
        _lib().lc0mi_k_set_bf16(0)


def _h(a):
    """16-bit operand: halves, or bfloat16 bits inside `with bf16()`."""
    return to_bf16(a) if _BF16 else np.ascontiguousarray(a, dtype=np.float16)


def _out16(shape):
    return np.zeros(shape, np.uint16 if _BF16 else np.float16)


def _ret16(out):
    return from_bf16(out) if _BF16 and out.dtype == np.uint16 else out


def _ptr(a):
    return a.ctypes.data if a is not None else None


def gemm(a, w, bias=None, scale=1.0, act=ACT_NONE, out_f32=False, time_iters=0):
    """a [batch?, M, K], w [batch?, N, K] (any float dtype, rounded to fp16) ->
    act(scale * a @ w^T + bias). Returns (C, ms) if time_iters else C."""
    a, w = _h(a), _h(w)
    batched = a.ndim == 3
    if not batched:
        a, w = a[None], w[None]
    batch, m, k = a.shape
    n = w.shape[1]
    out = np.zeros((batch, m, n), np.float32) if out_f32 else _out16((batch, m, n))
    b = np.ascontiguousarray(bias, np.float32) if bias is not None else None
    ms = C.c_double(0)
    _check(_lib().lc0mi_k_gemm(_ptr(a), k, m * k, _ptr(w), k, n * k, _ptr(b), m, n, k, batch, scale, act,
                               int(out_f32), _ptr(out), n, m * n, time_iters, C.byref(ms)))
    out = _ret16(out if batched else out[0])
    return (out, ms.value) if time_iters else out


def gemm_variant_name(m, n, k, batch=1, latency_first=False):
    """Tile shape the launcher picks for a half-precision product of this shape (host-side logic, no GPU needed)."""
    return _lib().lc0mi_k_gemm_variant_name(m, n, k, batch, int(latency_first)).decode()


def set_gemm_row_split(on):
    """Lets the launcher cut large products along their rows (default) or not; process-wide."""
    _lib().lc0mi_k_set_gemm_row_split(int(bool(on)))


def gemm_row_split(m, n, k):
    """Rows of the first launch when the launcher cuts a product of this shape along its rows (0: one launch)."""
    return _lib().lc0mi_k_gemm_row_split(m, n, k)


STORES_AUTO, STORES_AUTO_KEEP, STORES_CACHED, STORES_STREAM, STORES_WRITE_THROUGH = range(5)


def set_out_stores(kind):
    """Kind of output stores of gemm, gemm_f8 (256-row direct-to-LDS tiles) and layer_norm: STORES_AUTO (by size),
    STORES_AUTO_KEEP, STORES_CACHED, STORES_STREAM, STORES_WRITE_THROUGH."""
    _check(_lib().lc0mi_k_set_out_stores(int(kind)))


def set_cold_cache(mib):
    """Profiling: with mib > 0 every timed launch (time_iters) is preceded by an untimed copy of mib MiB, so that the
    kernel reads its operands from memory as inside a forward pass; 0 restores back-to-back launches."""
    _lib().lc0mi_k_set_cold_cache(int(mib))


def set_gemm_variant(variant):
    """-1 automatic, 0..2 direct-to-LDS 256x{256,192,128} tiles, 3 128x128, 4 64x64, 5 direct-to-LDS 128x128,
    6 row panels (16x16 to 64x32 outputs per workgroup, K split over its waves), 7 direct-to-LDS 128x64,
    8 unused (automatic choice), 9 direct-to-LDS 128x32 (very many rows, at most 32 columns), 10 direct-to-LDS
    64x64 (a few hundred rows)."""
    _lib().lc0mi_k_set_gemm_variant(int(variant))


def gemm_norm_producer(a, w, bias, skip, scale=1.0, skip_stats=None, skip_gamma=None, skip_beta=None, eps=1e-6,
                       time_iters=0):
    """U = scale * a @ w^T + bias + s (halves) and the partial row sums of U, [M, parts, 2]; s = skip, or the layer
    norm of skip's rows when skip_stats [M, parts, 2] (with skip_gamma, skip_beta) is given.
    Returns (U, stats) or (U, stats, ms)."""
    a, w, skip = _h(a), _h(w), _h(skip)
    m, k = a.shape
    n = w.shape[0]
    b = np.ascontiguousarray(bias, np.float32) if bias is not None else None
    st = np.ascontiguousarray(skip_stats, np.float32) if skip_stats is not None else None
    g = np.ascontiguousarray(skip_gamma, np.float32) if skip_stats is not None else None
    be = np.ascontiguousarray(skip_beta, np.float32) if skip_stats is not None else None
    u = np.zeros((m, n), np.float16)
    cap_parts = (n + 63) // 64
    stats = np.zeros((m, cap_parts, 2), np.float32)
    parts = C.c_int(0)
    ms = C.c_double(0.0)
    _check(_lib().lc0mi_k_gemm_norm_producer(
        _ptr(a), k, _ptr(w), k, _ptr(b), m, n, k, scale, _ptr(skip), _ptr(st),
        0 if st is None else st.shape[1], _ptr(g), _ptr(be), eps, _ptr(u), _ptr(stats), stats.size,
        C.byref(parts), time_iters, C.byref(ms)))
    stats = stats.reshape(-1)[:m * parts.value * 2].reshape(m, parts.value, 2).copy()
    return (u, stats, ms.value) if time_iters else (u, stats)


def gemm_norm_consumer(u, w, col_c, bias, stats, eps=1e-6, act=ACT_NONE, latency_first=False, time_iters=0):
    """act(rstd * (u @ w^T - mean x col_c) + bias) with the row statistics of u from stats [M, parts, 2]."""
    u, w = _h(u), _h(w)
    m, k = u.shape
    n = w.shape[0]
    c = np.ascontiguousarray(col_c, np.float32)
    b = np.ascontiguousarray(bias, np.float32) if bias is not None else None
    st = np.ascontiguousarray(stats, np.float32)
    out = np.zeros((m, n), np.float16)
    ms = C.c_double(0.0)
    _check(_lib().lc0mi_k_gemm_norm_consumer(
        _ptr(u), k, _ptr(w), k, _ptr(c), _ptr(b), m, n, k, _ptr(st), st.shape[1], eps, act,
        int(latency_first), _ptr(out), n, time_iters, C.byref(ms)))
    return (out, ms.value) if time_iters else out


def gemm_splitk(a, w, bias=None, split_k=4, scale=1.0):
    """a [M,K], w [N,K] -> float32 a @ w^T * scale + bias, reduced over split_k K-slices."""
    a, w = _h(a), _h(w)
    m, k = a.shape
    n = w.shape[0]
    out = np.zeros((m, n), np.float32)
    b = np.ascontiguousarray(bias, np.float32) if bias is not None else None
    _check(_lib().lc0mi_k_gemm_splitk(_ptr(a), k, _ptr(w), k, _ptr(b), m, n, k, split_k, scale, _ptr(out), n))
    return out


def layer_norm_rows(x, skip, gamma, beta, alpha, eps, pre_act=ACT_NONE, x_is_f32=False):
    """One workgroup per row: LN(act(x) * alpha + skip)."""
    xf = np.ascontiguousarray(x, np.float32) if x_is_f32 else None
    xh = None if x_is_f32 else _h(x)
    s = _h(skip) if skip is not None else None
    g = np.ascontiguousarray(gamma, np.float32)
    b = np.ascontiguousarray(beta, np.float32)
    rows, c = np.shape(x)
    y = _out16((rows, c))
    _check(_lib().lc0mi_k_layer_norm_rows(_ptr(xf), _ptr(xh), pre_act, _ptr(s), _ptr(g), _ptr(b), rows, c, alpha, eps,
                                          _ptr(y)))
    return _ret16(y)


def gemm_f32(a, w, bias=None, scale=1.0, act=ACT_NONE):
    a = np.ascontiguousarray(a, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    m, k = a.shape
    n = w.shape[0]
    out = np.zeros((m, n), np.float32)
    b = np.ascontiguousarray(bias, np.float32) if bias is not None else None
    _check(_lib().lc0mi_k_gemm_f32(_ptr(a), k, _ptr(w), k, _ptr(b), m, n, k, scale, act, _ptr(out), n))
    return out


def layer_norm(x, skip, gamma, beta, alpha, eps, time_iters=0):
    x = _h(x)
    s = _h(skip) if skip is not None else None
    g = np.ascontiguousarray(gamma, np.float32)
    b = np.ascontiguousarray(beta, np.float32)
    y = np.zeros_like(x)
    ms = C.c_double(0)
    _check(_lib().lc0mi_k_layer_norm(_ptr(x), _ptr(s), _ptr(g), _ptr(b), x.shape[0], x.shape[1], alpha, eps,
                                     _ptr(y), time_iters, C.byref(ms)))
    y = _ret16(y)
    return (y, ms.value) if time_iters else y


def attention(qkv, bias, batch, heads, scale, time_iters=0, depth=32):
    """qkv [B*64, 3*heads*depth], bias [B, heads, 64, 64] or None -> [B*64, heads*depth]."""
    qkv = _h(qkv)
    b = _h(bias) if bias is not None else None
    out = _out16((batch * 64, heads * depth))
    ms = C.c_double(0)
    _check(_lib().lc0mi_k_attention(_ptr(qkv), _ptr(b), batch, heads, depth, scale, _ptr(out), time_iters,
                                    C.byref(ms)))
    out = _ret16(out)
    return (out, ms.value) if time_iters else out


_DTYPES = {"half": (0, np.float16), "bf16": (1, np.uint16), "float": (2, np.float32)}


def _typed(a, dtype):
    return to_bf16(a) if dtype == "bf16" else np.ascontiguousarray(a, _DTYPES[dtype][1])


def attention_generic(qkv, bias, batch, heads, depth, scale, dtype="float"):
    """The general attention kernel: any head depth up to 128, dtype half / bf16 / float. Returns float32."""
    q = _typed(qkv, dtype)
    b = _typed(bias, dtype) if bias is not None else None
    out = np.zeros((batch * 64, heads * depth), _DTYPES[dtype][1])
    _check(_lib().lc0mi_k_attention_generic(_DTYPES[dtype][0], _ptr(q), _ptr(b), batch, heads, depth, scale, _ptr(out)))
    return from_bf16(out) if dtype == "bf16" else out.astype(np.float32)


def layer_norm_generic(x, skip, gamma, beta, alpha, eps, pre_act=ACT_NONE, dtype="float"):
    """The general layer norm: LN(act(x) * alpha + skip) for any row length, dtype half / bf16 / float."""
    xt = _typed(x, dtype)
    st = _typed(skip, dtype) if skip is not None else None
    g = np.ascontiguousarray(gamma, np.float32)
    b = np.ascontiguousarray(beta, np.float32)
    y = np.zeros(xt.shape, _DTYPES[dtype][1])
    _check(_lib().lc0mi_k_layer_norm_generic(_DTYPES[dtype][0], _ptr(xt), _ptr(st), _ptr(g), _ptr(b), xt.shape[0],
                                             xt.shape[1], alpha, eps, pre_act, _ptr(y)))
    return from_bf16(y) if dtype == "bf16" else y.astype(np.float32)


def gemm_f8(a, w, col_scale, bias=None, act=ACT_NONE, out_f8=False, out_mul=1.0, time_iters=0):
    """a [M,K], w [N,K] uint8 e4m3 -> act(col_scale * a.w^T + bias) as half (or e4m3 bytes of it * out_mul)."""
    a = np.ascontiguousarray(a, np.uint8)
    w = np.ascontiguousarray(w, np.uint8)
    cs = np.ascontiguousarray(col_scale, np.float32)
    b = np.ascontiguousarray(bias, np.float32) if bias is not None else None
    m, k = a.shape
    n = w.shape[0]
    out = np.zeros((m, n), np.uint8 if out_f8 else np.float16)
    ms = C.c_double(0)
    _check(_lib().lc0mi_k_gemm_f8(_ptr(a), k, _ptr(w), k, _ptr(cs), _ptr(b), m, n, k, act, int(out_f8),
                                  C.c_float(out_mul), _ptr(out), n, time_iters, C.byref(ms)))
    return (out, ms.value) if time_iters else out


def quantize_f8(x, mul=1.0):
    x = _h(x)
    y = np.zeros(x.shape, np.uint8)
    _check(_lib().lc0mi_k_quantize_f8(_ptr(x), C.c_longlong(x.size), C.c_float(mul), _ptr(y)))
    return y


def layer_norm_f8(x, skip, gamma, beta, alpha, eps, f8_mul):
    x = _h(x)
    s = _h(skip) if skip is not None else None
    g = np.ascontiguousarray(gamma, np.float32)
    b = np.ascontiguousarray(beta, np.float32)
    y = np.zeros_like(x)
    yq = np.zeros(x.shape, np.uint8)
    _check(_lib().lc0mi_k_layer_norm_f8(_ptr(x), _ptr(s), _ptr(g), _ptr(b), x.shape[0], x.shape[1], C.c_float(alpha),
                                        C.c_float(eps), C.c_float(f8_mul), _ptr(y), _ptr(yq)))
    return y, yq


def attention_f8(qkv, bias, batch, heads, scale, out_mul):
    qkv = _h(qkv)
    b = _h(bias) if bias is not None else None
    out = np.zeros((batch * 64, heads * 32), np.uint8)
    _check(_lib().lc0mi_k_attention_f8(_ptr(qkv), _ptr(b), batch, heads, C.c_float(scale), C.c_float(out_mul),
                                       _ptr(out)))
    return out


def smolgen_attention(qkv, gen, w, batch, heads, scale, f8_out=False, out_mul=1.0, time_iters=0):
    """qkv [B*64, 3*heads*32], gen [B, heads, gen_sz], w [4096, gen_sz] -> [B*64, heads*32] (halves, or e4m3 bytes)."""
    qkv, gen, w = _h(qkv), _h(gen), _h(w)
    out = np.zeros((batch * 64, heads * 32), np.uint8) if f8_out else _out16((batch * 64, heads * 32))
    ms = C.c_double(0)
    _check(_lib().lc0mi_k_smolgen_attention(_ptr(qkv), _ptr(gen), _ptr(w), batch, heads, w.shape[1], scale,
                                            int(f8_out), out_mul, _ptr(out), time_iters, C.byref(ms)))
    out = _ret16(out)
    return (out, ms.value) if time_iters else out


def expand_planes_attn(masks, values, ld=176, time_iters=0):
    masks = np.ascontiguousarray(masks, np.uint64)
    values = np.ascontiguousarray(values, np.float32)
    n = masks.shape[0]
    out = np.zeros((n * 64, ld), np.float16)
    ms = C.c_double(0)
    _check(_lib().lc0mi_k_expand_planes_attn(_ptr(masks), _ptr(values), n, ld, _ptr(out), time_iters, C.byref(ms)))
    return (out, ms.value) if time_iters else out


def expand_planes_nchw(masks, values):
    masks = np.ascontiguousarray(masks, np.uint64)
    values = np.ascontiguousarray(values, np.float32)
    n = masks.shape[0]
    out = np.zeros((n, 112, 64), np.float32)
    _check(_lib().lc0mi_k_expand_planes_nchw(_ptr(masks), _ptr(values), n, _ptr(out)))
    return out


def attn_policy_gather(logits, keys, ppo):
    """logits f32 [B,64,64], keys [B*64, pd], ppo f32 [4, pd] -> [B, 1858]."""
    logits = np.ascontiguousarray(logits, np.float32)
    keys = _h(keys)
    ppo = np.ascontiguousarray(ppo, np.float32)
    n = logits.shape[0]
    out = np.zeros((n, 1858), np.float32)
    _check(_lib().lc0mi_k_attn_policy_gather(_ptr(logits), _ptr(keys), _ptr(ppo), keys.shape[1], n, _ptr(out)))
    return out


def legal_softmax(policy, move_lists, temperature=1.359):
    """policy f32 [B,1858]; move_lists: B sequences of policy indices -> list of B probability arrays
    (softmax over the listed moves with lc0's FastExp, 1/temperature formed in float as the search wrapper does)."""
    policy = np.ascontiguousarray(policy, np.float32)
    n = policy.shape[0]
    offsets = np.zeros(n + 1, np.int32)
    offsets[1:] = np.cumsum([len(m) for m in move_lists])
    ids = np.ascontiguousarray(np.concatenate([np.asarray(m, np.uint16) for m in move_lists]) if offsets[-1]
                               else np.zeros(0, np.uint16), np.uint16)
    probs = np.zeros(max(int(offsets[-1]), 1), np.float32)
    inv_t = float(np.float32(1.0) / np.float32(temperature))
    _check(_lib().lc0mi_k_legal_softmax(_ptr(policy), _ptr(offsets), _ptr(ids) if ids.size else None, inv_t, n,
                                        _ptr(probs)))
    return [probs[offsets[i]:offsets[i + 1]].copy() for i in range(n)]


def winograd_conv(x, filt, bias, skip=None, se=None, act=ACT_RELU, fp16=False, fused_next=False):
    """x [B,64,Cin] (NHWC), filt [Cout,Cin,3,3], se = (w1 [K,C], b1, w2 [2C,K], b2) or None -> [B,64,Cout].
    fused_next: also returns the next convolution's transformed input [36, B*4, Cout] twice: from the
    fused output+input transform kernel and from the stand-alone input transform of the output."""
    x = np.ascontiguousarray(x, np.float32)
    filt = np.ascontiguousarray(filt, np.float32)
    bias = np.ascontiguousarray(bias, np.float32)
    b, _, cin = x.shape
    cout = filt.shape[0]
    sk = np.ascontiguousarray(skip, np.float32) if skip is not None else None
    if se is not None:
        w1, b1, w2, b2 = [np.ascontiguousarray(a, np.float32) for a in se]
        k = w1.shape[0]
    else:
        w1 = b1 = w2 = b2 = None
        k = 0
    out = np.zeros((b, 64, cout), np.float32)
    vf = np.zeros((36, b * 4, cout), np.float32) if fused_next else None
    vs = np.zeros((36, b * 4, cout), np.float32) if fused_next else None
    _check(_lib().lc0mi_k_winograd_conv(_ptr(x), _ptr(filt), _ptr(bias), _ptr(sk), _ptr(w1), _ptr(b1), _ptr(w2),
                                        _ptr(b2), k, b, cin, cout, act, int(fp16), _ptr(out), _ptr(vf), _ptr(vs)))
    return (out, vf, vs) if fused_next else out


def expand_planes_nhwc(masks, values):
    masks = np.ascontiguousarray(masks, np.uint64)
    values = np.ascontiguousarray(values, np.float32)
    n = masks.shape[0]
    out = np.zeros((n, 64, 112), np.float32)
    _check(_lib().lc0mi_k_expand_planes_nhwc(_ptr(masks), _ptr(values), n, _ptr(out)))
    return out
