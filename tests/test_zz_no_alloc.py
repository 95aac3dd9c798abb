"""The split-K GEMM entry point that allocates nothing (its partial sums live in a fixed array in device
memory) against lc0mi_k_gemm_splitk, which allocates its buffers per call: same kernels, same slice order,
so the results must be bit-identical. Two calls in a row share the fixed array; the second is smaller, so
stale partial sums of the first would show up as wrong elements."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _noalloc(lib, torch, a, w, bias, split_k, scale):
    m, k = a.shape
    n = w.shape[0]
    da = torch.from_numpy(a.view(np.int16)).cuda()
    dw = torch.from_numpy(w.view(np.int16)).cuda()
    db = torch.from_numpy(bias).cuda() if bias is not None else None
    dc = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    vp, ci, cf = C.c_void_p, C.c_int, C.c_float
    lib.lc0mi_k_gemm_splitk_noalloc.argtypes = [vp, ci, vp, ci, vp, ci, ci, ci, ci, cf, vp, ci, vp]
    rc = lib.lc0mi_k_gemm_splitk_noalloc(da.data_ptr(), k, dw.data_ptr(), k, db.data_ptr() if db is not None else None,
                                         m, n, k, split_k, scale, dc.data_ptr(), n, None)
    assert rc == 0, lib.lc0mi_last_error().decode()
    torch.cuda.synchronize()
    return dc.cpu().numpy()


def test_no_alloc_splitk_gemm_equals_allocating_entry_point():
    import torch

    from lc0_amd import kernels as K
    from lc0_amd import load_library

    lib = load_library()
    rng = np.random.default_rng(5)
    # The second call is smaller in every dimension and uses fewer slices.
    for (m, n, k, split_k, with_bias) in [(96, 320, 2048, 8, True), (24, 72, 512, 3, False)]:
        a = rng.standard_normal((m, k)).astype(np.float16)
        w = (rng.standard_normal((n, k)) * 0.05).astype(np.float16)
        bias = rng.standard_normal(n).astype(np.float32) if with_bias else None
        print("no-alloc split-K gemm", m, n, k, split_k, flush=True)
        got = _noalloc(lib, torch, a, w, bias, split_k, 0.5)
        want = K.gemm_splitk(a, w, bias, split_k=split_k, scale=0.5)
        assert got.shape == want.shape
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        ref = a.astype(np.float64) @ w.astype(np.float64).T * 0.5 + (bias if bias is not None else 0.0)
        assert np.abs(got - ref).max() < 2e-3


def test_no_alloc_splitk_gemm_rejects_sizes_beyond_the_fixed_array():
    import torch

    from lc0_amd import load_library

    lib = load_library()
    vp, ci, cf = C.c_void_p, C.c_int, C.c_float
    lib.lc0mi_k_gemm_splitk_noalloc.argtypes = [vp, ci, vp, ci, vp, ci, ci, ci, ci, cf, vp, ci, vp]
    m, n, k, split_k = 2048, 1024, 64, 4  # 8 Mi floats of partial sums > 4 Mi
    da = torch.zeros((m, k), dtype=torch.float16, device="cuda")
    dw = torch.zeros((n, k), dtype=torch.float16, device="cuda")
    dc = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    rc = lib.lc0mi_k_gemm_splitk_noalloc(da.data_ptr(), k, dw.data_ptr(), k, None, m, n, k, split_k, 1.0,
                                         dc.data_ptr(), n, None)
    assert rc != 0
    assert b"scratch" in lib.lc0mi_last_error()
    # A host pointer is refused before anything is launched.
    host = np.zeros((8, 64), np.float16)
    rc = lib.lc0mi_k_gemm_splitk_noalloc(host.ctypes.data, 64, dw.data_ptr(), 64, None, 8, 8, 64, 2, 1.0,
                                         dc.data_ptr(), 8, None)
    assert rc != 0
