"""The launcher's choice of tile shape for large half-precision products (host logic, no GPU): held to the measured
time of every shape on 92 problem sizes (tests/golden/gemm_variant_timings.txt, written on an MI355X by
tests/golden/make_gemm_variant_timings.py)."""
import os

import numpy as np

from lc0_amd import kernels as K

COLUMN = {"gemm_dma_256x256x64": 0, "gemm_dma_256x192x64": 1, "gemm_dma_256x128x32": 2, "gemm_dma_128x128x64": 3,
          "gemm_dma_128x64x64": 4}


def _table():
    path = os.path.join(os.path.dirname(__file__), "golden", "gemm_variant_timings.txt")
    rows = [line.split() for line in open(path) if line.strip() and not line.startswith("#")]
    return [(int(r[0]), int(r[1]), int(r[2]), [float(t) for t in r[3:8]]) for r in rows]


def test_chosen_tile_shape_is_close_to_the_fastest_measured_one():
    regrets = []
    for m, n, k, times in _table():
        name = K.gemm_variant_name(m, n, k)
        assert name in COLUMN, (m, n, k, name)
        regrets.append(times[COLUMN[name]] / min(times) - 1.0)
    regrets = np.array(regrets)
    print("mean %.4f max %.4f over %d problems" % (regrets.mean(), regrets.max(), len(regrets)))
    assert len(regrets) >= 90
    assert regrets.mean() <= 0.012
    assert regrets.max() <= 0.10


def test_choices_for_the_encoder_layers_at_batch_256():
    """The four projections of a 15x1024 layer at 256 positions: whole rounds of 256 tiles on the 256 CUs."""
    assert K.gemm_variant_name(16384, 3072, 1024) == "gemm_dma_256x256x64"   # 768 tiles
    assert K.gemm_variant_name(16384, 1024, 1024) == "gemm_dma_256x256x64"   # 256 tiles
    assert K.gemm_variant_name(16384, 1536, 1024) == "gemm_dma_256x192x64"   # 512 tiles
    assert K.gemm_variant_name(16384, 1024, 1536) == "gemm_dma_256x256x64"


def test_small_and_batched_products_keep_their_kernels():
    assert K.gemm_variant_name(1, 3072, 1024) == "gemm_rowpanel"
    assert K.gemm_variant_name(64, 64, 1024, batch=256) == "gemm_64x64x64"    # policy logits, one product per position
    assert K.gemm_variant_name(16384, 32, 1024) == "gemm_64x64x64"            # smolgen compression beside the projection
    assert K.gemm_variant_name(16384, 32, 1024, latency_first=True) == "gemm_rowpanel"
