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


def _time_of_choice(m, n, k, table):
    """Measured time of what the launcher does for this problem; None for a product cut along its rows into parts
    the table does not hold."""
    name = K.gemm_variant_name(m, n, k)
    if not name.endswith("+rest"):
        return table[(m, n, k)][COLUMN[name]]
    m1 = K.gemm_row_split(m, n, k)
    assert 0 < m1 < m and m1 % 256 == 0, (m, n, k, m1)
    if (m1, n, k) not in table or (m - m1, n, k) not in table:
        return None
    return table[(m1, n, k)][COLUMN[name[:-5]]] + _time_of_choice(m - m1, n, k, table)


def test_chosen_tile_shape_is_close_to_the_fastest_measured_one():
    table = {(m, n, k): times for m, n, k, times in _table()}
    regrets, cut = [], 0
    for (m, n, k), times in table.items():
        t = _time_of_choice(m, n, k, table)
        cut += K.gemm_row_split(m, n, k) > 0
        if t is not None:
            regrets.append(t / min(times) - 1.0)   # (below zero where two launches beat every single shape)
    print("%d of %d problems are cut along their rows" % (cut, len(table)))
    regrets = np.array(regrets)
    print("mean %.4f max %.4f over %d problems" % (regrets.mean(), regrets.max(), len(regrets)))
    assert len(regrets) >= 85
    assert regrets.mean() <= 0.012
    assert regrets.max() <= 0.10


def test_choices_for_the_encoder_layers_at_batch_256():
    """The four projections of a 15x1024 layer at 256 positions: whole rounds of 256 tiles on the 256 CUs."""
    assert K.gemm_variant_name(16384, 3072, 1024) == "gemm_dma_256x256x64"   # 768 tiles
    assert K.gemm_variant_name(16384, 1024, 1024) == "gemm_dma_256x256x64"   # 256 tiles
    assert K.gemm_variant_name(16384, 1536, 1024) == "gemm_dma_256x192x64"   # 512 tiles
    assert K.gemm_variant_name(16384, 1024, 1536) == "gemm_dma_256x256x64"


def test_products_that_leave_a_partial_round_are_cut_along_their_rows():
    """Whole rounds of large tiles first, the rest on whatever suits it; products that fill their rounds stay whole."""
    assert K.gemm_row_split(20480, 1024, 1536) == 16384
    assert K.gemm_variant_name(20480, 1024, 1536) == "gemm_dma_256x256x64+rest"
    assert K.gemm_row_split(24576, 1024, 1024) == 16384
    for m, n, k in ((16384, 3072, 1024), (16384, 1024, 1024), (16384, 1536, 1024), (32768, 1024, 1536), (4096, 1024, 1024),
                    (65536, 3072, 1024)):
        assert K.gemm_row_split(m, n, k) == 0, (m, n, k)
    assert K.gemm_row_split(20480, 64, 1024) == 0 and K.gemm_row_split(1 << 20, 1024, 256) == 0   # outside the model


def test_small_and_batched_products_keep_their_kernels():
    assert K.gemm_variant_name(1, 3072, 1024) == "gemm_rowpanel"
    assert K.gemm_variant_name(64, 64, 1024, batch=256) == "gemm_64x64x64"    # policy logits, one product per position
    assert K.gemm_variant_name(16384, 32, 1024) == "gemm_64x64x64"            # smolgen compression beside the projection
    assert K.gemm_variant_name(16384, 32, 1024, latency_first=True) == "gemm_rowpanel"
