"""Writes tests/golden/gemm_variant_timings.txt: the time of every direct-to-LDS tile shape of the half-precision
GEMM on a grid of problem sizes, measured on the GPU this runs on (MI355X). The launcher's cost model
(PickGemmVariantHalf in lc0_amd/csrc/gemm_kernels.hip) was fitted to this table, and tests/test_gemm_variant_choice.py
holds the launcher's choice to it.

    python tests/golden/make_gemm_variant_timings.py > tests/golden/gemm_variant_timings.txt
"""
import numpy as np

from lc0_amd import kernels as K

VARIANTS = (0, 1, 2, 5, 7)   # 256x256, 256x192, 256x128, 128x128, 128x64 (kernels.set_gemm_variant)
WIDE = ((1024, 1024), (1536, 1024), (1024, 1536), (3072, 1024))
OTHER = ((768, 768), (2304, 768), (1024, 768), (768, 1024), (512, 512), (1536, 512), (2048, 1024), (1024, 2048))


def main():
    rng = np.random.default_rng(0)
    print("# M N K, then microseconds per launch (mean of 20 to 30 back-to-back launches, HIP events) on")
    print("# 256x256 256x192 256x128 128x128 128x64 tiles; random normal operands, bias, no activation")
    shapes = [(m, n, k) for m in (4096, 6144, 8192, 10240, 12288, 16384, 20480, 24576, 32768) for n, k in WIDE]
    shapes += [(m, n, k) for m in (4096, 8192, 12288, 16384, 24576, 32768) for n, k in OTHER]
    shapes += [(65536, n, k) for n, k in OTHER[:6] + ((2048, 1024), (1536, 1024))]
    for m, n, k in shapes:
        a = rng.standard_normal((m, k), dtype=np.float32)
        w = rng.standard_normal((n, k), dtype=np.float32) * 0.03
        b = rng.standard_normal(n).astype(np.float32)
        times = []
        for v in VARIANTS:
            K.set_gemm_variant(v)
            try:
                _, ms = K.gemm(a, w, b, 1.0, K.ACT_NONE, time_iters=25)
            finally:
                K.set_gemm_variant(-1)
            times.append("%.1f" % (ms * 1000))
        print(m, n, k, *times, flush=True)


if __name__ == "__main__":
    main()
