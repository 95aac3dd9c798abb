"""Runs one kernel of the library a few times so that `rocprofv3` can attribute
counters to it. Meant to be launched under the profiler:

  rocprofv3 --pmc FETCH_SIZE -- python3 -m lc0_amd.profile_kernels copy --mib 256
  rocprofv3 --pmc WRITE_SIZE -- python3 -m lc0_amd.profile_kernels gemm --m 16384 --n 3072 --k 1024
  rocprofv3 --kernel-trace --stats -- python3 -m lc0_amd.profile_kernels gemm_f8 --m 16384 --n 3072 --k 1024
  rocprofv3 --kernel-trace --stats -- python3 -m lc0_amd.profile_kernels attention --batch 256 --heads 32
  rocprofv3 --kernel-trace --stats -- python3 -m lc0_amd.profile_kernels smolgen_attention --batch 256 --heads 32

`copy` moves a known number of bytes (reads N, writes N) and calibrates the HBM byte counters.
"""
import argparse
import ctypes as C

import numpy as np

from . import kernels as K
from .backend import load_library


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("kernel", choices=["copy", "gemm", "gemm_f8", "attention", "smolgen_attention", "layer_norm", "expand"])
    ap.add_argument("--mib", type=int, default=256)
    ap.add_argument("--m", type=int, default=16384)
    ap.add_argument("--n", type=int, default=3072)
    ap.add_argument("--k", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--gemm-batch", type=int, default=1, help="independent GEMMs in one launch (gemm only)")
    ap.add_argument("--iters", type=int, default=5)
    ap.add_argument("--data", choices=["random", "zeros", "const"], default="random",
                    help="operand values for gemm / gemm_f8: the same instruction stream runs faster on "
                         "constant operands (less switching power, higher sustained clock)")
    ap.add_argument("--variant", type=int, default=-1, help="force a GEMM tile variant (see kernels.set_gemm_variant)")
    ap.add_argument("--cold-mib", type=int, default=0,
                    help="copy this many MiB before every timed launch, so that the kernel reads its operands from "
                         "memory as inside a forward pass (0: back-to-back launches on cached operands)")
    args = ap.parse_args()
    if args.cold_mib > 0:
        K.set_cold_cache(args.cold_mib)
    if args.variant >= 0:
        K.set_gemm_variant(args.variant)
    rng = np.random.default_rng(0)
    if args.kernel == "copy":
        lib = load_library()
        lib.lc0mi_k_copy.argtypes = [C.c_longlong, C.c_int, C.POINTER(C.c_double)]
        ms = C.c_double(0)
        nbytes = args.mib << 20
        assert lib.lc0mi_k_copy(nbytes, args.iters, C.byref(ms)) == 0
        print("copy %d MiB: %.1f us per launch, %.0f GB/s (read+write)" % (args.mib, ms.value * 1e3,
                                                                          2 * nbytes / (ms.value * 1e-3) / 1e9))
    elif args.kernel == "gemm":
        nb = args.gemm_batch
        a = rng.standard_normal((nb, args.m, args.k), dtype=np.float32).astype(np.float16)
        w = (rng.standard_normal((nb, args.n, args.k), dtype=np.float32) * 0.02).astype(np.float16)
        if args.data != "random":
            a[:] = 0.0 if args.data == "zeros" else 1.0
            w[:] = 0.0 if args.data == "zeros" else 0.125
        _, ms = K.gemm(a, w, np.zeros(args.n, np.float32), time_iters=args.iters)
        print("gemm (%s data) %d x %dx%dx%d: %.1f us, %.0f TFLOP/s" % (
            args.data, nb, args.m, args.n, args.k, ms * 1e3, 2.0 * nb * args.m * args.n * args.k / (ms * 1e-3) / 1e12))
    elif args.kernel == "gemm_f8":
        a = rng.integers(0, 120, (args.m, args.k), dtype=np.uint8) | (rng.integers(0, 2, (args.m, args.k), dtype=np.uint8) << 7)
        w = rng.integers(0, 127, (args.n, args.k), dtype=np.uint8) | (rng.integers(0, 2, (args.n, args.k), dtype=np.uint8) << 7)
        if args.data != "random":
            a[:] = 0 if args.data == "zeros" else 0x38
            w[:] = 0 if args.data == "zeros" else 0x30
        _, ms = K.gemm_f8(a, w, np.full(args.n, 1e-3, np.float32), np.zeros(args.n, np.float32), time_iters=args.iters)
        print("gemm_f8 (%s data) %dx%dx%d: %.1f us, %.0f TFLOP/s" % (args.data, args.m, args.n, args.k, ms * 1e3,
                                                          2.0 * args.m * args.n * args.k / (ms * 1e-3) / 1e12))
    elif args.kernel == "attention":
        d = args.heads * 32
        qkv = rng.standard_normal((args.batch * 64, 3 * d), dtype=np.float32).astype(np.float16)
        bias = rng.standard_normal((args.batch, args.heads, 64, 64), dtype=np.float32).astype(np.float16)
        _, ms = K.attention(qkv, bias, args.batch, args.heads, 32 ** -0.5, time_iters=args.iters)
        nbytes = args.batch * args.heads * (4 * 64 * 32 * 2 + 8192)
        print("attention B=%d H=%d: %.1f us, %.0f GB/s algorithmic" % (args.batch, args.heads, ms * 1e3,
                                                                      nbytes / (ms * 1e-3) / 1e9))
    elif args.kernel == "smolgen_attention":
        d = args.heads * 32
        qkv = rng.standard_normal((args.batch * 64, 3 * d), dtype=np.float32).astype(np.float16)
        gen = rng.standard_normal((args.batch, args.heads, 256), dtype=np.float32).astype(np.float16)
        w = (rng.standard_normal((4096, 256), dtype=np.float32) * 0.1).astype(np.float16)
        _, ms = K.smolgen_attention(qkv, gen, w, args.batch, args.heads, 32 ** -0.5, time_iters=args.iters)
        nbytes = args.batch * args.heads * (4 * 64 * 32 * 2 + 512)
        print("smolgen_attention B=%d H=%d: %.1f us, %.0f GB/s algorithmic, %.0f TFLOP/s" % (
            args.batch, args.heads, ms * 1e3, nbytes / (ms * 1e-3) / 1e9,
            args.batch * args.heads * (2.0 * 4096 * 256 + 4.0 * 64 * 64 * 32) / (ms * 1e-3) / 1e12))
    elif args.kernel == "layer_norm":
        x = rng.standard_normal((args.m, args.k), dtype=np.float32).astype(np.float16)
        _, ms = K.layer_norm(x, x, np.ones(args.k, np.float32), np.zeros(args.k, np.float32), 0.5, 1e-6,
                             time_iters=args.iters)
        print("layer_norm %dx%d: %.1f us, %.0f GB/s algorithmic" % (args.m, args.k, ms * 1e3,
                                                                   6.0 * args.m * args.k / (ms * 1e-3) / 1e9))
    else:
        masks = rng.integers(0, 2 ** 63, (args.batch, 112), dtype=np.uint64)
        vals = np.ones((args.batch, 112), np.float32)
        _, ms = K.expand_planes_attn(masks, vals, 176, time_iters=args.iters)
        print("expand_planes B=%d: %.1f us" % (args.batch, ms * 1e3))


if __name__ == "__main__":
    main()
