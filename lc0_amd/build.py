"""Builds lc0_amd/liblc0mi.so (the C-ABI library: host C++ + gfx950 kernels)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "liblc0mi.so")
SOURCES = ["weights.cc", "tables.cc", "network.cc", "capi.cc", "kernel_api.cc", "kernels.hip", "gemm_kernels.hip", "smolgen_attention.hip", "resnet_kernels.hip"]
# -packed-fp32-ops off: packed fp32 forms are not trusted on this hardware pool.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result", "-Wno-unknown-warning-option"]


def build(verbose=False):
    objs = []
    build_dir = os.path.join(HERE, "build")
    os.makedirs(build_dir, exist_ok=True)
    procs = []
    for src in SOURCES:
        obj = os.path.join(build_dir, src.replace(".", "_") + ".o")
        cmd = ["hipcc"] + FLAGS + DEVICE_FLAGS + ["-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if p.returncode != 0:
            failed = True
            sys.stderr.write("\n".join(lines) + "\n")
        elif verbose and lines:
            print("\n".join(lines))
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = ["hipcc", "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs + ["-lz"]
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
