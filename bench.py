"""Benchmark of the NN-evaluation hot path on one MI355X.

Metric: NN evals/sec at batch 256 on the BT4-shape fp16 net,
with the dominant kernel's fraction of the MFMA roofline and the CPU oracle's
evals/sec on the same host next to it. A "step" is one device pass over one
batch of 256 seeded random-playout positions already resident in HBM: `value` is
that rate. The same path with the host copies (H2D of the planes, D2H of the
outputs) is printed next to it as `with_host_io_evals_per_s`.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME] [--batch B]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16/bf16 MFMA peak
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA peak
PEAK_FP32_TFLOPS = 157.3    # MI355X dense fp32 MFMA peak
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E peak

# HBM bytes per launch of a kernel cannot be read from inside the process: they come from two rocprofv3 --pmc
# runs of this same command (FETCH_SIZE, WRITE_SIZE, scaled by the copy-kernel calibration). The summary of such
# a run is a small JSON file {"workload", "batch", "source", "kernels": {kernel: bytes per launch}}; when one
# for this workload and batch is given (or sits under profiles/), roofline.traffic is taken from it, else null.
def measured_traffic(path, workload, batch, kernel):
    """(bytes per launch, where they come from). None when there is no record for this workload, batch and kernel,
    or when the record was measured on other kernel sources than the ones in the tree now (its sources_sha16)."""
    path = path or os.path.join(ROOT, "profiles", "hbm_traffic_%s_batch%d.txt" % (workload, batch))
    try:
        rec = json.load(open(path))
    except (OSError, ValueError):
        return None, None
    if rec.get("workload") != workload or rec.get("batch") != batch:
        return None, None
    from lc0_amd.profile_summary import sources_sha16
    now = sources_sha16()
    if rec.get("sources_sha16") != now:
        return None, "stale: %s was measured on kernel sources %s, the tree holds %s" % (
            os.path.relpath(path, ROOT), rec.get("sources_sha16"), now)
    return rec.get("kernels", {}).get(kernel), "%s (sources %s); %s" % (os.path.relpath(path, ROOT), now, rec.get("source"))


WORKLOADS = {
    "c2_bt4_15x1024": dict(batch=256, desc="BT4-shape attention body: 15 layers, d=1024, 32 heads, dff 1536, "
                                           "smolgen 32/256/256, fp16 with fp32 accumulation"),
    "c1_attn_10x256": dict(batch=64, desc="attention body: 10 layers, d=256, 8 heads, dff 1024, fp16"),
    "c0_resnet_6x64": dict(batch=32, options="precision=fp32", dtype="fp32",
                           desc="SE-ResNet 6x64, SE ratio 4, classical policy, WDL, fp32"),
    "c3_resnet_20x256": dict(batch=512, desc="SE-ResNet 20x256, SE ratio 4, winograd F(4x4,3x3), fp16"),
    "c4_bt4_fp8": dict(batch=1024, net="c2_bt4_15x1024", options="precision=fp8", dtype="fp8_e4m3",
                       desc="BT4-shape attention body with e4m3 operands (fp32 accumulation) in the QKV, attention-output "
                            "and FFN GEMMs; weights scaled per output row, activations per tensor; the rest fp16"),
    "c2_bt4_bf16": dict(batch=256, net="c2_bt4_15x1024", options="precision=bf16", dtype="bf16",
                        desc="BT4-shape attention body as c2_bt4_15x1024 with bfloat16 weights and activations "
                             "(bf16 matrix instructions, fp32 accumulation)"),
    "bt4_dense_15x1024": dict(batch=256, desc="BT4 as published: PE_DENSE embedding (64 channels, embedding FFN 1536), "
                                              "15 layers, d=1024, 32 heads, dff 1536, smolgen, multi-head format, fp16"),
    "tiny_attn": dict(batch=64, desc="tiny smolgen attention body (test net)"),
}


def _host_description():
    model = "unknown CPU"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    blas = "numpy's bundled BLAS"
    try:
        from threadpoolctl import threadpool_info
        libs = ["%s %s (%s threads)" % (i.get("internal_api"), i.get("version"), i.get("num_threads"))
                for i in threadpool_info() if i.get("user_api") == "blas"]
        if libs:
            blas = ", ".join(libs)
    except ImportError:
        pass
    return model, blas


def cpu_baseline(path, masks, values, batch, sample=0, seconds_budget=27.0):
    """Oracle (numpy/BLAS restatement of the blas backend) timed on this host: three timed passes over one
    sample of the workload's batch (the whole batch when three passes fit the time budget)."""
    from oracle import netread as nr
    from oracle import nn as onn
    bn = onn.BlasNetwork(nr.load(path), batch_size=max(batch, 1))
    bn.forward(masks[:2], values[:2])  # warm-up
    if not sample:
        probe = min(8, batch)
        t0 = time.perf_counter()
        bn.forward(masks[:probe], values[:probe])
        rate = probe / (time.perf_counter() - t0)
        sample = int(max(probe, min(batch, rate * seconds_budget / 3.0)))
    m, v = masks[:sample], values[:sample]
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        bn.forward(m, v)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    model, blas = _host_description()
    out = {"value": sample / med, "unit": "evals/s", "cores": cores, "kind": "port",
           "sample": "%d of the batch's %d positions per pass, 3 timed passes, median; numpy float32, sgemm of %s; %s"
                     % (sample, batch, blas, model)}
    # The reference blas backend defaults to one thread (network_blas.cc:994): same oracle, BLAS pinned to 1 thread.
    try:
        from threadpoolctl import threadpool_limits
        small = max(1, min(4, sample))
        with threadpool_limits(limits=1):
            bn.forward(m[:1], v[:1])
            t1 = []
            t_end = time.time() + 6.0
            while len(t1) < 2 or (time.time() < t_end and len(t1) < 5):
                t0 = time.perf_counter()
                bn.forward(m[:small], v[:small])
                t1.append(time.perf_counter() - t0)
        t1.sort()
        out["one_thread"] = {"value": small / t1[len(t1) // 2], "unit": "evals/s", "cores": 1,
                             "sample": "%d positions per pass, %d timed passes, median" % (small, len(t1))}
    except ImportError:
        pass
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c2_bt4_15x1024", choices=sorted(WORKLOADS))
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-sample", type=int, default=0, help="positions per CPU pass (0: as many of the batch as "
                                                              "three passes fit in about 27 s)")
    ap.add_argument("--traffic-json", default="", help="HBM bytes per launch from a rocprofv3 --pmc run of this command "
                                                       "(default: profiles/hbm_traffic_<config>_batch<B>.txt if present)")
    ap.add_argument("--options", default="", help="backend options appended to the workload's own (name=value,...)")
    ap.add_argument("--sweep", default="", help="comma-separated batch sizes: adds their resident-batch evals/s "
                                                "as \"batch_sweep\" to the JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend evaluates on one GPU (batch rows are independent; more GPUs means "
                 "one backend instance per GPU fed by lc0's demux, nothing to measure here). Use --gpus 1.")

    import numpy as np

    from lc0_amd import Network, netgen
    from oracle import chess as oc   # input generator only (seeded random playouts)

    wl = WORKLOADS[args.config]
    batch = args.batch or wl["batch"]
    path = netgen.cached_config(wl.get("net", args.config))
    sweep = [int(b) for b in args.sweep.split(",") if b]
    pos = oc.random_positions(min(max([batch, args.cpu_sample] + sweep), 1024), seed=20240)
    masks, values = pos["masks"], pos["values"]

    if max([batch] + sweep) > masks.shape[0]:
        reps = -(-max([batch] + sweep) // masks.shape[0])
        masks, values = np.tile(masks, (reps, 1)), np.tile(values, (reps, 1))
    net = Network(path, "gpu=0,max_batch=%d" % max([batch, 16] + sweep) + ("," + wl["options"] if wl.get("options") else "") +
                  ("," + args.options if args.options else ""))
    # Arithmetic type of the pass: the workload's own, or what a precision= option given on the command line says.
    dtype = wl.get("dtype", "fp16")
    for item in args.options.split(","):
        if item.startswith("precision="):
            dtype = {"fp8": "fp8_e4m3"}.get(item.split("=", 1)[1], item.split("=", 1)[1])
    comp = net.NewComputation()
    comp.AddInputs(masks[:batch], values[:batch])
    comp.ComputeBlocking()          # stages the batch into HBM and warms everything up
    checksum = float(np.abs(comp.results()["policy"]).sum())

    # Whole path including host staging (H2D of planes, D2H of 1858 logits): reported, never `value`.
    io_iters = max(3, min(10, args.steps))

    def timed_blocking(c):
        for _ in range(3):          # the GPU's clocks fall while the host prepares inputs: warm up first
            c.ComputeBlocking()
        t0 = time.perf_counter()
        for _ in range(io_iters):
            c.ComputeBlocking()
        return (time.perf_counter() - t0) * 1e3 / io_iters

    io_ms = timed_blocking(comp)

    # The same with each position's legal moves listed: the policy softmax over them runs on the
    # device and only those probabilities are downloaded instead of 1858 logits per position.
    comp_legal = net.NewComputation()
    for i in range(batch):
        comp_legal.AddInputs(masks[i:i + 1], values[i:i + 1])
        comp_legal.AddLegalMoves(pos["legal"][i % len(pos["legal"])])
    io_legal_ms = timed_blocking(comp_legal)
    comp_legal.close()

    # Two and four search threads, each with its own computation in flight on the shared network (host I/O
    # included): how lc0 drives a backend (backendbench.cc:177-184 does the same with --threads). Passes of
    # different lanes overlap on the GPU, so the aggregate rate is above that of one computation at a time.
    import threading

    def threads_ms(n_threads):
        comps = [comp]
        for _ in range(n_threads - 1):
            c = net.NewComputation()
            c.AddInputs(masks[:batch], values[:batch])
            c.ComputeBlocking()
            comps.append(c)
        gate = threading.Barrier(n_threads + 1)

        def search_thread(c):
            for _ in range(2):
                c.ComputeBlocking()
            gate.wait()
            for _ in range(io_iters):
                c.ComputeBlocking()
            gate.wait()

        workers = [threading.Thread(target=search_thread, args=(c,)) for c in comps]
        for w in workers:
            w.start()
        gate.wait()
        t0 = time.perf_counter()
        gate.wait()
        ms = (time.perf_counter() - t0) * 1e3 / io_iters
        for w in workers:
            w.join()
        for c in comps[1:]:
            c.close()
        return ms

    two_threads_ms = threads_ms(2)
    four_threads_ms = threads_ms(4)

    # Timed region: K device passes over the resident batch, bracketed by stream
    # synchronisation on both sides (inside TimeResidentForward) and by the host clock.
    if args.warmup > 0:
        net.TimeResidentForward(batch, args.warmup)
    t0 = time.perf_counter()
    ev_ms = net.TimeResidentForward(batch, args.steps)
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # Per-kernel HIP-event timing of one more pass (events on the compute stream).
    net.SetProfiling(True)
    prof_iters = 3
    for _ in range(prof_iters):
        comp.ComputeBlocking()
    prof = net.TakeProfile()
    net.SetProfiling(False)
    total_kernel_ms = sum(k.ms for k in prof) / prof_iters
    kernels = sorted(prof, key=lambda k: -k.ms)
    matrix = [k for k in prof if k.name.startswith("gemm") or k.name in ("attention", "smolgen_attention")]
    gemm_ms = sum(k.ms for k in matrix) / prof_iters
    gemm_flops = sum(k.flops for k in matrix) / prof_iters
    # Group call sites by the kernel that ran them ("call_site|kernel_variant"): the
    # roofline is quoted for the kernel (as rocprofv3 sees it), not for one call site.
    from collections import namedtuple
    Agg = namedtuple("Agg", ["name", "ms", "launches", "flops", "bytes"])
    groups = {}
    for k in prof:
        variant = k.name.split("|")[1] if "|" in k.name else k.name
        g = groups.get(variant, Agg(variant, 0.0, 0, 0.0, 0.0))
        groups[variant] = Agg(variant, g.ms + k.ms, g.launches + k.launches, g.flops + k.flops, g.bytes + k.bytes)
    dom = max(groups.values(), key=lambda g: g.ms)
    peak = (PEAK_FP8_TFLOPS if dom.name.startswith("gemm_f8") else
            PEAK_FP32_TFLOPS if dom.name.startswith("gemm_f32") else PEAK_FP16_TFLOPS)   # (bf16 has the fp16 peak)
    # A matrix kernel is priced against the MFMA peak only when its flops per algorithmic byte lie above the ridge
    # point peak flops / peak bandwidth (fp16: 312 flop/B); below it the memory roofline is the one that bounds it
    # (the 36 batched winograd-domain GEMMs of a 256-filter convolution: 121 flop/B).
    mfma_bound = dom.flops > 0 and (dom.bytes <= 0 or dom.flops / dom.bytes >= peak * 1e12 / (PEAK_HBM_GBS * 1e9))
    if mfma_bound:
        achieved = dom.flops / dom.launches / (dom.ms / dom.launches * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": dom.name, "achieved": achieved, "peak": peak,
                    "unit": "TFLOP/s", "frac": achieved / peak, "traffic": None,
                    "avg_launch_ms": dom.ms / dom.launches, "launches_per_step": dom.launches // prof_iters}
    else:
        achieved = dom.bytes / dom.launches / (dom.ms / dom.launches * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": dom.name, "achieved": achieved, "peak": PEAK_HBM_GBS,
                    "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS, "traffic": None,
                    "avg_launch_ms": dom.ms / dom.launches, "launches_per_step": dom.launches // prof_iters}

    roofline["traffic"], roofline["traffic_source"] = measured_traffic(args.traffic_json, args.config, batch, dom.name)
    roofline["algorithmic_bytes"] = dom.bytes / dom.launches if dom.bytes else None

    result = {
        "metric": "NN evals/sec at batch 256, BT4-shape fp16" if args.config == "c2_bt4_15x1024" else "NN evals/sec",
        "value": batch / (wall_ms * 1e-3),
        "unit": "evals/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": args.config, "description": wl["desc"], "batch": batch,
                   "inputs": "seeded random-playout positions, classical 112 planes",
                   **({"extra_options": args.options} if args.options else {})},
        "roofline": roofline,
        "event_ms_per_step": ev_ms,
        "with_host_io_evals_per_s": batch / (io_ms * 1e-3),
        "with_host_io_legal_policy_evals_per_s": batch / (io_legal_ms * 1e-3),
        "with_host_io_two_threads_evals_per_s": 2 * batch / (two_threads_ms * 1e-3),
        "with_host_io_four_threads_evals_per_s": 4 * batch / (four_threads_ms * 1e-3),
        "all_gemm_attention": {"ms_per_step": gemm_ms, "tflops": gemm_flops / (gemm_ms * 1e-3) / 1e12 if gemm_ms else None,
                               "frac_of_mfma_peak": gemm_flops / (gemm_ms * 1e-3) / 1e12 / PEAK_FP16_TFLOPS if gemm_ms else None},
        "kernel_ms_per_step": {k.name: round(k.ms / prof_iters, 4) for k in kernels},
        "kernel_variant_ms_per_step": {g.name: round(g.ms / prof_iters, 4) for g in sorted(groups.values(), key=lambda g: -g.ms)},
        "sum_kernel_ms_per_step": total_kernel_ms,
        # bandwidth-bound kernels: algorithmic bytes / HIP-event time against the 8 TB/s HBM peak
        "hbm_kernels": {g.name: {"GBps": round(g.bytes / (g.ms * 1e-3) / 1e9, 1),
                                 "frac_of_hbm_peak": round(g.bytes / (g.ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 3),
                                 "avg_launch_us": round(g.ms / g.launches * 1e3, 2)}
                        for g in sorted(groups.values(), key=lambda g: -g.ms) if g.flops == 0 and g.ms > 0},
        "policy_checksum": checksum,
    }
    if sweep:
        result["batch_sweep"] = {}
        for b in sweep:
            c = net.NewComputation()
            c.AddInputs(masks[:b], values[:b])
            c.ComputeBlocking()
            iters = max(5, min(200, int(2000 / max(b, 8))))
            net.TimeResidentForward(b, 3)
            t0 = time.perf_counter()
            net.TimeResidentForward(b, iters)
            ms = (time.perf_counter() - t0) * 1e3 / iters
            result["batch_sweep"][str(b)] = {"evals_per_s": b / (ms * 1e-3), "ms_per_step": ms}
            c.close()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(path, masks, values, batch, args.cpu_sample)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
