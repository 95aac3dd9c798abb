"""Turns rocprofv3 output into the short summaries kept under profiles/.

  python -m lc0_amd.profile_summary stats DIR [--bench BENCH.json]
      DIR holds r_kernel_stats.csv of `rocprofv3 --kernel-trace --stats --output-format csv -d DIR -o r -- ...`;
      prints a table of the kernels by total time (and, with --bench, the bench line of the same run).
  python -m lc0_amd.profile_summary traffic --fetch DIR --write DIR --copy-fetch DIR --copy-write DIR
                                            --workload NAME --batch B [--json OUT]
      The four DIRs hold r_counter_collection.csv of `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs of the
      bench command and of `python3 -m lc0_amd.profile_kernels copy --mib 256` (the copy kernel of known size that
      scales the counters); prints the per-kernel table and, with --json, writes the record bench.py reads
      roofline.traffic from. The record carries a hash of the kernel sources it was measured on (sources_sha16).
  python -m lc0_amd.profile_summary counters DIR [DIR ...] [--kernel SUBSTRING]
      per-dispatch averages of every counter found in the DIRs' r_counter_collection.csv for the kernels whose
      name contains SUBSTRING.
"""
import argparse
import collections
import csv
import glob
import hashlib
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def sources_sha16():
    """Hash of the kernel and host sources under lc0_amd/csrc: a traffic record measured on other sources is stale."""
    h = hashlib.sha256()
    for path in sorted(glob.glob(os.path.join(HERE, "csrc", "*"))):
        if os.path.isfile(path):
            h.update(os.path.basename(path).encode())
            h.update(open(path, "rb").read())
    return h.hexdigest()[:16]


def short_name(n):
    n = n.replace("_ZN5lc0mi12_GLOBAL__N_1", "").replace("void lc0mi::(anonymous namespace)::", "").replace("_ZN5lc0mi", "")
    n = re.sub(r"^\d+", "", n)
    m = re.match(r"(\w+?)I(L[ib]\d+E)+", n)
    if m:
        nums = re.findall(r"L[ib](\d+)E", n.split("NS_")[0].split("DF16")[0])
        tail = " e4m3" if "GemmF8" in n else " bf16" if "DF16b" in n else ""
        if m.group(1) == "gemm_dma_kernel" and "ArgsE" in n:
            # template arguments behind the argument struct: output type, kind of output stores, epilogue, stages
            rest = re.findall(r"L[ib](\d+)E", n.split("ArgsE", 1)[1])
            if rest:
                tail += ", " + {"0": "ordinary", "1": "streaming", "2": "written-through"}.get(rest[0], rest[0]) + " stores"
        return "%s<%s>%s" % (m.group(1), ",".join(nums), tail)
    return re.sub(r"E[PKv].*$", "", n)[:70]


def _find(dirname, leaf):
    hits = glob.glob(os.path.join(dirname, "**", "*" + leaf), recursive=True)
    if not hits:
        sys.exit("no %s under %s" % (leaf, dirname))
    return hits[0]


def cmd_stats(args):
    rows = list(csv.DictReader(open(_find(args.dir, "kernel_stats.csv"))))
    print("| kernel | calls | avg us | total ms | % |\n|---|---|---|---|---|")
    for r in rows[:args.top]:
        print("| `%s` | %s | %.2f | %.2f | %.1f |" % (short_name(r["Name"]), r["Calls"], float(r["AverageNs"]) / 1e3,
                                                  float(r["TotalDurationNs"]) / 1e6, float(r["Percentage"])))
    if args.bench:
        d = json.loads(open(args.bench).read().strip().splitlines()[-1])
        rf = d["roofline"]
        print()
        print("bench.py in the same run: %.0f evals/s (%.3f ms per step); dominant kernel by HIP events `%s`: average "
              "launch %.4f ms over %d launches per pass, %.0f %s = %.3f of the %.0f %s peak; all GEMMs and attention "
              "%.3f of the fp16 MFMA peak." % (d["value"], d["ms_per_step"], rf["kernel"], rf["avg_launch_ms"],
                                               rf["launches_per_step"], rf["achieved"], rf["unit"], rf["frac"],
                                               rf["peak"], rf["unit"], d["all_gemm_attention"]["frac_of_mfma_peak"]))


def _per_kernel(dirname, counter=None):
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    for r in csv.DictReader(open(_find(dirname, "counter_collection.csv"))):
        if counter is None or r["Counter_Name"] == counter:
            agg[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return agg


def cmd_traffic(args):
    scale = {}
    for counter, d in (("FETCH_SIZE", args.copy_fetch), ("WRITE_SIZE", args.copy_write)):
        v = _per_kernel(d, counter)
        k = [x for x in v if "copy_kernel" in x][0]
        vals = v[k][counter][1:] or v[k][counter]
        mean = sum(vals) / len(vals)
        scale[counter] = (mean, args.copy_mib * 1024.0 / mean)
    fetch = _per_kernel(args.fetch, "FETCH_SIZE")
    write = _per_kernel(args.write, "WRITE_SIZE")
    print("| copy_kernel, %d KiB each way | counter per dispatch | scale to true KiB |\n|---|---|---|" % (args.copy_mib * 1024))
    for c in ("FETCH_SIZE", "WRITE_SIZE"):
        print("| %s | %.1f | x %.3f |" % (c, scale[c][0], scale[c][1]))
    print()
    print("| kernel | dispatches | fetch KiB | write KiB |\n|---|---|---|---|")
    rows = []
    for k in fetch:
        if "rocclr" in k:
            continue
        fv = fetch[k]["FETCH_SIZE"]
        wv = write.get(k, {}).get("WRITE_SIZE", [0.0])
        f = sum(fv) / len(fv) * scale["FETCH_SIZE"][1]
        w = sum(wv) / len(wv) * scale["WRITE_SIZE"][1]
        rows.append((len(fv) * (f + w), short_name(k), len(fv), f, w))
    for _, n, cnt, f, w in sorted(rows, reverse=True)[:args.top]:
        print("| `%s` | %d | %.0f | %.0f |" % (n, cnt, f, w))
    if args.json:
        def find(prefix):
            # bytes per dispatch, averaged over the dispatches of every instance of the kernel (kinds of stores,
            # stage counts): the same set of launches that bench.py times under this name
            hits = [(cnt, (f + w) * 1024) for _, n, cnt, f, w in rows
                    if n.startswith(prefix) and "bf16" not in n and "e4m3" not in n]
            total = sum(c for c, _ in hits)
            return int(sum(c * b for c, b in hits) / total) if total else None
        rec = {"workload": args.workload, "batch": args.batch, "sources_sha16": sources_sha16(),
               "source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of bench.py, KiB per dispatch x 1024, copy-kernel "
                         "factors %.3f / %.3f (python -m lc0_amd.profile_summary traffic)"
                         % (scale["FETCH_SIZE"][1], scale["WRITE_SIZE"][1]),
               "kernels": {"gemm_dma_256x256x64": find("gemm_dma_kernel<256,256,128"),
                           "gemm_dma_256x192x64": find("gemm_dma_kernel<256,192,128"),
                           "smolgen_attention": find("smolgen_attention_kernel"),
                           "layer_norm_skip": find("layer_norm_kernel")}}
        json.dump(rec, open(args.json, "w"), indent=1)


def cmd_counters(args):
    total = collections.defaultdict(lambda: collections.defaultdict(list))
    for d in args.dirs:
        for k, cs in _per_kernel(d).items():
            if args.kernel in k:
                for c, vals in cs.items():
                    total[short_name(k)][c] += vals
    for k, cs in total.items():
        print("kernel `%s`" % k)
        print("| counter | per dispatch | dispatches |\n|---|---|---|")
        for c in sorted(cs):
            vals = cs[c][1:] or cs[c]   # the first dispatch carries one-time costs
            print("| %s | %.0f | %d |" % (c, sum(vals) / len(vals), len(vals)))


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    s = sub.add_parser("stats")
    s.add_argument("dir")
    s.add_argument("--bench", default="")
    s.add_argument("--top", type=int, default=14)
    t = sub.add_parser("traffic")
    for name in ("fetch", "write", "copy-fetch", "copy-write"):
        t.add_argument("--" + name, required=True)
    t.add_argument("--copy-mib", type=int, default=256)
    t.add_argument("--workload", required=True)
    t.add_argument("--batch", type=int, required=True)
    t.add_argument("--json", default="")
    t.add_argument("--top", type=int, default=12)
    c = sub.add_parser("counters")
    c.add_argument("dirs", nargs="+")
    c.add_argument("--kernel", default="")
    args = ap.parse_args()
    {"stats": cmd_stats, "traffic": cmd_traffic, "counters": cmd_counters}[args.cmd](args)


if __name__ == "__main__":
    main()
