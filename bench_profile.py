#!/usr/bin/env python3
"""Turn raw rocprofv3 output of bench.py runs into a committed summary under profiles/ and into
profiles/traffic.json, which bench.py reads its ``roofline.traffic`` figures from.

Nothing here touches a GPU: it reads the CSV files that three profiler runs per (workload, path) left behind,

    rocprofv3 --kernel-trace --stats --output-format csv -d <dir>/<w>_<p>/stats -o x -- python3 bench.py --workload <w> --path <p> --no-cpu-baseline --no-others --copy-probe --steps 10 --warmup 3
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir>/<w>_<p>/fetch -o x -- python3 bench.py --workload <w> --path <p> --no-cpu-baseline --no-others --copy-probe --steps 3 --warmup 1
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir>/<w>_<p>/write -o x -- python3 bench.py --workload <w> --path <p> --no-cpu-baseline --no-others --copy-probe --steps 3 --warmup 1

and writes

    python bench_profile.py <dir> --name <summary> [--placement "..."]

``profiles/<summary>.md`` (one table row per kernel of this library: launches, average / minimum / maximum duration,
algorithmic bytes, achieved rate, bytes read and written) and the entries of ``profiles/traffic.json`` for the
workloads found.  The counters are scaled by what they read for the one kernel of known traffic in the same run:
``--copy-probe`` launches ``torch.neg`` over exactly 1 GiB (1 048 576 KiB read, 1 048 576 KiB written).
"""
import argparse
import csv
import glob
import json
import os
import re
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

GIB_KIB = 1048576.0
ENTRY_POINTS = [                      # kernel name pattern -> (entry point, direction)
    (r"layer_lif_backward<", ("exodus_layer_lif_backward", "bwd")),
    (r"layer_lif_forward<", ("exodus_layer_lif_forward", "fwd")),
    (r"layer_leaky_backward<", ("exodus_layer_leaky_backward", "bwd")),
    (r"layer_leaky_forward<", ("exodus_layer_leaky_forward", "fwd")),
    (r"scan_\w*kernel<\(anonymous namespace\)::SynLifBwdOp", ("exodus_synlif_backward", "bwd")),
    (r"scan_\w*kernel<\(anonymous namespace\)::SynLifFwdOp", ("exodus_synlif_forward", "fwd")),
    (r"scan_\w*kernel<\(anonymous namespace\)::LifBwdOp", ("exodus_lif_backward_fused", "bwd")),
    (r"scan_\w*kernel<\(anonymous namespace\)::LifFwdOp", ("exodus_lif_forward", "fwd")),
    (r"scan_\w*kernel<\(anonymous namespace\)::LeakyBwdOp", ("exodus_leaky_backward_fused", "bwd")),
    (r"scan_\w*kernel<\(anonymous namespace\)::LeakyFwdOp", ("exodus_leaky_forward", "fwd")),
]


def short(name):
    """``layer_lif_backward<true, 1, 2, true, false, false>`` out of the full demangled signature"""
    name = name.replace("(anonymous namespace)::", "")
    name = re.sub(r"^void ", "", name)
    depth, out = 0, []
    for ch in name:
        if ch == "(" and depth == 0:
            break
        depth += ch == "<"
        depth -= ch == ">"
        out.append(ch)
    return "".join(out)


def entry_of(name):
    for pattern, value in ENTRY_POINTS:
        if re.search(pattern, name):
            return value
    return None


def kernel_stats(path):
    rows = {}
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            if entry_of(r["Name"]):
                rows[r["Name"]] = dict(calls=int(r["Calls"]), avg=float(r["AverageNs"]) / 1e6, min=float(r["MinNs"]) / 1e6,
                                       max=float(r["MaxNs"]) / 1e6)
    return rows


def counter_means(path, counter):
    """mean counter value per dispatch by kernel name, and the reading of the 1 GiB elementwise kernel"""
    sums, probe = {}, []
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            if r["Counter_Name"] != counter:
                continue
            name, value = r["Kernel_Name"], float(r["Counter_Value"])
            if "neg_kernel" in name:
                probe.append(value)
            if entry_of(name):
                s = sums.setdefault(name, [0.0, 0])
                s[0] += value
                s[1] += 1
    return {k: v[0] / v[1] for k, v in sums.items()}, probe


def one(pattern):
    found = sorted(glob.glob(pattern))
    return found[0] if found else None


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("directory", help="holds one folder <workload>_<path> per profiled run, each with stats/, fetch/, write/")
    ap.add_argument("--name", required=True, help="file name (without .md) of the summary under profiles/")
    ap.add_argument("--placement", default="bench.py's default (sinabs.exodus.hbm.enable(): inputs from the ordinary "
                                           "allocator, outputs in the striped range)")
    ap.add_argument("--extra-flags", default="", help="flags the profiled bench.py commands carried beyond the ones above")
    args = ap.parse_args()
    import bench

    lines, traffic = [], []
    notes = []
    for folder in sorted(glob.glob(os.path.join(args.directory, "*_*"))):
        tag = os.path.basename(folder)
        if "_" not in tag:
            continue
        key, path = tag.split("_", 1)
        if key not in bench.WORKLOADS or path not in ("layer", "rows"):
            continue
        stats_file = one(os.path.join(folder, "stats", "*kernel_stats.csv"))
        if not stats_file:
            continue
        w = bench.WORKLOADS[key]
        n_t = w["batch"] * w["steps"] * w["neurons"]
        per_dir = dict(zip(("fwd", "bwd"), (8, 12) if path == "layer" else w["bytes"]))
        stats = kernel_stats(stats_file)
        fetch_file = one(os.path.join(folder, "fetch", "*counter_collection.csv"))
        write_file = one(os.path.join(folder, "write", "*counter_collection.csv"))
        fetch, fprobe = counter_means(fetch_file, "FETCH_SIZE") if fetch_file else ({}, [])
        write, wprobe = counter_means(write_file, "WRITE_SIZE") if write_file else ({}, [])
        f_scale = GIB_KIB / (sum(fprobe) / len(fprobe)) if fprobe else None
        w_scale = GIB_KIB / (sum(wprobe) / len(wprobe)) if wprobe else None
        if f_scale and w_scale:
            notes.append(f"{tag}: 1 GiB elementwise kernel reads FETCH_SIZE = {sum(fprobe) / len(fprobe):,.0f}, "
                         f"WRITE_SIZE = {sum(wprobe) / len(wprobe):,.0f} KiB -> factors {f_scale:.3f} / {w_scale:.3f}")
        for name, st in sorted(stats.items(), key=lambda kv: -kv[1]["avg"]):
            entry, direction = entry_of(name)
            alg = n_t * per_dir[direction]
            rd = fetch.get(name) * f_scale * 1024 if name in fetch and f_scale else None
            wr = write.get(name) * w_scale * 1024 if name in write and w_scale else None
            total = rd + wr if rd is not None and wr is not None else None
            gb = lambda v: "-" if v is None else f"{v / 1e9:.2f} GB"
            lines.append(f"| {key} {path} | `{short(name)}` | {st['calls']} | {st['avg']:.3f} | {st['min']:.3f} | {st['max']:.3f} | "
                         f"{alg / 1e9:.2f} GB | {alg / st['avg'] / 1e9:.2f} TB/s = {alg / st['avg'] / 1e9 / 8 * 100:.1f} % | "
                         f"{gb(rd)} | {gb(wr)} | {gb(total)}" + (f" ({total / alg:.3f} x)" if total else "") + " |")
            if total:
                traffic.append({"workload": key, "path": path, "entry_point": entry, "kernel": short(name),
                                "bytes_per_launch": round(total), "read_bytes": round(rd), "written_bytes": round(wr),
                                "algorithmic_bytes": alg, "avg_ms": round(st["avg"], 4), "launches": st["calls"],
                                "source": f"profiles/{args.name}.md"})
    if not lines:
        sys.exit(f"no profiled runs found under {args.directory}")
    os.makedirs(os.path.join(ROOT, "profiles"), exist_ok=True)
    flags = (" " + args.extra_flags.strip()) if args.extra_flags.strip() else ""
    where = args.directory.rstrip("/")                         # as given on the command line
    md = [f"# Kernel trace and HBM counters of the bench workloads — {args.name.replace('_', ' ')}", "",
          f"Placement: {args.placement}.", "",
          "Commands (GPU box, repo root, after `cd /tmp && export TMPDIR=/tmp && cd $GRAFT_REPO_ROOT`), for each `<w>_<p>` below:", "",
          f"    rocprofv3 --kernel-trace --stats --output-format csv -d {where}/<w>_<p>/stats -o x -- python3 bench.py --workload <w> --path <p> --no-cpu-baseline --no-others --copy-probe --steps 10 --warmup 3{flags}",
          f"    rocprofv3 --pmc FETCH_SIZE --output-format csv -d {where}/<w>_<p>/fetch -o x -- python3 bench.py --workload <w> --path <p> --no-cpu-baseline --no-others --copy-probe --steps 3 --warmup 1{flags}",
          f"    rocprofv3 --pmc WRITE_SIZE --output-format csv -d {where}/<w>_<p>/write -o x -- python3 bench.py --workload <w> --path <p> --no-cpu-baseline --no-others --copy-probe --steps 3 --warmup 1{flags}",
          f"    python bench_profile.py {where} --name {args.name}", "",
          "Durations in ms from the kernel trace.  Read / written: mean FETCH_SIZE / WRITE_SIZE per dispatch, scaled by what the same",
          "counter reads for the 1 GiB elementwise kernel of the same run (`--copy-probe`: 1 048 576 KiB read and written):", ""]
    md += [f"* {n}" for n in notes]
    md += ["", "| workload | kernel | launches | avg | min | max | algorithmic bytes | achieved (algorithmic / avg) | read | written | HBM traffic |",
           "|---|---|---|---|---|---|---|---|---|---|---|"] + lines + [""]
    with open(os.path.join(ROOT, "profiles", args.name + ".md"), "w") as f:
        f.write("\n".join(md))
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    old = []
    if os.path.exists(tpath):
        with open(tpath) as f:
            old = json.load(f).get("kernels", [])
    fresh = {(e["workload"], e["entry_point"]) for e in traffic}
    merged = [e for e in old if (e["workload"], e["entry_point"]) not in fresh] + traffic
    merged.sort(key=lambda e: (e["workload"], e.get("path", ""), e["entry_point"]))
    with open(tpath, "w") as f:
        json.dump({"unit": "bytes per launch (FETCH_SIZE + WRITE_SIZE, scaled by a 1 GiB elementwise kernel of the same run)",
                   "kernels": merged}, f, indent=1)
        f.write("\n")
    print(f"wrote profiles/{args.name}.md ({len(lines)} kernels) and profiles/traffic.json ({len(merged)} entries)")


if __name__ == "__main__":
    main()
