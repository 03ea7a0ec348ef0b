"""Profiler runs of the layer, and the counter file the benchmark reads its measured HBM traffic from.

    python -m titanic-flash-41_amd.counters run   --out DIR [--workloads c2,c3,c4,c5] [--shader]
    python -m titanic-flash-41_amd.counters stamp DIR [--to profiles/counters.json]

`run` needs a GPU.  For every workload it starts rocprofv3 on the stand-alone layer driver (tf_layer_probe: the benchmark
geometry, pseudo-random operands, the layer's own schedule) once per pass: a kernel trace with statistics, then one counter
a run (FETCH_SIZE, WRITE_SIZE; with --shader also the L2 hit counters and the shader counters of the many-row GEMM).  Every
run ends with plain copies of 256 MiB, a kernel whose traffic is known, which the counters are scaled by.  The raw CSV files
stay under DIR.

`stamp` needs no GPU.  It reads DIR, scales the counters, and writes one JSON file: per workload, for the routed experts' two
launches and the copy kernel, the calls, the mean duration, the HBM bytes a launch (fetched + written), the algorithmic bytes
the driver computed, and their ratio, per kernel and summed over a projection's kernels (every other kernel: its mean duration); stamped with the library's SHA-256 (the build manifest's) and, where a git work tree is
present, its commit.  bench.py multiplies that ratio with the algorithmic bytes of its own launches.
"""
import argparse
import csv
import glob
import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
COPY_BYTES = 256 << 20
# rows, passes, batches, copies, skew, rows a request: the probe's arguments.  16,384 rows: the skew that gives the probe's
# operands the benchmark workload's shape (every expert active, about 911 tiles of 128 rows, the same algorithmic bytes).
# 32 rows: four requests of eight draft tokens whose routes overlap as the benchmark's correlated rows do (about 40 tiles).
WORKLOADS = {
    "c2": ("4", "64", "16", "4", "0"),
    "c3": ("32", "64", "16", "4", "0", "8"),
    "c4": ("4096", "6", "2", "4", "0"),
    "c5": ("16384", "4", "2", "4", "0.02"),
}
PASSES = {
    "trace": ["--kernel-trace", "--stats"],
    "fetch": ["--pmc", "FETCH_SIZE"],
    "write": ["--pmc", "WRITE_SIZE"],
}
SHADER_PASSES = {
    "l2": ["--pmc", "TCC_HIT_sum", "TCC_MISS_sum", "TCC_REQ_sum"],
    "shader": ["--pmc", "SQ_WAVE_CYCLES", "SQ_BUSY_CYCLES", "SQ_WAIT_INST_ANY", "SQ_ACTIVE_INST_ANY", "SQ_VALU_MFMA_BUSY_CYCLES",
               "SQ_INSTS_VALU_MFMA_MOPS_F8", "SQ_WAIT_INST_LDS", "SQ_INSTS_LDS"],
}
# which kernel is which part of the layer: few rows / many rows
ROLES = [("fc1", "tf_phase1_stream"), ("fc2", "tf_phase2_stream"), ("fc1", "tf_grouped_gemm<0"), ("fc2", "tf_grouped_gemm<2"),
         ("shared_fc1", "tf_grouped_gemm<1"), ("shared_fc2", "tf_grouped_gemm<3"), ("copy", "tf_probe_copy")]


def role_of(kernel):
    for role, part in ROLES:
        if part in kernel:
            return role
    return None


def run(out, workloads, shader):
    probe, lib = os.path.join(HERE, "tf_layer_probe"), os.path.join(HERE, "libtitanic_moe_hip.so")
    for path in (probe, lib):
        if not os.path.exists(path):
            sys.exit("missing %s: build first" % path)
    os.makedirs(out, exist_ok=True)
    manifest = os.path.join(HERE, "manifest.json")
    with open(os.path.join(out, "run.json"), "w") as f:
        json.dump({"manifest": json.load(open(manifest)) if os.path.exists(manifest) else None, "workloads": workloads}, f)
    env = dict(os.environ, TMPDIR="/tmp")
    for w in workloads:
        passes = dict(PASSES)
        if shader and int(WORKLOADS[w][0]) > 64:
            passes.update(SHADER_PASSES)
        for name, flags in passes.items():
            target = os.path.join(out, w, name)
            os.makedirs(target, exist_ok=True)
            cmd = ["rocprofv3"] + flags + ["--output-format", "csv", "-d", target, "-o", "w", "--", probe, lib] + list(WORKLOADS[w])
            print("[counters] %s %s: %s" % (w, name, " ".join(cmd)), flush=True)
            with open(os.path.join(target, "stdout.txt"), "w") as so, open(os.path.join(target, "stderr.txt"), "w") as se:
                try:
                    rc = subprocess.run(cmd, cwd="/tmp", env=env, stdout=so, stderr=se, timeout=150).returncode
                except subprocess.TimeoutExpired:
                    sys.exit("[counters] %s %s: no end after 150 s; stopping here" % (w, name))
            if rc != 0:
                sys.exit("[counters] %s %s: exit %d; stopping here (see %s)" % (w, name, rc, target))
            with open(os.path.join(target, "command.txt"), "w") as f:
                f.write(" ".join(cmd) + "\n")
    print("[counters] done", flush=True)


def find(target, suffix):
    hits = glob.glob(os.path.join(target, "**", "*" + suffix), recursive=True)
    return hits[0] if hits else None


def counter_means(target):
    """kernel name -> counter -> (mean value a dispatch, dispatches)."""
    path = find(target, "counter_collection.csv")
    sums = {}
    if not path:
        return sums
    with open(path) as f:
        for r in csv.DictReader(f):
            s = sums.setdefault(r["Kernel_Name"], {}).setdefault(r["Counter_Name"], [0.0, 0])
            s[0] += float(r["Counter_Value"])
            s[1] += 1
    return {k: {c: (s[0] / s[1], s[1]) for c, s in v.items()} for k, v in sums.items()}


def stamp(src, to):
    meta = json.load(open(os.path.join(src, "run.json")))
    out = {"source": "rocprofv3 on tf_layer_probe (benchmark geometry, pseudo-random operands), one counter a run; "
                     "FETCH_SIZE and WRITE_SIZE in KiB a dispatch, each scaled by its reading for a 256 MiB copy kernel",
           "library_sha256": (meta.get("manifest") or {}).get("library_sha256"),
           "git": None, "workloads": {}}
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "HEAD"], capture_output=True, text=True)
        dirty = subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--", "titanic-flash-41_amd", "include"], capture_output=True, text=True)
        if head.returncode == 0:
            out["git"] = head.stdout.strip() + ("+uncommitted" if dirty.stdout.strip() else "")
    except OSError:
        pass
    for w in meta["workloads"]:
        base = os.path.join(src, w)
        entry = {"probe_arguments": " ".join(WORKLOADS[w]), "kernels": {}, "commands": {}}
        for name in sorted(os.listdir(base)):
            c = os.path.join(base, name, "command.txt")
            if os.path.exists(c):
                entry["commands"][name] = open(c).read().strip()
        for line in open(os.path.join(base, "trace", "stdout.txt")):
            if line.startswith("{"):
                entry.update(json.loads(line))
        stats = find(os.path.join(base, "trace"), "kernel_stats.csv")
        with open(stats) as f:
            for r in csv.DictReader(f):
                entry["kernels"][r["Name"]] = {"calls": int(r["Calls"]), "avg_us": float(r["AverageNs"]) / 1e3, "min_us": float(r["MinNs"]) / 1e3,
                                               "role": role_of(r["Name"])}
        fetch, write = counter_means(os.path.join(base, "fetch")), counter_means(os.path.join(base, "write"))
        copy_f = [v["FETCH_SIZE"][0] for k, v in fetch.items() if "tf_probe_copy" in k]
        copy_w = [v["WRITE_SIZE"][0] for k, v in write.items() if "tf_probe_copy" in k]
        if not copy_f or not copy_w:
            sys.exit("no copy kernel in the counter runs of " + w)
        entry["copy_kernel"] = {"bytes_each_way": COPY_BYTES, "FETCH_SIZE_KiB": copy_f[0], "WRITE_SIZE_KiB": copy_w[0]}
        scale_f, scale_w = COPY_BYTES / (copy_f[0] * 1024), COPY_BYTES / (copy_w[0] * 1024)
        entry["scale"] = {"fetch": scale_f, "write": scale_w}
        for k, rec in entry["kernels"].items():
            if k in fetch and k in write:
                rec["FETCH_SIZE_KiB"], rec["WRITE_SIZE_KiB"] = fetch[k]["FETCH_SIZE"][0], write[k]["WRITE_SIZE"][0]
                rec["hbm_bytes"] = rec["FETCH_SIZE_KiB"] * 1024 * scale_f + rec["WRITE_SIZE_KiB"] * 1024 * scale_w
                algorithmic = entry.get(rec["role"] + "_algorithmic_bytes") if rec["role"] in ("fc1", "fc2") else None
                if algorithmic:
                    rec["algorithmic_bytes"], rec["traffic_over_algorithmic"] = algorithmic, rec["hbm_bytes"] / algorithmic
        # a projection may run as more than one launch a pass (the many-row GEMM: the long units, then the experts' odd last
        # tiles): its traffic and duration are the sums over its kernels, which run once a pass each
        entry["roles"] = {}
        for role in ("fc1", "fc2"):
            recs = [r for r in entry["kernels"].values() if r["role"] == role and "hbm_bytes" in r]
            algorithmic = entry.get(role + "_algorithmic_bytes")
            if recs and algorithmic:
                total = sum(r["hbm_bytes"] for r in recs)
                entry["roles"][role] = {"kernels": len(recs), "avg_us": sum(r["avg_us"] for r in recs), "hbm_bytes": total,
                                        "algorithmic_bytes": algorithmic, "traffic_over_algorithmic": total / algorithmic}
                for r in recs:
                    if len(recs) > 1:
                        r.pop("traffic_over_algorithmic", None)
        for extra in ("l2", "shader"):
            for k, v in counter_means(os.path.join(base, extra)).items():
                if k in entry["kernels"]:
                    entry["kernels"][k].setdefault("counters", {}).update({c: m for c, (m, _) in v.items()})
        # the summary keeps the routed projections and the copy kernel in full, every other kernel as its mean duration
        entry["other_kernels_avg_us"] = {k: round(r["avg_us"], 1) for k, r in entry["kernels"].items() if r.get("role") is None}
        entry["kernels"] = {k: r for k, r in entry["kernels"].items() if r.get("role") is not None}
        out["workloads"][w] = entry
    os.makedirs(os.path.dirname(os.path.abspath(to)), exist_ok=True)
    with open(to, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    for w, entry in out["workloads"].items():
        for k, rec in entry["kernels"].items():
            if rec.get("role") in ("fc1", "fc2"):
                print("%s %-4s %-50s %9.1f us  hbm %.4g B" % (w, rec["role"], k[:50], rec["avg_us"], rec.get("hbm_bytes", float("nan"))))
        for role, rec in entry["roles"].items():
            print("%s %-4s %d kernel(s) %9.1f us  hbm %.4g B  x%.3f" % (w, role, rec["kernels"], rec["avg_us"], rec["hbm_bytes"], rec["traffic_over_algorithmic"]))


def load(path=None):
    """The stamped counter file, or None: read by bench.py."""
    path = path or os.path.join(ROOT, "profiles", "counters.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f)


def traffic_ratio(counters, workload, role="fc1"):
    """Measured HBM bytes over algorithmic bytes of the workload's kernel of that role, or None."""
    if not counters or workload not in counters.get("workloads", {}):
        return None
    entry = counters["workloads"][workload]
    if role in entry.get("roles", {}):
        return entry["roles"][role]["traffic_over_algorithmic"]
    for rec in entry["kernels"].values():
        if rec.get("role") == role and "traffic_over_algorithmic" in rec:
            return rec["traffic_over_algorithmic"]
    return None


def main():
    ap = argparse.ArgumentParser()
    sub = ap.add_subparsers(dest="what", required=True)
    r = sub.add_parser("run")
    r.add_argument("--out", required=True, help="directory for the raw profiler output")
    r.add_argument("--workloads", default="c2,c3,c4,c5")
    r.add_argument("--shader", action="store_true")
    s = sub.add_parser("stamp")
    s.add_argument("dir")
    s.add_argument("--to", default=os.path.join(ROOT, "profiles", "counters.json"))
    args = ap.parse_args()
    if args.what == "run":
        run(os.path.abspath(args.out), [w for w in args.workloads.split(",") if w in WORKLOADS], args.shader)
    else:
        stamp(args.dir, args.to)


if __name__ == "__main__":
    main()
