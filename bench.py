#!/usr/bin/env python3
"""Benchmark of the MoE FFN layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|c4|c5|r6|r4096] [--numerics benchmark|reference]

A step is one pass of the whole layer (gate product, top-k + plan + token quantization, routed FC1 + SwiGLU, FC2, shared
expert, ordered sum + shared addition) over one batch of synthetic token rows that is already resident in HBM, replayed
as a captured HIP graph as the reference replays its layer (src/probe.rs:1527-1542).  Sixteen distinct input batches
(two at many rows) are cycled so every step routes to other experts and streams their weights from HBM, not from the last
step's cache.  A graph holds one pass over each batch; a step count that is no multiple of the batch count ends with a
shorter graph over the first batches, so exactly --steps steps are timed after exactly --warmup warm-up steps.

Prints ONE JSON line.  Without --config its top level is the decode step (c2, the configuration the metric is quoted on):
whole-layer tokens/s, the roofline of the dominant kernel (FC1 + SwiGLU of the routed experts; algorithmic bytes over its
average duration, measured with two HIP events that take the kernel's start and completion on its launch stream), and the
CPU baseline (the C oracle, a port of the reference semantics: the reference has no CPU path) timed on a bounded sample of
the same workload: its vectorised build with all threads (the reported value), the scalar build with all threads and with one.  `configs` then holds the same measurement of the speculative-verify step
(c3) and the two prefill chunks (c4, c5: the routed FC1 launch between events recorded around it; its flops a byte say which
roof it lies under: at 4,096 rows an expert's weights serve 96 rows, 339 flop/B against the machine's 625, so HBM; at 16,384
rows the matrix units; the line carries the fractions of both peaks either way).  With --config only that configuration runs and is the top level.

`roofline.traffic` is the measured HBM bytes a launch of the dominant kernel: the ratio of measured to algorithmic bytes
that the committed counter file holds for the same workload (profiles/counters.json, written by
`python -m titanic-flash-41_amd.counters`; its library hash and commit are copied into the line) times the algorithmic
bytes of this run's launches; null where the file has no run of the workload.

--copy-probe appends four plain device copies of 256 MiB after the timed region: a counter run (rocprofv3 --pmc
FETCH_SIZE / WRITE_SIZE) of this program then holds a kernel of known traffic to scale the counters by.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
BATCHES = 16

CONFIGS = {
    "c2": dict(rows=4, hidden=4096, experts=256, topk=6, inter=2048, shared=2048,
               workload="decode step, 4 requests x 1 token; H 4096, E 256, top-6, I 2048, 1 shared expert (I 2048)"),
    "c3": dict(rows=32, hidden=4096, experts=256, topk=6, inter=2048, shared=2048,
               workload="speculative verify, 4 requests x 8 draft tokens = 32 rows; H 4096, E 256, top-6, I 2048, 1 shared expert"),
    "c4": dict(rows=4096, hidden=4096, experts=256, topk=6, inter=2048, shared=2048,
               workload="prefill chunk of 4096 tokens, uniform routing (iid N(0, 1) logits, no selection bias); H 4096, E 256, top-6, I 2048, 1 shared expert"),
    "c5": dict(rows=16384, hidden=4096, experts=256, topk=6, inter=2048, shared=2048,
               workload="long prefill of 16384 tokens, Zipf(1.1) expert popularity; H 4096, E 256, top-6, I 2048, 1 shared expert"),
    # not benchmark configurations: the reference's own layer (runtime/model/config.json; src/ffn.rs:65-66, 245-258), in its own numerics
    # unless --numerics says otherwise.  The expert widths (2,304) are uploaded zero-padded to 2,560; bytes and flops below count 2,304.
    "r6": dict(rows=6, hidden=5120, experts=384, topk=6, inter=2304, shared=2304,
               workload="the reference's layer, decode / verify plan of 6 rows; H 5120, E 384, top-6, I 2304, 1 shared expert (I 2304)"),
    "r4096": dict(rows=4096, hidden=5120, experts=384, topk=6, inter=2304, shared=2304,
                  workload="the reference's layer, prefill chunk of 4096 tokens; H 5120, E 384, top-6, I 2304, 1 shared expert (I 2304)"),
}
HEADLINE, OTHERS = "c2", ["c3", "c4", "c5"]
MFMA_FP8_PEAK_TFLOPS, MFMA_FP4_PEAK_TFLOPS = 5000.0, 10100.0


def make_inputs(synth, name, cfg, device, batches=BATCHES):
    import torch
    xs = []
    for step in range(batches):
        if name == "c3":   # tokens of a request share a base vector: correlated router logits
            base = synth.normal("c3/base.%d" % step, (4, 1, cfg["hidden"]), device=device)
            noise = synth.normal("c3/noise.%d" % step, (4, 8, cfg["hidden"]), std=0.3, device=device)
            xs.append(synth.to_bf16_bits((base + noise).reshape(32, cfg["hidden"])).contiguous())
        else:
            xs.append(synth.activations(name, cfg["rows"], cfg["hidden"], device=device, step=step).contiguous())
    torch.cuda.synchronize()
    return xs


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(pkg, g, ops, xs, taps_ids, budget_s=12.0, scalar_budget_s=8.0, single_budget_s=8.0):
    """Times the C oracle (staged, active experts only) on host cores for a bounded number of steps: its vectorised build
    (AVX2 + FMA projection loops, OpenMP over weight rows) with every thread the process may use (at most 16) -- the reported
    value --, then the scalar oracle with the same threads and with one thread."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle
    import helpers
    allowed = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    threads = max(1, min(allowed, 16))
    rows = xs[0].shape[0]
    # gather the operands the steps touch outside the timed regions (the oracle reads host memory)
    subsets = [_HostSubset(ops, ids, g) for ids in taps_ids]
    host_xs = [x.cpu() for x in xs]

    def timed(n_threads, budget, simd):
        oracle.set_threads(n_threads)
        done, spent = 0, 0.0
        while done < 4096 and (done == 0 or spent + spent / done < budget):
            t0 = time.perf_counter()
            helpers.oracle_layer(g, subsets[done % len(xs)], host_xs[done % len(xs)], simd=simd)
            spent += time.perf_counter() - t0
            done += 1
        return done, spent

    simd = oracle.simd_available()
    if simd:
        timed(threads, 0.0, True)           # first touch of the operands
    done, spent = timed(threads, budget_s, simd)
    done_s, spent_s = timed(threads, scalar_budget_s, False)
    done1, spent1 = timed(1, single_budget_s, False)
    oracle.set_threads(threads)
    build = "vectorised C oracle (AVX2 + FMA projection loops)" if simd else "scalar C oracle (the host has no AVX2 + FMA)"
    return {"value": rows * done / spent, "unit": "tokens/s", "cores": threads, "threads": threads, "kind": "port",
            "nproc": os.cpu_count(), "cpus_allowed": allowed, "cpu_model": cpu_model(),
            "sample": "%d steps of this workload (%d rows each), %s with %d OpenMP threads, %.1f s" % (done, rows, build, threads, spent),
            "scalar": {"value": rows * done_s / spent_s, "unit": "tokens/s", "cores": threads,
                       "sample": "%d steps of this workload, the scalar C oracle (one look-up and one fused multiply-add a product) with %d OpenMP threads, %.1f s"
                                 % (done_s, threads, spent_s)},
            "single_thread": {"value": rows * done1 / spent1, "unit": "tokens/s", "cores": 1,
                              "sample": "%d steps of this workload, the same scalar C oracle with one thread, %.1f s" % (done1, spent1)}}


class _HostSubset:
    """Host copies of the operands one step reads: the step's active experts (others stay zero) and the dense parts."""

    def __init__(self, ops, ids, g):
        import torch
        active = sorted(set(int(e) for e in ids.ravel() if e >= 0))
        pick = torch.as_tensor(active, dtype=torch.long, device=ops.w13.device)
        self.active = active
        for name in ["gate_w", "bias", "bias_alt", "sh_w13", "sh_s13", "sh_w2", "sh_s2"]:
            setattr(self, name, getattr(ops, name).cpu())
        for name in ["w13", "s13", "w2", "s2"]:
            full = getattr(ops, name)
            setattr(self, name, _Sparse(full, pick, active))


class _Sparse:
    """Expert-major tensor of which only some experts are held on the host; indexing with a tensor of expert ids returns them."""

    def __init__(self, full, pick, active):
        self.data = full[pick].cpu()
        self.index = {e: i for i, e in enumerate(active)}
        self.device = self.data.device

    def __getitem__(self, ids):
        import torch
        at = [self.index[int(e)] for e in ids]
        if at == list(range(self.data.shape[0])):      # the held experts in their own order: no copy
            return self.data
        return self.data[torch.as_tensor(at, dtype=torch.long)]


def geometry_of(native, cfg, numerics):
    if numerics == "benchmark":
        return native.Geometry(cfg["hidden"], cfg["experts"], cfg["topk"], cfg["inter"], cfg["shared"], 0, 1.0, 128, 128, 128, -1, 10.0)
    return native.Geometry(cfg["hidden"], cfg["experts"], cfg["topk"], cfg["inter"], cfg["shared"], 1, 1.5, 32, 32, 32, 129264, 10.0)


def measure(pkg, name, numerics, steps, warmup, profile_steps, overlap, operands, counter_file, with_cpu):
    """One configuration: the whole-layer rate by graph replay, the dominant kernel's duration by HIP events, the
    algorithmic bytes and flops of the launches that ran.  Returns the record and what the CPU baseline needs."""
    import copy
    import numpy as np
    import torch
    native, synth, host, counters = pkg.native, pkg.synth, pkg.host, pkg.counters
    cfg = CONFIGS[name]
    g = geometry_of(native, cfg, numerics)
    B, BN, BK = g.act_block, g.shared_bn, g.shared_bk
    t0 = time.time()
    wide = cfg["rows"] > 64
    batches = 2 if wide else BATCHES
    if wide:
        steps, warmup, profile_steps = min(steps, 200), min(warmup, 20), min(profile_steps, 8)
    key = (cfg["hidden"], cfg["experts"], cfg["inter"], cfg["shared"], numerics)
    if key not in operands:     # the benchmark configurations share one geometry: one set of synthetic weights serves them all
        operands[key] = synth.LayerOperands(g, "bench/%d/%d" % (cfg["hidden"], cfg["experts"]), device="cuda")
    ops = operands[key]
    if name == "c4":      # uniform routing: no selection bias (the layer's N(0, 0.1) bias alone gives the busiest expert ten times the mean load)
        ops = copy.copy(ops)
        ops.bias = torch.zeros_like(ops.bias)
    if name == "c5":      # expert popularity ~ rank^-1.1: the busiest experts take more than ten times the mean load
        ops = copy.copy(ops)
        ops.bias = synth.zipf_bias(g.experts, 1.1, 0.06, device="cuda")
    xs = make_inputs(synth, name, cfg, "cuda", batches)
    layer = host.Layer(g, ops, cfg["rows"]) if overlap is None else host.Layer(g, ops, cfg["rows"], overlap=bool(overlap))
    layer.set_tokens()
    layer.keep_intermediate(False)      # many rows: FC2 reads the FP8 codes; the BF16 copy is a tap the tests ask for
    setup_s = time.time() - t0

    # per-kernel durations (HIP events on the launch stream) and the routing of every batch
    ids_per_batch, parts = [], np.zeros(7)
    tiles_per_batch = []
    fc1_kernel = 0.0
    if wide:
        # many rows: one eager pass at a time, events around each part (router, front-end, FC1, FC2, shared expert, sum)
        for x in xs:                      # warm every batch once
            layer.profile_step(x)
        passes = 0
        for i in range(profile_steps):
            x = xs[i % batches]
            parts += np.array(layer.profile_step(x))
            passes += 1
            if i < batches:
                ids_per_batch.append(layer.tap("ids").reshape(cfg["rows"], cfg["topk"]).copy())
                tiles_per_batch.append(int(layer.tap("tile_base")[-1]))
        parts /= passes
    else:
        # few rows: the schedule of the timed region itself (front-end, FC1 and FC2 with the shared expert inside, sum), eager,
        # every pass enqueued before the first wait, the library's marks between the launches
        for x in xs:
            layer.run(x)
            ids_per_batch.append(layer.tap("ids").reshape(cfg["rows"], cfg["topk"]).copy())
            tiles_per_batch.append(int(layer.tap("tile_base")[-1]))
        layer.profile_marks(xs, batches)
        front, fc1, fc2, total, whole, _ = layer.profile_marks(xs, max(profile_steps, batches) * 4)
        fc1_kernel = layer.profile_marks(xs, max(profile_steps, batches) * 4, exact=True)[5]
        parts = np.array([0.0, front, fc1, fc2, 0.0, total, whole])
    H, I, S, E, K, rows = cfg["hidden"], cfg["inter"], cfg["shared"], cfg["experts"], cfg["topk"], cfg["rows"]
    distinct = float(np.mean([len(set(ids[ids >= 0].ravel().tolist())) for ids in ids_per_batch]))
    tiles = float(np.mean(tiles_per_batch))
    routes = float(np.mean([(ids >= 0).sum() for ids in ids_per_batch]))
    if wide:
        # grouped GEMM: every expert with rows streams its weights and scales once, every route reads its token's codes and
        # scales once and writes FP8 codes and block scales of the intermediate (FC2: reads those, writes BF16 route outputs)
        fc1_bytes = distinct * (2 * I * H // 2 + 2 * I * H // 32) + routes * (H + H / B) + routes * (I + I / B)
        fc2_bytes = distinct * (H * I // 2 + H * I // 32) + routes * (I + I / B) + routes * H * 2
    else:
        # streaming launches: every 16-row tile reads one expert's up + gate weights and scales once
        fc1_bytes = tiles * (2 * I * H // 2 + 2 * I * H // 32) + rows * (H + H // B) + rows * K * I * 2
        fc2_bytes = tiles * (H * I // 2 + H * I // 32) + rows * K * I * 2 + rows * K * H * 2
    shared_bytes = 3 * H * S + rows * (H + 2 * S * 2 + S * 2 + H * 2)
    router_bytes = 2 * E * H + rows * H * 2
    step_bytes = fc1_bytes + fc2_bytes + shared_bytes + router_bytes + rows * (K + 2) * H * 2
    # few rows: the shared expert's projections stream inside the same two launches
    shared_fc1_bytes = 2 * S * H + (2 * S // BN) * (H // BK) + rows * (H + H // B) + rows * S * 2
    shared_fc2_bytes = H * S + (H // BN) * (S // BK) + rows * S * 2 + rows * H * 2
    # owners of at most eight rows: the shared expert's first projection streams inside the front-end launch, not in this one
    early_shared = rows <= 64 and H <= 5120
    phase1_bytes = fc1_bytes + (0 if wide or early_shared else shared_fc1_bytes)
    phase2_bytes = fc2_bytes + (0 if wide else shared_fc2_bytes)
    fc1_ms = float(parts[2])
    # few rows: the dominant kernel's own duration, between two events that take its start and its completion (the interval
    # between the marks before and after it also holds the gap to the previous launch, about 3 us)
    fc1_kernel_ms = float(fc1_kernel) if not wide and fc1_kernel > 0 else fc1_ms
    achieved = phase1_bytes / (fc1_kernel_ms * 1e-3) / 1e9
    fc1_flops, fc2_flops = routes * 2 * (2 * I) * H, routes * 2 * H * I
    step_flops = fc1_flops + fc2_flops + rows * (6 * H * S + 2 * H * E)
    max_load = float(np.mean([np.bincount(ids[ids >= 0].ravel(), minlength=E).max() for ids in ids_per_batch]))

    # whole-layer throughput by graph replay (as the reference replays a graph of its forty layers' passes); a step is one pass,
    # the input batches take turns.  A graph holds `per_graph` passes; a count that is no multiple of it ends with a graph of
    # exactly the remainder, so exactly the steps asked for run, in the warm-up and in the timed region (a short count is one
    # graph of its own: a second graph's first launch costs the region about 30 us)
    per_graph = batches if wide else 16 * batches
    graphs = {}

    def graph_of(passes):
        if passes not in graphs:
            graphs[passes] = layer.capture([xs[i % batches] for i in range(passes)])
        return graphs[passes]

    def launches(count):
        order = [graph_of(per_graph)] * (count // per_graph)
        if count % per_graph:
            order.append(graph_of(count % per_graph))
        return order
    warm_order, timed_order = launches(warmup), launches(steps)
    torch.cuda.synchronize()
    ms = layer.time(warm_order + timed_order, len(warm_order), len(timed_order))
    torch.cuda.synchronize()
    ms_per_step = ms / steps
    value = rows / (ms_per_step * 1e-3)

    ratio = counters.traffic_ratio(counter_file, name) if numerics == "benchmark" else None
    traffic_source = None
    if ratio is not None:
        traffic_source = {"file": "profiles/counters.json", "git": counter_file.get("git"), "library_sha256": counter_file.get("library_sha256"),
                          "same_library_as_this_run": counter_file.get("library_sha256") == native.library_sha256(),
                          "traffic_over_algorithmic": ratio}
    if wide:
        tflops = fc1_flops / (fc1_ms * 1e-3) / 1e12
        # which roof the launch lies under: its flops a byte against the machine's (FP8 peak over HBM peak, 625 flop/B)
        gbs = fc1_bytes / (fc1_ms * 1e-3) / 1e9
        intensity, ridge = fc1_flops / fc1_bytes, MFMA_FP8_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
        hbm_side = intensity < ridge
        roofline = {"bound": "hbm" if hbm_side else "mfma", "kernel": "tf_grouped_gemm<FC1> (routed FC1 + SwiGLU + FP8 requantization)",
                    "achieved": gbs if hbm_side else tflops, "peak": HBM_PEAK_GBS if hbm_side else MFMA_FP8_PEAK_TFLOPS,
                    "unit": "GB/s" if hbm_side else "TFLOP/s", "frac": gbs / HBM_PEAK_GBS if hbm_side else tflops / MFMA_FP8_PEAK_TFLOPS,
                    "flop_per_byte": intensity, "ridge_flop_per_byte": ridge,
                    "tflops": tflops, "frac_of_fp8_peak": tflops / MFMA_FP8_PEAK_TFLOPS, "frac_of_fp4_peak": tflops / MFMA_FP4_PEAK_TFLOPS,
                    "frac_of_hbm_peak": gbs / HBM_PEAK_GBS,
                    "operands": "A = FP8 E4M3 activations, B = FP4 E2M1 weights: issues at the FP8 rate (measured)",
                    "traffic": ratio * fc1_bytes if ratio is not None else None, "traffic_source": traffic_source,
                    "bytes_or_flops_per_launch": fc1_flops, "per_launch_unit": "flop", "algorithmic_bytes_per_launch": fc1_bytes,
                    "avg_launch_ms": fc1_ms,
                    "timing": "HIP events recorded around the launch on its stream, eager passes of the layer's schedule"}
    else:
        roofline = {"bound": "hbm", "kernel": ("tf_phase1_stream (FC1 + SwiGLU of the routed experts; the shared expert's first projection streams in the front-end launch)"
                                               if early_shared else "tf_phase1_stream (FC1 + SwiGLU of the routed experts and the shared expert in one launch)"),
                    "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                    "traffic": ratio * phase1_bytes if ratio is not None else None, "traffic_source": traffic_source,
                    "bytes_or_flops_per_launch": phase1_bytes, "per_launch_unit": "byte", "avg_launch_ms": fc1_kernel_ms, "launch_to_launch_ms": fc1_ms,
                    "timing": "HIP events bound to the kernel's start and completion (hipExtLaunchKernelGGL) on its launch stream, eager passes of the layer's schedule"}
    record = {
        "value": value, "unit": "tokens/s", "steps": steps, "warmup": warmup, "ms_per_step": ms_per_step,
        "steps_note": "%d steps after %d warm-up steps: replays of a %d-pass graph, a graph of exactly the remainder after them" % (steps, warmup, per_graph),
        "config": {"workload": name + ": " + cfg["workload"],
                   "numerics": ("sigmoid top-k renormalised, 128-wide activation blocks" if numerics == "benchmark" else
                                "reference numerics: sqrt-softplus scores x 1.5, 32-wide activation blocks, 32 x 32 shared weight blocks"),
                   "input_batches": batches, "distinct_experts_per_step": distinct, "schedule": "HIP graph replay (%d passes a graph)" % per_graph},
        "roofline": roofline,
        "step_tflops": step_flops / (ms_per_step * 1e-3) / 1e12, "busiest_expert_rows": max_load, "phys_tiles": tiles,
        "step_bytes": step_bytes, "step_gbs": step_bytes / (ms_per_step * 1e-3) / 1e9, "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "kernel_ms": {"router": float(parts[0]), "front_end": float(parts[1]), "fc1_swiglu": fc1_ms, "fc2": float(parts[3]),
                      "shared_expert": float(parts[4]), "sum_shared": float(parts[5]), "eager_pass": float(parts[6])},
        "kernel_gbs": {"fc2": phase2_bytes / (float(parts[3]) * 1e-3) / 1e9},
        "kernel_tflops": {"fc2": fc2_flops / (float(parts[3]) * 1e-3) / 1e12},
        "setup_s": setup_s,
    }
    if with_cpu:
        record["cpu_baseline"] = cpu_baseline(pkg, g, ops, xs, ids_per_batch)
    layer.close()
    del layer, xs
    torch.cuda.empty_cache()
    return record


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--config", default=None, choices=sorted(CONFIGS),
                    help="measure only this configuration; default: c2 as the headline and c3, c4, c5 under `configs`")
    ap.add_argument("--numerics", default=None, choices=["benchmark", "reference"],
                    help="benchmark: sigmoid scores, renormalised, 128-wide activation blocks, 128 x 128 shared weight blocks (the headline); "
                         "reference: the reference's own numerics (sqrt-softplus x 1.5, 32-wide blocks, 32 x 32, image-token bias)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--overlap", type=int, default=None, choices=[0, 1],
                    help="many rows: the shared expert on a second stream beside the routed experts (the reference's dual-stream schedule, "
                         "src/ffn.rs:1000-1040) or after them on the same stream; default: the layer's own choice")
    ap.add_argument("--copy-probe", action="store_true", help="append four 256 MiB device copies (counter calibration)")
    ap.add_argument("--profile-steps", type=int, default=64, help="eager passes with per-kernel HIP events for the roofline")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the layer runs on a single MI355X (no sharding, no collectives); --gpus %d is not supported" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import torch
    pkg = importlib.import_module("titanic-flash-41_amd")
    pkg.counters = importlib.import_module("titanic-flash-41_amd.counters")
    torch.cuda.set_device(0)
    counter_file = pkg.counters.load()
    headline = args.config or HEADLINE
    numerics = args.numerics or ("reference" if headline.startswith("r") else "benchmark")
    operands = {}
    record = measure(pkg, headline, numerics, args.steps, args.warmup, args.profile_steps, args.overlap, operands, counter_file,
                     not args.no_cpu_baseline)
    line = {"metric": "MoE-layer tokens/s", "value": record.pop("value"), "unit": record.pop("unit"), "n_gpus": 1,
            "steps": record.pop("steps"), "warmup": record.pop("warmup"), "ms_per_step": record.pop("ms_per_step"),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "fp4 (e2m1 weights, ue8m0 scales) x fp8 (e4m3 activations), f32 accumulate", "data": "synthetic"}
    line.update(record)
    if args.config is None:
        # the other benchmark configurations, each with its own step counts (the headline's are the ones asked for)
        line["configs"] = {}
        for name in OTHERS:
            line["configs"][name] = measure(pkg, name, "benchmark", 2000, 200, args.profile_steps, args.overlap, operands, counter_file, False)
    if args.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
