#!/usr/bin/env python3
"""Benchmark of the MoE FFN layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c3|c4|c5|r6|r4096] [--numerics benchmark|reference]

A step is one pass of the whole layer (gate product, top-k + plan + token quantization, routed FC1 + SwiGLU, FC2, shared
expert, ordered sum + shared addition) over one batch of synthetic token rows that is already resident in HBM, replayed
as a captured HIP graph as the reference replays its layer (src/probe.rs:1527-1542).  Sixteen distinct input batches
are cycled so every step routes to other experts and streams their weights from HBM, not from the last step's cache.

Prints one JSON line: whole-layer tokens/s, the roofline of the dominant kernel (FC1 + SwiGLU of the routed experts;
algorithmic bytes over its average duration, measured with two HIP events that take the kernel's start and completion
on its launch stream; many rows: events recorded around the launch), and the CPU baseline (the C oracle, a port of the reference semantics: the
reference has no CPU path) timed on a bounded sample of the same workload.

--copy-probe appends four plain device copies of 256 MiB after the timed region: a counter run (rocprofv3 --pmc
FETCH_SIZE / WRITE_SIZE) then holds a kernel of known traffic to scale the counters by.
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
               workload="prefill chunk of 4096 tokens, uniform routing; H 4096, E 256, top-6, I 2048, 1 shared expert"),
    "c5": dict(rows=16384, hidden=4096, experts=256, topk=6, inter=2048, shared=2048,
               workload="long prefill of 16384 tokens, Zipf(1.1) expert popularity; H 4096, E 256, top-6, I 2048, 1 shared expert"),
    # not benchmark configurations: the reference's own layer (runtime/model/config.json; src/ffn.rs:65-66, 245-258), in its own numerics
    # unless --numerics says otherwise.  The expert widths (2,304) are uploaded zero-padded to 2,560; bytes and flops below count 2,304.
    "r6": dict(rows=6, hidden=5120, experts=384, topk=6, inter=2304, shared=2304,
               workload="the reference's layer, decode / verify plan of 6 rows; H 5120, E 384, top-6, I 2304, 1 shared expert (I 2304)"),
    "r4096": dict(rows=4096, hidden=5120, experts=384, topk=6, inter=2304, shared=2304,
                  workload="the reference's layer, prefill chunk of 4096 tokens; H 5120, E 384, top-6, I 2304, 1 shared expert (I 2304)"),
}
MFMA_FP8_PEAK_TFLOPS, MFMA_FP4_PEAK_TFLOPS = 5000.0, 10100.0
# Measured HBM traffic of the dominant kernel over its algorithmic bytes, from the counter runs summarized under profiles/
# (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, on tf_layer_probe: the same geometry, rows and schedule with random operands;
# each counter scaled by its reading for a 256 MiB copy kernel).  The line's `traffic` is this ratio times the algorithmic
# bytes of this run's launches; None where no counter run exists for the configuration.
TRAFFIC_OVER_ALGORITHMIC = {"c2": 1.0003}
# Many rows: HBM bytes a launch of the routed FC1 kernel, measured the same way at the same number of rows.
WIDE_TRAFFIC_BYTES = {"c4": 3.24e9, "c5": 6.92e9}


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


def cpu_baseline(pkg, g, ops, xs, taps_ids, budget_s=20.0):
    """Times the C oracle (staged, active experts only) on host cores for a bounded number of steps."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle
    import helpers
    threads = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    threads = max(1, min(threads, 16))
    oracle.set_threads(threads)
    rows = xs[0].shape[0]
    done, spent = 0, 0.0
    while done < 4 * len(xs) and (done == 0 or spent + spent / done < budget_s):
        x = xs[done % len(xs)]
        # gather the operands the step touches outside the timed region (the oracle reads host memory)
        small_ops = _HostSubset(ops, taps_ids[done % len(xs)], g)
        t0 = time.perf_counter()
        helpers.oracle_layer(g, small_ops, x.cpu())
        spent += time.perf_counter() - t0
        done += 1
    return {"value": rows * done / spent, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": "%d steps of this workload (%d rows each), C oracle with %d OpenMP threads, %.1f s" % (done, rows, threads, spent)}


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
        return self.data[torch.as_tensor([self.index[int(e)] for e in ids], dtype=torch.long)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
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
    import numpy as np
    import torch
    pkg = importlib.import_module("titanic-flash-41_amd")
    native, synth, host = pkg.native, pkg.synth, pkg.host
    cfg = CONFIGS[args.config]
    if args.numerics is None:
        args.numerics = "reference" if args.config.startswith("r") else "benchmark"
    if args.numerics == "benchmark":
        g = native.Geometry(cfg["hidden"], cfg["experts"], cfg["topk"], cfg["inter"], cfg["shared"], 0, 1.0, 128, 128, 128, -1, 10.0)
    else:
        g = native.Geometry(cfg["hidden"], cfg["experts"], cfg["topk"], cfg["inter"], cfg["shared"], 1, 1.5, 32, 32, 32, 129264, 10.0)
    B, BN, BK = g.act_block, g.shared_bn, g.shared_bk
    torch.cuda.set_device(0)
    t0 = time.time()
    wide = cfg["rows"] > 64
    batches = 2 if wide else BATCHES
    if wide:
        args.steps, args.warmup, args.profile_steps = min(args.steps, 200), min(args.warmup, 20), min(args.profile_steps, 8)
    ops = synth.LayerOperands(g, args.config, device="cuda")
    if args.config == "c5":      # expert popularity ~ rank^-1.1: the busiest experts take more than ten times the mean load
        ops.bias = synth.zipf_bias(g.experts, 1.1, 0.06, device="cuda")
    xs = make_inputs(synth, args.config, cfg, "cuda", batches)
    layer = host.Layer(g, ops, cfg["rows"]) if args.overlap is None else host.Layer(g, ops, cfg["rows"], overlap=bool(args.overlap))
    layer.set_tokens()
    layer.keep_intermediate(False)      # many rows: FC2 reads the FP8 codes; the BF16 copy is a tap the tests ask for
    setup_s = time.time() - t0

    # per-kernel durations (HIP events on the launch stream) and the routing of every batch
    ids_per_batch, parts = [], np.zeros(7)
    tiles_per_batch = []
    if wide:
        # many rows: one eager pass at a time, events around each part (router, front-end, FC1, FC2, shared expert, sum)
        for x in xs:                      # warm every batch once
            layer.profile_step(x)
        passes = 0
        for i in range(args.profile_steps):
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
        front, fc1, fc2, total, whole, _ = layer.profile_marks(xs, max(args.profile_steps, batches) * 4)
        fc1_kernel = layer.profile_marks(xs, max(args.profile_steps, batches) * 4, exact=True)[5]
        parts = np.array([0.0, front, fc1, fc2, 0.0, total, whole])
    H, I, S, E, K, rows = cfg["hidden"], cfg["inter"], cfg["shared"], cfg["experts"], cfg["topk"], cfg["rows"]
    distinct = float(np.mean([len(set(ids.ravel().tolist())) for ids in ids_per_batch]))
    tiles = float(np.mean(tiles_per_batch))
    # algorithmic bytes: every streamed tile of FC1 reads one expert's up + gate weights and scales once
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
    routes = float(np.mean([(ids >= 0).sum() for ids in ids_per_batch]))
    fc1_flops, fc2_flops = routes * 2 * (2 * I) * H, routes * 2 * H * I
    step_flops = fc1_flops + fc2_flops + rows * (6 * H * S + 2 * H * E)
    max_load = float(np.mean([np.bincount(ids[ids >= 0].ravel(), minlength=E).max() for ids in ids_per_batch]))

    # whole-layer throughput: one graph holds a pass over each of the sixteen batches (as the reference's graph holds its forty
    # layers' passes); a step is one pass, so steps and warmup are rounded up to whole replays
    graph = layer.capture(xs)
    torch.cuda.synchronize()
    replays, warm = -(-args.steps // batches), -(-args.warmup // batches)
    args.steps, args.warmup = replays * batches, warm * batches
    ms = layer.time([graph], warm, replays)
    torch.cuda.synchronize()
    ms_per_step = ms / args.steps
    value = rows / (ms_per_step * 1e-3)

    line = {
        "metric": "MoE-layer tokens/s", "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp4 (e2m1 weights, ue8m0 scales) x fp8 (e4m3 activations), f32 accumulate",
        "data": "synthetic", "config": {"workload": args.config + ": " + cfg["workload"], "numerics": ("sigmoid top-k renormalised, 128-wide activation blocks" if args.numerics == "benchmark" else
                                                     "reference numerics: sqrt-softplus scores x 1.5, 32-wide activation blocks, 32 x 32 shared weight blocks"),
                                        "input_batches": batches, "distinct_experts_per_step": distinct, "schedule": "HIP graph replay (%d passes a graph)" % batches},
        "roofline": ({"bound": "mfma", "kernel": "tf_gemm<fp4, FC1> (routed FC1 + SwiGLU + FP8 requantization)",
                      "achieved": fc1_flops / (fc1_ms * 1e-3) / 1e12, "peak": MFMA_FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
                      "frac": fc1_flops / (fc1_ms * 1e-3) / 1e12 / MFMA_FP8_PEAK_TFLOPS,
                      "frac_of_fp4_peak": fc1_flops / (fc1_ms * 1e-3) / 1e12 / MFMA_FP4_PEAK_TFLOPS,
                      "operands": "A = FP8 E4M3 activations, B = FP4 E2M1 weights: issues at the FP8 rate (measured)",
                      "traffic": WIDE_TRAFFIC_BYTES.get(args.config) if args.numerics == "benchmark" else None, "traffic_source": "rocprofv3 counters on tf_layer_probe at the same rows (profiles/)",
                      "flops_per_launch": fc1_flops, "avg_launch_ms": fc1_ms, "weight_gbs": fc1_bytes / (fc1_ms * 1e-3) / 1e9} if wide else
                     {"bound": "hbm", "kernel": ("tf_phase1_stream (FC1 + SwiGLU of the routed experts; the shared expert's first projection streams in the front-end launch)"
                                                  if early_shared else "tf_phase1_stream (FC1 + SwiGLU of the routed experts and the shared expert in one launch)"),
                      "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                      "traffic": (TRAFFIC_OVER_ALGORITHMIC[args.config] * phase1_bytes
                                  if args.config in TRAFFIC_OVER_ALGORITHMIC and args.numerics == "benchmark" else None),
                      "bytes_per_launch": phase1_bytes, "avg_launch_ms": fc1_kernel_ms, "launch_to_launch_ms": fc1_ms,
                      "timing": "HIP events bound to the kernel's start and completion (hipExtLaunchKernelGGL) on its launch stream, eager passes of the layer's schedule"}),
        "step_tflops": step_flops / (ms_per_step * 1e-3) / 1e12, "busiest_expert_rows": max_load, "phys_tiles": tiles,
        "step_bytes": step_bytes, "step_gbs": step_bytes / (ms_per_step * 1e-3) / 1e9, "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "kernel_ms": {"router": float(parts[0]), "front_end": float(parts[1]), "fc1_swiglu": fc1_ms, "fc2": float(parts[3]),
                      "shared_expert": float(parts[4]), "sum_shared": float(parts[5]), "eager_pass": float(parts[6])},
        "kernel_gbs": {"fc2": phase2_bytes / (float(parts[3]) * 1e-3) / 1e9},
        "setup_s": setup_s,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(pkg, g, ops, xs, ids_per_batch)
    if args.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
    layer.close()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
