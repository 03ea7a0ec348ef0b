"""GPU regression tests of the boundary's robustness items: the front-end's bounded in-launch waits (a wait that expires makes
the waiter do the work itself and marks the hand-off region; later launches stay correct; the host's reset restores the
fast path), layers of two geometries alive in one process, and the few-row dense product of entry `gemm.dense`."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import GpuLayer, bf16_ulp_distance, configure, geometry, native, np_of, pkg, synth
from test_gpu_layer import check_layer

pytestmark = pytest.mark.gpu
host = pkg.host
DIRTY_WORD = 32 * 19          # the word a kernel sets when one of its waits has expired (words of four bytes)


@pytest.mark.parametrize("rows,hidden,experts,topk,inter,shared,mode", [
    (4, 1024, 64, 2, 512, 512, "benchmark"),      # owners of at most eight rows: block 0 takes the logits from the mailbox
    (40, 2048, 64, 6, 1024, 1024, "reference"),   # more rows: row groups route themselves; the shared expert's item blocks wait for the quantizer blocks
])
def test_expired_waits_keep_every_launch_right(rows, hidden, experts, topk, inter, shared, mode):
    g = geometry(hidden, experts, topk, inter, shared, mode)
    name = "handoff-%d" % rows
    ops = synth.LayerOperands(g, name, device="cuda")
    xs = [synth.activations(name, rows, hidden, step=i) for i in range(4)]
    layer = host.Layer(g, ops, rows)
    # the larger owner also carries padding rows of a batched step (its last four rows take the routes of rows 0 - 3 with zero
    # weights): after an expired wait block 0 writes them, and the row groups' own routers, still running, must leave them alone
    live, padding = None, None
    if rows > 16:
        live = rows - 4
        padding = np.full(rows, -1, np.int32)
        padding[live:] = np.arange(4)
    layer.set_tokens(live=live, padding=padding)

    def run(x):
        layer.run(x.cuda())
        check_layer(g, ops, x, layer.taps(), live=live, padding=padding, exact_logits=rows <= 16, max_rel=2e-2)
        return layer.tap("sync")

    sync = run(xs[0])                               # ordinary launch: every hand-off in time, the region is left zero
    assert not sync.any()
    layer.spin_limit(0)                             # every wait gives up at once: each waiter does the work itself (all kernels end normally)
    sync = run(xs[1])
    assert sync[DIRTY_WORD] == 1                    # ... and says so; what the late producers posted stays in the region
    layer.spin_limit(1 << 18)
    sync = run(xs[2])                               # the next ordinary launch trusts nothing of the marked region: still right
    assert sync[DIRTY_WORD] == 1
    layer.zero_sync()                               # the host's reset
    sync = run(xs[3])                               # fast path again, and the region is zero after it
    assert not sync.any()
    layer.close()


def test_two_geometries_side_by_side():
    """The reference keeps a 384-expert target and a 128-expert drafter in one process (src/layer_id.rs:39-47): two layers of
    different geometries, their launches interleaved, each with the by-name functions of its own context."""
    ga, gb = geometry(1024, 16, 2, 512, 512, "reference"), geometry(512, 8, 1, 512, 1024, "benchmark")
    opa, opb = synth.LayerOperands(ga, "side-a", device="cuda"), synth.LayerOperands(gb, "side-b", device="cuda")
    # separate gate product, top-k, shared SwiGLU and addition: the functions that read a geometry
    la = host.Layer(ga, opa, 6, overlap=False, sum_shared=False, route_front=False, fold_shared=False, gate_front=False)
    lb = host.Layer(gb, opb, 5, overlap=False, sum_shared=False, route_front=False, fold_shared=False, gate_front=False)
    la.set_tokens()
    lb.set_tokens()
    xa, xb = synth.activations("side-a", 6, 1024), synth.activations("side-b", 5, 512)
    for _ in range(2):
        la.run(xa.cuda())
        lb.run(xb.cuda())
        check_layer(ga, opa, xa, la.taps(), max_rel=2e-2)
        check_layer(gb, opb, xb, lb.taps(), max_rel=2e-2)
    la.close()
    lb.close()


def test_dense_product_of_few_rows():
    """Entry `gemm.dense` at the row counts the reference launches it with (6: src/fp8_linear.rs:883-897)."""
    g = geometry(1024, 16, 2, 512, 512, "reference")
    ctx = configure(g)
    rng = np.random.default_rng(5)
    for m, n, k in [(6, 512, 1024), (1, 1024, 512), (33, 512, 1024)]:
        a = (rng.standard_normal((m, k)) * 2).astype(np.float32)
        aq, a_s = oracle.quantize_rows(oracle.f32_to_bf16(a), g.act_block, 1e-4)
        wq = rng.integers(0, 256, (n, k), dtype=np.uint8) & 0xBF                      # finite E4M3 codes below 2
        ws = rng.integers(118, 122, (n // g.shared_bn, k // g.shared_bk), dtype=np.uint8)
        want = oracle.fp8_linear(aq, a_s, g.act_block, wq, ws, g.shared_bn, g.shared_bk)
        dev = lambda v: torch.from_numpy(np.ascontiguousarray(v)).cuda()
        d_w, d_wp = dev(wq), torch.empty(n * k, dtype=torch.uint8, device="cuda")
        native.launch("ca_dense_compact_fp8", (n * (k // 16) + 255) // 256, 256, [d_w, d_wp, n, k, 0])
        out = torch.zeros((m, n), dtype=torch.int16, device="cuda")
        st = native.primitives_launch(ctx, 4, [dev(aq), dev(a_s), d_wp, dev(ws), out], [m, n, k])
        torch.cuda.synchronize()
        assert st == 0, st
        assert bf16_ulp_distance(np_of(out).view(np.uint16), want) <= 1.0, (m, n, k)
    native.load().ca_primitives_close(ctypes.c_void_p(ctx))


def test_micro_sequence_keeps_fp32_projections_and_equals_entry_0():
    # the reference's micro sequence (src/moe.rs:379-393, 625-629): gemm.mxfp8_quant_cute, moe.w4a8.compact_micro with an FP32
    # projections buffer, moe.w4a16.topk_sum, through entries 12, 11, 2 with the operand lists of
    # contracts/runtime-contract-micro-m4.json.  Route outputs and the sum: the bits of entry 0 (same arithmetic, a pair's
    # result does not depend on how the routes are grouped); the FP32 projections: the oracle's within FP32 accumulation order.
    import json
    import os
    from helpers import oracle_config
    g = geometry(1024, 16, 2, 512, 512, "reference")
    ops = synth.LayerOperands(g, "micro", device="cuda")
    rows = 4
    x = synth.activations("micro", rows, g.hidden).cuda().contiguous()
    layer = GpuLayer(g, ops, rows)
    taps = layer.run(x, fuse_route=False)
    K, H, I, E, B = g.topk, g.hidden, g.intermediate, g.experts, g.act_block
    pairs = rows * K
    tiles = -(-pairs // 16) - 1 + min(E, pairs)
    d = "cuda"
    values = torch.zeros((rows, H), dtype=torch.uint8, device=d)
    scale_rows = torch.zeros((rows, H // B), dtype=torch.uint8, device=d)
    scale_mma = torch.zeros((rows, H // B), dtype=torch.uint8, device=d)
    assert native.primitives_launch(layer.ctx, 12, [x, values, scale_rows, scale_mma], [rows, H, rows * 10]) == 0
    torch.cuda.synchronize()
    assert np.array_equal(np_of(values), taps["xq"]) and np.array_equal(np_of(scale_rows), taps["xs"]) and torch.equal(scale_rows, scale_mma)
    floored = torch.zeros_like(values), torch.zeros_like(scale_rows)
    assert native.primitives_launch(layer.ctx, 13, [x, floored[0], floored[1], None], [rows, H, 0]) == 0
    torch.cuda.synchronize()
    assert np.array_equal(np_of(floored[0]), taps["xq_min"]) and np.array_equal(np_of(floored[1]), taps["xs_min"])
    inter = torch.zeros((tiles * 16, I), dtype=torch.int16, device=d)
    proj = torch.full((pairs, 2 * I), float("nan"), dtype=torch.float32, device=d)
    route_out = torch.zeros((rows, K, H), dtype=torch.int16, device=d)
    ones = torch.ones(16, dtype=torch.float32, device=d)
    tables = [torch.full((tiles,), -1, dtype=torch.int32, device=d), torch.full((tiles,), -1, dtype=torch.int32, device=d),
              torch.full((E + 1,), -1, dtype=torch.int32, device=d), torch.full((tiles * 16,), -1, dtype=torch.int32, device=d),
              torch.zeros((tiles * 16,), dtype=torch.float32, device=d)]
    micro = [values, scale_rows, layer.w13, layer.s13, inter, proj, layer.weights, layer.ids, ones, ones, layer.w2, layer.s2, route_out, ones, ones] + tables
    assert native.primitives_launch(layer.ctx, 11, micro, [pairs, 48]) == 0
    out = torch.zeros((rows, H), dtype=torch.int16, device=d)
    assert native.primitives_launch(layer.ctx, 2, [route_out, out, out], [rows, 0, 0]) == 0      # third pointer: reserved, never read
    torch.cuda.synchronize()
    assert np.array_equal(np_of(route_out).view(np.uint16), taps["route_out"])
    assert np.array_equal(np_of(out).view(np.uint16), taps["routed"])
    _, want_proj = oracle.expert_fc1(oracle_config(g), taps["xq"], taps["xs"], np_of(ops.w13), np_of(ops.s13), taps["ids"], want_proj=True)
    got = np_of(proj).reshape(rows, K, 2 * I)
    assert np.isfinite(got).all()
    assert np.abs(got - want_proj).max() <= 2e-5 * np.abs(want_proj).max()
    # argument checks: a pair count that is no multiple of top-k, too many rows
    assert native.primitives_launch(layer.ctx, 11, micro, [pairs + 1, 48]) == -1
    assert native.primitives_launch(layer.ctx, 11, micro, [65 * K, 48]) == -1
    # the committed contract names these entries and operand lists
    root = os.path.join(os.path.dirname(os.path.abspath(native.__file__)), "contracts")
    contract = json.load(open(os.path.join(root, "runtime-contract-micro-m4.json")))
    bindings = json.load(open(os.path.join(root, "bindings.json")))
    assert [n["kernel_id"] for n in contract["nodes"]] == ["gemm.mxfp8_quant_cute", "moe.w4a8.compact_micro", "moe.w4a16.topk_sum"]
    assert contract["projection_dtype"] == "float32"
    for node in contract["nodes"]:
        entry = bindings["entries"][node["entry"]]
        assert entry["kernel_id"] == node["kernel_id"] and set(entry["pointers"]) == set(node["pointers"]) and set(entry["i32_scalars"]) == set(node["scalars"])
    layer.close()
