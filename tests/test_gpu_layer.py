"""GPU parity of the few-row (decode / speculative verify) path through the C ABI against the CPU oracle.

Bit-exact: gate logits (few-row kernel), routing ids and order, routing weights, plan tables and permutation maps, MXFP8
codes and scales of the token rows (both quantizer flavours), requantization codes of the intermediate and shared
activation given the activation the GPU itself produced.  Tolerance (stated per check): everything downstream of a
matrix-core accumulation, whose order the oracle cannot reproduce.
Output tolerance of the layer: max |got - want| / max |want| <= 1e-2 and mean |got - want| <= 1e-3.
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import (CONFIGS, GpuLayer, assert_output_tolerance, bf, bf16_ulp_distance, error_stats, geometry, native, np_of, oracle_fc2_from, oracle_layer,
                     synth, u16)

pytestmark = pytest.mark.gpu

MAX_REL, MEAN_ABS = 1e-2, 1e-3


def make(config, mode, device, rows=None, seed_name=None):
    c = CONFIGS[config]
    g = geometry(c["hidden"], c["experts"], c["topk"], c["inter"], c["shared"], mode)
    ops = synth.LayerOperands(g, seed_name or config, device=device)
    rows = rows or c["rows"]
    x = synth.activations(seed_name or config, rows, g.hidden, device=device)
    return g, ops, x, rows


def check_layer(g, ops, x, taps, tokens=None, live=None, padding=None, exact_logits=True, max_rel=MAX_REL):
    rows = x.shape[0]
    K, I, B = g.topk, g.intermediate, g.act_block
    want = oracle_layer(g, ops, x, tokens, live, padding)
    if exact_logits:
        assert np.array_equal(taps["logits"].view(np.uint32), want["logits"].view(np.uint32)), "gate logits differ"
    else:   # matrix-core gate product: another summation order, FP32 throughout
        live_rows = rows if live is None else live
        assert np.allclose(taps["logits"][:live_rows], want["logits"][:live_rows], rtol=1e-4, atol=2e-4), "gate logits differ beyond FP32 reordering"
    # routing from the GPU's own logits must equal the oracle's routing of those logits, bit for bit
    again = oracle_layer(g, ops, x, tokens, live, padding, logits=taps["logits"]) if not exact_logits else want
    assert np.array_equal(taps["ids"], again["ids"]), "routing ids / order differ"
    assert np.array_equal(taps["weights"].view(np.uint32), again["weights"].view(np.uint32)), "routing weights differ"
    for name in ["xq", "xs", "xq_min", "xs_min"]:
        assert np.array_equal(taps[name], want[name]), name
    tile_m = 16 if rows <= 64 else 128
    base, te, tv, tmap, tw = oracle.plan(again["ids"], again["weights"], g.experts, 1, tile_m, capacity_tiles=len(taps["task_expert"]))
    tiles = int(base[-1])
    assert np.array_equal(taps["tile_base"], base)
    assert np.array_equal(taps["task_expert"][:tiles], te[:tiles]) and np.array_equal(taps["task_valid"][:tiles], tv[:tiles])
    occupied = tmap >= 0
    assert np.array_equal(taps["token_map"][occupied], tmap[occupied]), "permutation map differs"
    assert np.array_equal(taps["token_weights"][occupied].view(np.uint32), tw[occupied].view(np.uint32))
    # intermediate: tolerance (matrix-core accumulation), in physical-row order -> route order
    phys = np.nonzero(occupied)[0]
    route = tmap[phys]
    h_gpu = taps["h"][phys]
    h_want = again["h"].reshape(rows * K, I)[route]
    assert bf16_ulp_distance(h_gpu, h_want) <= 2.0, "FC1 + SwiGLU differs by more than the rounding of its BF16 boundary"
    # requantization codes: bit-exact for the activation the GPU produced
    hq, hs = oracle.quantize_rows(h_gpu, B, 0.0)
    assert np.array_equal(taps["hq"][phys], hq) and np.array_equal(taps["hs"][phys], hs), "intermediate FP8 codes differ"
    # FC2 given the codes the GPU itself consumed: only the accumulation order and one BF16 rounding may differ
    live_routes = again["ids"].ravel() >= 0
    hq_routes = np.zeros((rows * K, I), np.uint8)
    hs_routes = np.zeros((rows * K, I // B), np.uint8)
    hq_routes[route], hs_routes[route] = taps["hq"][phys], taps["hs"][phys]
    fc2 = oracle_fc2_from(g, ops, again["ids"], again["weights"], hq_routes.reshape(rows, K, I), hs_routes.reshape(rows, K, -1))
    got_routes = taps["route_out"].reshape(rows * K, -1)[live_routes]
    assert bf16_ulp_distance(got_routes, fc2.reshape(rows * K, -1)[live_routes]) <= 2.0, "FC2 differs for the GPU's own codes"
    print("  route outputs vs independent oracle (max rel, mean abs):", error_stats(got_routes, again["route_out"].reshape(rows * K, -1)[live_routes]))
    # shared expert: same chain
    assert bf16_ulp_distance(taps["shared_up"], want["shared_up"]) <= 2.0, "shared up projection"
    act, aq, asc = oracle.shared_swiglu_quant(taps["shared_up"], B, g.swiglu_limit)
    assert np.array_equal(taps["shared_act"], act), "shared activation differs for the GPU's own projections"
    assert np.array_equal(taps["shared_aq"], aq) and np.array_equal(taps["shared_as"], asc), "shared FP8 codes differ"
    down = oracle.fp8_linear(taps["shared_aq"], taps["shared_as"], B, np_of(ops.sh_w2), np_of(ops.sh_s2), g.shared_bn, g.shared_bk)
    assert bf16_ulp_distance(taps["shared_down"], down) <= 2.0, "shared down differs for the GPU's own codes"
    print("  shared down vs independent oracle (max rel, mean abs):", error_stats(taps["shared_down"], want["shared_down"]))
    n_live = rows if live is None else min(live, rows)
    routed, out = oracle.ffn_sum_shared(taps["route_out"], taps["shared_down"], n_live)
    assert np.array_equal(taps["routed"][:n_live], routed[:n_live]) and np.array_equal(taps["out"], out), "combine differs"
    r = assert_output_tolerance("layer output", taps["out"], again["out"], max_rel=max_rel, mean_abs=MEAN_ABS)
    return r["max_rel"], r["mean_abs"]


@pytest.mark.parametrize("mode", ["benchmark", "reference"])
def test_c1_layer(mode):
    g, ops, x, rows = make("c1", mode, "cpu")
    layer = GpuLayer(g, ops, rows)
    taps = layer.run(x)
    # reference mode at this size (32-wide requantization blocks over I = 512): one scale-byte flip between two valid
    # accumulation orders moves an output by more than 1 % of the largest magnitude, so the end-to-end bound is 2e-2 there;
    # every stage is still held to its own bound given the GPU's upstream taps
    print("c1", mode, check_layer(g, ops, x, taps, max_rel=MAX_REL if mode == "benchmark" else 2e-2))
    layer.close()


def test_c1_reference_mode_live_padding_and_image_token():
    g, ops, x, rows = make("c1", "reference", "cpu")
    layer = GpuLayer(g, ops, rows)
    tokens = [5, 129264, 7, 129264, 1, 2, 3, 4]
    padding = [-1, -1, -1, -1, 0, 2, -1, -1]
    taps = layer.run(x, tokens=tokens, live=4, padding=padding)
    check_layer(g, ops, x, taps, tokens=tokens, live=4, padding=np.array(padding, np.int32), max_rel=2e-2)
    assert (taps["ids"][6:] == -1).all() and (taps["weights"][4:] == 0).all()
    assert np.array_equal(taps["ids"][4], taps["ids"][0]) and np.array_equal(taps["ids"][5], taps["ids"][2])
    layer.close()


def test_gate_product_inside_the_front_end():
    g, ops, x, rows = make("c1", "benchmark", "cpu")
    layer = GpuLayer(g, ops, rows)
    taps = layer.run(x, fuse_gate=True)
    check_layer(g, ops, x, taps)
    taps = layer.run(synth.activations("c1-third", rows, g.hidden), fuse_gate=True)      # the sync word was left at zero
    check_layer(g, ops, synth.activations("c1-third", rows, g.hidden), taps)
    layer.close()


def test_zero_input_gives_zero_output():
    # known answer recoverable from the reference (runtime/kernels/ffn-global-v1/index.json, case "zero": the output
    # digest is the digest of all-zero bytes)
    g, ops, x, rows = make("c1", "reference", "cpu")
    layer = GpuLayer(g, ops, rows)
    taps = layer.run(torch.zeros_like(x))
    assert not taps["out"].any() and not taps["route_out"].any() and not taps["shared_down"].any()
    layer.close()


def test_stale_scratch_between_runs():
    # the reference replays its graph to catch stale scratch (src/probe.rs:1527-1542): a second, different input through
    # the same buffers must give that input's own result
    g, ops, x, rows = make("c1", "benchmark", "cpu")
    layer = GpuLayer(g, ops, rows)
    layer.run(x)
    x2 = synth.activations("c1-second", rows, g.hidden)
    taps = layer.run(x2)
    check_layer(g, ops, x2, taps)
    layer.close()


@pytest.mark.parametrize("config,mode", [("c2", "benchmark"), ("c3", "benchmark"), ("c2", "reference")])
def test_full_size_few_rows(config, mode):
    g, ops, x, rows = make(config, mode, "cuda")
    if config == "c3":   # 4 requests x 8 draft tokens with correlated router inputs: x = base + 0.3 noise per token
        base = synth.normal("c3/base", (4, 1, g.hidden), device="cuda")
        noise = synth.normal("c3/noise", (4, 8, g.hidden), std=0.3, device="cuda")
        x = synth.to_bf16_bits((base + noise).reshape(32, g.hidden))
    layer = GpuLayer(g, ops, rows)
    taps = layer.run(x)
    distinct = len(set(taps["ids"].ravel().tolist()))
    print(config, mode, "distinct experts", distinct, check_layer(g, ops, x, taps))
    layer.close()
