"""Committed golden fixtures (tests/golden/): the reference contracts' capacity scalars, and the smallest configuration's
inputs with every tap of the layer as the CPU oracle computes it.  CPU tests hold the oracle, the seeded generator and the
capacity formula to the fixtures; the GPU test holds the HIP path (through the C ABI) to them."""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import CONFIGS, GpuLayer, assert_output_tolerance, bf16_ulp_distance, geometry, oracle_layer, pkg, synth

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
NAMES = ["gate_w", "bias", "bias_alt", "w13", "s13", "w2", "s2", "sh_w13", "sh_s13", "sh_w2", "sh_s2"]
EXACT = ["logits", "ids", "weights", "xq", "xs", "xq_min", "xs_min", "h", "hq", "hs", "route_out", "shared_up", "shared_act",
         "shared_aq", "shared_as", "shared_down", "routed", "out"]


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.float32 else a


def load(mode):
    f = np.load(os.path.join(GOLDEN, "c1_%s.npz" % mode), allow_pickle=False)
    c = CONFIGS["c1"]
    g = geometry(c["hidden"], c["experts"], c["topk"], c["inter"], c["shared"], mode)
    ops = synth.LayerOperands(g, "c1", device="cpu")
    return f, g, ops, torch.from_numpy(f["x"].view(np.int16).copy())      # BF16 bits, as synth.activations returns them


def test_capacity_formula_reproduces_every_reference_contract():
    # runtime/kernels/moe-runtime-*/runtime-contract.json; src/moe.rs:1253-1257 checks these scalars at load time
    rows = json.load(open(os.path.join(GOLDEN, "reference_contract_capacities.json")))
    assert len(rows) >= 20
    for r in rows:
        tile_m = r["rows_padded"] // r["max_phys_tiles"]
        assert tile_m in (16, 64) and tile_m * r["max_phys_tiles"] == r["rows_padded"], r
        pairs = r["num_tokens"] * r["topk"]
        assert pkg.contracts.max_phys_tiles(pairs, tile_m, r["experts"]) == r["max_phys_tiles"], r
        assert r["max_tasks"] == 5 * r["max_phys_tiles"], r      # five N-groups of FC1 (src/moe.rs:1261)


@pytest.mark.parametrize("mode", ["benchmark", "reference"])
def test_oracle_and_generator_reproduce_the_c1_fixture(mode):
    f, g, ops, x = load(mode)
    digests = json.loads(str(f["weight_digests"]))
    for n in NAMES:
        t = getattr(ops, n).contiguous()
        assert hashlib.sha256(t.view(-1).view(dtype=torch.uint8).numpy().tobytes()).hexdigest() == digests[n], n
    taps = oracle_layer(g, ops, x, f["tokens"], int(f["live"]), f["padding"])
    for n in EXACT:
        assert np.array_equal(bits(taps[n]), bits(f[n])), n
    base, te, tv, tmap, tw = oracle.plan(taps["ids"], taps["weights"], g.experts, 1, 16)
    for got, n in [(base, "tile_base"), (te, "task_expert"), (tv, "task_valid"), (tmap, "token_map"), (tw, "token_weights")]:
        assert np.array_equal(bits(got), bits(f[n])), n
    # what the fixture must show: row 7 is not live, row 6 repeats row 2's experts with zero weights
    assert (f["ids"][7] == -1).all() and np.array_equal(f["ids"][6], f["ids"][2]) and not f["weights"][6].any()
    assert not f["routed"][7].any()


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["benchmark", "reference"])
def test_gpu_layer_matches_the_c1_fixture(mode):
    f, g, ops, x = load(mode)
    layer = GpuLayer(g, ops, CONFIGS["c1"]["rows"])
    taps = layer.run(x, tokens=f["tokens"].tolist(), live=int(f["live"]), padding=f["padding"].tolist())
    # integer / index / code work: bit-exact
    for n in ["logits", "ids", "weights", "xq", "xs", "xq_min", "xs_min", "tile_base"]:
        assert np.array_equal(bits(taps[n]), bits(f[n])), n
    tiles = int(f["tile_base"][-1])
    assert np.array_equal(taps["task_expert"][:tiles], f["task_expert"][:tiles])
    assert np.array_equal(taps["task_valid"][:tiles], f["task_valid"][:tiles])
    occupied = f["token_map"] >= 0
    n = len(taps["token_map"])
    assert not occupied[n:].any()
    assert np.array_equal(taps["token_map"][occupied[:n]], f["token_map"][:n][occupied[:n]])
    assert np.array_equal(bits(taps["token_weights"])[occupied[:n]], bits(f["token_weights"])[:n][occupied[:n]])
    # floating point downstream of a matrix-core accumulation: the intermediate within its BF16 boundary's rounding, the
    # layer output within max |got - want| / max |want| <= 2e-2 (32- or 128-wide requantization blocks over I = 512: one
    # scale-byte flip between two valid accumulation orders moves an output by more than 1 %) and mean |got - want| <= 1e-3
    phys = np.nonzero(occupied[:n])[0]
    K, I = g.topk, g.intermediate
    assert bf16_ulp_distance(taps["h"][phys], f["h"].reshape(-1, I)[f["token_map"][phys]]) <= 2.0
    assert_output_tolerance("layer output against the fixture", taps["out"], f["out"], max_rel=2e-2, mean_abs=1e-3)
    assert not taps["out"][7].any() or np.array_equal(taps["out"][7], taps["shared_down"][7])   # row 7: no routed part
    layer.close()
