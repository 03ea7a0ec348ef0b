"""Pins the CPU oracle: every function is checked against something other than its own formula -- the OCP format
definitions evaluated exhaustively, torch's independent BF16 / E4M3 conversions, libm, float64 dense algebra, brute
force, invariants, and the golden values the reference's own tests hold (src/config.rs:1381-1390 scale-code offsets;
runtime/kernels/ffn-global-v1/index.json zero case; runtime/kernels/shared-swiglu-quant-v1/manifest.json constants)."""
import hashlib
import math

import numpy as np
import pytest
import torch

import oracle
from helpers import bf, geometry, oracle_config, oracle_layer, synth, u16

L = oracle.lib()


# ---- formats --------------------------------------------------------------------------------------------------------
def e4m3_definition(code):
    s, e, m = code >> 7, (code >> 3) & 15, code & 7
    if e == 15 and m == 7:
        return math.nan
    v = m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
    return -v if s else v


def test_e4m3_decode_table_matches_ocp_definition_and_torch():
    codes = np.arange(256, dtype=np.uint8)
    ours = np.array([L.orc_e4m3_to_f32(int(c)) for c in codes])
    spec = np.array([e4m3_definition(int(c)) for c in codes])
    assert np.array_equal(np.isnan(ours), np.isnan(spec)) and np.array_equal(ours[~np.isnan(spec)], spec[~np.isnan(spec)])
    t = torch.from_numpy(codes).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(ours[~np.isnan(spec)], t[~np.isnan(spec)])
    assert max(abs(v) for v in spec if not math.isnan(v)) == 448.0


def test_e4m3_encode_is_nearest_even_saturating():
    grid = sorted(set(e4m3_definition(c) for c in range(127)))   # non-negative finite values
    rng = np.random.default_rng(0)
    samples = np.concatenate([rng.uniform(-470, 470, 20000), rng.normal(0, 1, 20000), rng.normal(0, 0.01, 20000),
                              np.array(grid), (np.array(grid[:-1]) + np.array(grid[1:])) / 2,        # exact ties
                              [1e-30, 2.0 ** -10, 2.0 ** -10 * 1.0001, 463.9, 464.0, 1e9, np.inf, -np.inf]]).astype(np.float32)
    for v in samples:
        code = L.orc_f32_to_e4m3(float(v))
        got = e4m3_definition(code & 0x7f)
        a = min(abs(float(v)), 448.0)
        best = min(abs(a - q) for q in grid)
        assert abs(a - got) == best, (v, code)
        lo = [q for q in grid if abs(a - q) == best]
        if len(lo) == 2:                                           # tie: the even code wins
            assert (code & 1) == 0, (v, code)
        if v != 0 and not np.isnan(v):
            assert (code >> 7) == (1 if v < 0 else 0)
    assert L.orc_f32_to_e4m3(float("nan")) == 0x7f
    inside = samples[np.abs(samples) < 464]
    t = torch.from_numpy(inside).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(t, np.array([L.orc_f32_to_e4m3(float(v)) for v in inside], np.uint8))


def test_bf16_matches_torch():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.normal(0, 1, 50000), rng.normal(0, 1e-20, 1000), rng.normal(0, 1e20, 1000)]).astype(np.float32)
    x = np.concatenate([x, np.array([1.00390625, 1.01171875, -1.00390625, 3.3895314e38, np.inf], np.float32)])   # ties and overflow
    t = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(np.array([L.orc_f32_to_bf16(float(v)) for v in x], np.uint16), t)
    assert np.array_equal(oracle.f32_to_bf16(x), t)
    back = torch.from_numpy(t.view(np.int16)).view(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(oracle.bf16_to_f32(t), back)


def test_e2m1_and_ue8m0_tables():
    values = [0, 0.5, 1, 1.5, 2, 3, 4, 6]
    for c in range(16):
        assert L.orc_e2m1_to_f32(c) == (-1 if c & 8 else 1) * values[c & 7]
    for v in np.concatenate([np.linspace(-7, 7, 2801), [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 100.0]]).astype(np.float32):
        code = L.orc_f32_to_e2m1(float(v))
        a = min(abs(float(v)), 6.0)
        best = min(abs(a - q) for q in values)
        assert abs(a - values[code & 7]) == best
        if len([q for q in values if abs(a - q) == best]) == 2:
            assert (code & 1) == 0            # even mantissa on ties
    assert L.orc_ue8m0_to_f32(127) == 1.0 and L.orc_ue8m0_to_f32(130) == 8.0 and L.orc_ue8m0_to_f32(1) == 2.0 ** -126
    assert L.orc_ue8m0_to_f32(0) == 2.0 ** -127 and math.isnan(L.orc_ue8m0_to_f32(255))


def test_exp_log1p_logistic_against_libm():
    xs = np.concatenate([np.linspace(-87, 88, 20001), np.linspace(-1, 1, 2001)]).astype(np.float32)
    for x in xs[::7]:
        got, want = L.orc_exp(float(x)), math.exp(float(x))
        assert abs(got - want) <= 2 * np.spacing(np.float32(want)), x
    for e in np.concatenate([np.logspace(-30, 8.6, 4000), [1.0, 0.5, 3.0]]).astype(np.float32):
        got, want = L.orc_log1p_pos(float(e)), math.log1p(float(e))
        assert abs(got - want) <= 2 * np.spacing(np.float32(want)), e
    for x in np.linspace(-30, 30, 601):
        assert abs(L.orc_logistic(float(x)) - 1 / (1 + math.exp(-x))) <= 2e-7
    assert L.orc_exp(-1000.0) > 0 and math.isfinite(L.orc_exp(1000.0))


# ---- synthetic weight quantizers -------------------------------------------------------------------------------------
def test_weight_quantizers_follow_ocp_mx_and_match_the_torch_generator():
    w = synth.normal("pin/w", (64, 256), std=0.02)
    packed, scales = oracle.quantize_mxfp4(w.numpy())
    # closed form: scale exponent = floor(log2(amax)) - 2; dequantized error bounded by half a grid step (or saturation)
    blocks = w.numpy().reshape(64, 8, 32)
    amax = np.abs(blocks).max(axis=2)
    assert np.array_equal(scales.astype(np.int32) - 127, np.floor(np.log2(amax)).astype(np.int32) - 2)
    lo, hi = packed & 15, packed >> 4
    codes = np.stack([lo, hi], axis=-1).reshape(64, 256)
    table = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6])
    deq = table[codes] * np.repeat(2.0 ** (scales.astype(np.float64) - 127), 32, axis=1)
    step = np.repeat(2.0 ** (scales.astype(np.float64) - 127), 32, axis=1)
    assert (np.abs(deq - w.numpy()) <= 2 * step + 1e-12).all()      # half of the widest grid step (1 unit) or saturation at 6 (below 2 units)
    p2, s2 = synth.quantize_mxfp4(w)
    assert np.array_equal(p2.numpy(), packed) and np.array_equal(s2.numpy(), scales)
    for bn, bk in [(32, 32), (64, 128)]:
        c, s = oracle.quantize_fp8_blocks(w.numpy(), bn, bk)
        c2, s2 = synth.quantize_fp8_blocks(w, bn, bk)
        assert np.array_equal(c2.numpy(), c) and np.array_equal(s2.numpy(), s)


# ---- router -----------------------------------------------------------------------------------------------------------
def test_router_logits_against_float64():
    x = synth.activations("pin/logits", 5, 1024)
    w = synth.to_bf16_bits(synth.normal("pin/logits/w", (24, 1024), std=1 / 32))
    got = oracle.router_logits(u16(x), u16(w))
    want = bf(u16(x)) @ bf(u16(w)).T
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max() + 1e-6
    # a transposed operand or a dropped lane would break a one-hot probe
    onehot = np.zeros((1, 1024), np.float32)
    onehot[0, 777] = 1.0
    got = oracle.router_logits(oracle.f32_to_bf16(onehot), u16(w))
    assert np.array_equal(got[0], bf(u16(w))[:, 777].astype(np.float32))


def brute_topk(scores, bias, k):
    biased = np.where(np.isnan(scores + bias), np.inf, (scores + bias).astype(np.float32))
    order = sorted(range(len(scores)), key=lambda e: (-biased[e], e))
    return order[:k]


@pytest.mark.parametrize("scoring,scale,experts,topk", [(1, 1.5, 384, 6), (0, 1.0, 256, 6), (0, 1.0, 16, 2), (1, 1.5, 128, 3)])
def test_route_topk_against_brute_force(scoring, scale, experts, topk):
    cfg = oracle.config(1024, experts, topk, 512, 512, scoring, scale, 32, 32, 32, 129264)
    rows = 24
    logits = synth.normal("pin/topk", (rows, experts), std=2.0).numpy()
    logits[1, :] = 0.5
    logits[2, 9] = 25.0
    bias = synth.normal("pin/topk/bias", (experts,), std=0.1).numpy()
    alt = synth.normal("pin/topk/alt", (experts,), std=0.1).numpy()
    tokens = np.arange(rows, dtype=np.int64)
    tokens[3] = 129264
    ids, weights = oracle.route_topk(cfg, logits, bias, alt, tokens, live=20)
    for r in range(rows):
        if r >= 20:
            assert (ids[r] == -1).all() and (weights[r] == 0).all()
            continue
        x = logits[r].astype(np.float64)
        s = np.sqrt(np.where(x > 20, x, np.log1p(np.exp(x)))) if scoring == 1 else 1 / (1 + np.exp(-x))
        mine = np.array([math.sqrt(v) if scoring == 1 and v > 20 else (math.sqrt(L.orc_log1p_pos(L.orc_exp(float(v)))) if scoring == 1 else L.orc_logistic(float(v)))
                         for v in logits[r]], np.float32)
        assert np.abs(mine - s).max() <= 4e-7 * max(1.0, s.max())
        want = brute_topk(mine, alt if r == 3 else bias, topk)
        assert list(ids[r]) == want, r
        assert len(set(ids[r])) == topk
        total = mine[want].astype(np.float64).sum()
        assert np.allclose(weights[r], mine[want] / total * scale, rtol=3e-7)
        assert abs(weights[r].sum() - scale) < 1e-5
    tied, _ = oracle.route_topk(cfg, np.full((1, experts), 0.5, np.float32), np.zeros(experts, np.float32))
    assert list(tied[0]) == list(range(topk))         # all-equal scores: lowest ids first


def test_padding_rows_and_census():
    ids = np.array([[3, 1], [2, 0], [5, 5], [7, 7]], np.int32)
    w = np.full((4, 2), 0.5, np.float32)
    i2, w2 = oracle.route_padding_rows(ids, w, np.array([-1, -1, 0, 1], np.int32))
    assert i2.tolist() == [[3, 1], [2, 0], [3, 1], [2, 0]] and w2.tolist() == [[.5, .5], [.5, .5], [0, 0], [0, 0]]
    assert oracle.route_census(np.array([[0, 1], [1, 9], [1, 1]], np.int32), 2, 4).tolist() == [1, 2, 0, 0]


# ---- plan -------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("tile_m,groups", [(16, 1), (16, 5), (4, 2), (128, 1)])
def test_plan_invariants_and_brute_force(tile_m, groups):
    rng = np.random.default_rng(tile_m)
    rows, topk, experts = 37, 6, 24
    ids = np.stack([rng.choice(experts, topk, replace=False) for _ in range(rows)]).astype(np.int32)
    ids[5, 2] = -1
    ids[6, 0] = experts + 3
    weights = rng.random((rows, topk), dtype=np.float32)
    base, te, tv, tmap, tw = oracle.plan(ids, weights, experts, groups, tile_m)
    flat = ids.ravel()
    counts = np.array([(flat == e).sum() for e in range(experts)])
    tiles = -(-counts // tile_m)
    assert np.array_equal(base, np.concatenate([[0], np.cumsum(tiles)]))            # monotone exclusive prefix
    active = [t for t, e in enumerate(flat) if 0 <= e < experts]
    occupied = np.nonzero(tmap >= 0)[0]
    assert sorted(tmap[occupied].tolist()) == active                                 # bijection onto the active routes
    for p in occupied:
        t = tmap[p]
        e = flat[t]
        rank = int((flat[:t] == e).sum())                                            # stable in route order
        assert p == (base[e] + rank // tile_m) * tile_m + rank % tile_m
        assert tw[p] == weights.ravel()[t]
    for e in range(experts):
        for k in range(tiles[e]):
            for gidx in range(groups):
                slot = (base[e] + k) * groups + gidx
                assert te[slot] == e and tv[slot] == min(tile_m, counts[e] - k * tile_m)


# ---- quantizers -------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("block", [32, 128])
def test_quantize_rows_closed_form(block):
    x = synth.normal("pin/quant", (9, 512), std=1.0)
    x[0] = 0
    x[1] *= 1e-7
    x[2, :block] = 448.0
    xb = synth.to_bf16_bits(x)
    vals = bf(u16(xb))
    for min_amax in (0.0, 1e-4):
        codes, scales = oracle.quantize_rows(u16(xb), block, min_amax)
        amax = np.maximum(np.abs(vals.reshape(9, -1, block)).max(axis=2), min_amax)
        want = np.where(amax > 0, np.ceil(np.log2(np.maximum(amax, 1e-300) / 448.0)) + 127, 0).clip(0, 254)
        exact_pow2 = amax > 0
        assert np.array_equal(scales[exact_pow2].astype(np.int64), want[exact_pow2].astype(np.int64))
        if min_amax == 0.0:
            assert (scales[0] == 0).all() and (codes[0] == 0).all()                  # zero block: scale byte 0, zero payload
        else:
            assert (scales >= 105).all()                                             # 1e-4 floor: smallest shared code is 105
        inv = np.where(scales > 0, 2.0 ** (127 - scales.astype(np.float64)), 0.0)
        scaled = (vals.reshape(9, -1, block) * inv[:, :, None]).reshape(9, 512).astype(np.float32)
        assert np.abs(scaled).max() <= 448.0
        t = torch.from_numpy(scaled).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(codes, t)


def test_shared_swiglu_against_float64_and_constants():
    x = synth.normal("pin/swiglu", (7, 1152), std=4.0)     # 1152 -> 576 as in the reference's manifest
    x[0, :4] = torch.tensor([20.0, -20.0, 10.0, 0.0])
    x[0, 576:580] = torch.tensor([20.0, -20.0, -10.0, 5.0])
    xb = u16(synth.to_bf16_bits(x))
    act = oracle.shared_swiglu(xb)
    g = np.minimum(bf(xb[:, :576]), 10.0)
    u = np.clip(bf(xb[:, 576:]), -10.0, 10.0)
    want = g / (1 + np.exp(-g)) * u
    got = bf(act)
    ulp = np.maximum(np.abs(want), 2.0 ** -126) * 2.0 ** -8
    assert (np.abs(got - want) <= ulp).all()
    assert got[0, 0] == pytest.approx(100.0, rel=1e-2) and got[0, 1] == pytest.approx(0.0, abs=1e-6)
    a2, codes, scales = oracle.shared_swiglu_quant(xb, 32)
    assert np.array_equal(a2, act)
    wq, ws = oracle.quantize_rows(act, 32, 1e-4)
    assert np.array_equal(codes, wq) and np.array_equal(scales, ws)


# ---- projections --------------------------------------------------------------------------------------------------------
def dequant_fp4(packed, scales):
    table = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6])
    codes = np.stack([packed & 15, packed >> 4], axis=-1).reshape(packed.shape[0], -1)
    return table[codes] * np.repeat(2.0 ** (scales.astype(np.float64) - 127), 32, axis=1)


def dequant_fp8(codes, scales, bn, bk):
    vals = np.array([e4m3_definition(c) for c in range(256)])[codes]
    return vals * np.kron(2.0 ** (scales.astype(np.float64) - 127), np.ones((bn, bk)))


@pytest.mark.parametrize("block", [32, 128])
def test_expert_projections_against_float64(block):
    H, I, E, K, rows = 512, 256, 3, 2, 4
    cfg = oracle.config(H, E, K, I, I, 0, 1.0, block, 32, 32)
    x = u16(synth.activations("pin/fc", rows, H))
    xq, xs = oracle.quantize_rows(x, block)
    w13 = [oracle.quantize_mxfp4(synth.normal("pin/fc/w13.%d" % e, (2 * I, H), std=0.05).numpy()) for e in range(E)]
    w2 = [oracle.quantize_mxfp4(synth.normal("pin/fc/w2.%d" % e, (H, I), std=0.05).numpy()) for e in range(E)]
    ids = np.array([[0, 2], [1, 0], [2, -1], [1, 2]], np.int32)
    weights = np.array([[.6, .4], [.5, .5], [1, 0], [.3, .7]], np.float32)
    h, proj = oracle.expert_fc1(cfg, xq, xs, np.stack([w[0] for w in w13]), np.stack([w[1] for w in w13]), ids, want_proj=True)
    xd = dequant_fp8(xq, xs, 1, block)
    for r in range(rows):
        for k in range(K):
            e = ids[r, k]
            if e < 0:
                assert not h[r, k].any()
                continue
            want = dequant_fp4(*w13[e]) @ xd[r]
            assert np.abs(proj[r, k] - want).max() <= 2e-6 * np.abs(want).max() + 1e-7
            up, gate = want[:I], np.minimum(want[I:], 10.0)          # up rows first, then gate rows
            hw = gate / (1 + np.exp(-gate)) * np.clip(up, -10, 10)
            assert (np.abs(bf(h[r, k]) - hw) <= np.maximum(np.abs(hw), 1e-30) * 2.0 ** -7 + 1e-9).all()
    hq, hs = oracle.quantize_rows(h.reshape(rows * K, I), block)
    out = oracle.expert_fc2(cfg, hq.reshape(rows, K, I), hs.reshape(rows, K, -1), np.stack([w[0] for w in w2]),
                            np.stack([w[1] for w in w2]), ids, weights)
    hd = dequant_fp8(hq, hs, 1, block).reshape(rows, K, I)
    for r in range(rows):
        for k in range(K):
            e = ids[r, k]
            want = (dequant_fp4(*w2[e]) @ hd[r, k]) * weights[r, k] if e >= 0 else np.zeros(H)
            assert (np.abs(bf(out[r, k]) - want) <= np.abs(want) * 2.0 ** -7 + 1e-7 * (np.abs(want).max() + 1e-30)).all()


def test_fp8_linear_against_float64():
    rows, n, k = 3, 128, 512
    a = u16(synth.activations("pin/dense", rows, k))
    aq, as_ = oracle.quantize_rows(a, 32, 1e-4)
    w = synth.normal("pin/dense/w", (n, k), std=0.05).numpy()
    for bn, bk in [(32, 32), (128, 128)]:
        wq, ws = oracle.quantize_fp8_blocks(w, bn, bk)
        got = bf(oracle.fp8_linear(aq, as_, 32, wq, ws, bn, bk))
        want = dequant_fp8(aq, as_, 1, 32) @ dequant_fp8(wq, ws, bn, bk).T
        assert (np.abs(got - want) <= np.abs(want) * 2.0 ** -7 + 2e-6 * np.abs(want).max()).all()


# ---- combine ------------------------------------------------------------------------------------------------------------
def test_sum_order_and_flush_to_zero_add():
    # (a + b) + c differs from a + (b + c) in FP32: the sum must run in slot order from zero
    a, b, c = np.float32(1.0), np.float32(2.0 ** -24), np.float32(2.0 ** -24)
    routes = oracle.f32_to_bf16(np.array([[[a], [b], [c]]], np.float32))
    left = np.float32(np.float32(np.float32(0) + a) + b) + c
    assert bf(oracle.topk_sum(routes))[0, 0] == float(oracle.bf16_to_f32(oracle.f32_to_bf16(np.array([left])))[0])
    routes = oracle.f32_to_bf16(np.array([[[256.0], [1.0], [1.0]], [[1.0], [1.0], [256.0]]], np.float32))
    assert bf(oracle.topk_sum(routes))[:, 0].tolist() == [258.0, 258.0]
    prev = np.full((2, 1), 0x4000, np.uint16)
    kept = oracle.topk_sum(routes, live=1, previous=prev)
    assert kept[1, 0] == 0x4000 and bf(kept)[0, 0] == 258.0                          # rows past live keep their value
    tiny = np.array([0x0001, 0x8001, 0x0080], np.uint16)                             # two denormals and the smallest normal
    assert oracle.ffn_add(tiny, np.array([0x0001, 0x0001, 0x8080], np.uint16)).tolist() == [0, 0x8000 if False else 0, 0]
    x = oracle.f32_to_bf16(np.array([1.5, -2.25, 3.0], np.float32))
    y = oracle.f32_to_bf16(np.array([0.25, 2.25, 1e-3], np.float32))
    assert np.array_equal(oracle.ffn_add(x, y), oracle.f32_to_bf16(bf(x).astype(np.float32) + bf(y).astype(np.float32)))


# ---- layouts and codes -----------------------------------------------------------------------------------------------
def test_scale_code1_offsets_match_the_reference_test():
    f13, b13, c2, f2, b2, words = oracle.scale_code1_layout(384, 5120, 576)          # src/config.rs:1381-1390
    assert (f13, b13) == (384 * 2 * 200 * 16, 384 * 2 * 200 * 20)
    assert c2 == 384 * 2 * 200 * 20 + 768
    assert (f2, b2) == (c2 + 384 * 200 * 16, c2 + 384 * 200 * 20)
    assert words * 4 == 384 * 48_012
    assert oracle.scale_code1_layout(3, 5120, 576)[2] == 3 * 2 * 200 * 20 + 8


def test_scale_code1_round_trip_and_decode_formula():
    rng = np.random.default_rng(5)
    for n, columns in [(256, 32), (576, 160), (64, 6)]:                              # incl. the reference's 576 x 160 and tails
        matrices = 2
        scales = rng.choice(np.array([119, 119, 119, 120, 120, 118, 131], np.uint8), (matrices, n * columns))
        code, flags, bases = oracle.scale_code1(scales, matrices, n, columns)
        err, raw = oracle.scale_code1_check(scales, code, flags, bases, matrices, n, columns)
        assert err == 0 and raw > 0
        assert (bases == 119 * 0x01010101).all()
        for nib in range(16):                                                         # the decode multiply spreads 4 bits over 4 bytes
            spread = (nib * 0x00204081) & 0x01010101
            assert [(spread >> (8 * j)) & 1 for j in range(4)] == [(nib >> j) & 1 for j in range(4)]
        broken = code.copy()
        first = int(np.nonzero(code)[0][0])
        broken[first] ^= 1 << (4 * int((code[first] & -code[first]).bit_length() - 1) // 4 * 4 // 4) if False else 1
        # flipping a code bit of an unflagged row must be caught by the check
        err2, _ = oracle.scale_code1_check(scales, broken, np.zeros_like(flags), bases, matrices, n, columns)
        assert err2 & 1


def test_scale_codes4_round_trip_and_fail_closed():
    rng = np.random.default_rng(6)
    m, n, columns = 2, 256, 32
    scales = rng.integers(110, 124, (m, n, columns)).astype(np.uint8)
    coded, err = oracle.scale_codes4(scales, m, n, columns)
    assert err == 0 and coded[0] == 4 and np.array_equal(coded[16:16 + n], scales[0].min(axis=1))
    assert np.array_equal(oracle.scale_codes4_decode(coded, m, n, columns).reshape(scales.shape), scales)
    wide = scales.copy()
    wide[1, 7, 3] = 90
    assert oracle.scale_codes4(wide, m, n, columns)[1] == 1
    big = scales.copy()
    big[0, 0, 0] = 250
    assert oracle.scale_codes4(big, m, n, columns)[1] == 1


def test_nibble_permute_definition_and_inverse():
    x = np.array([0x76543210, 0xfedcba98], np.uint32)
    y = oracle.nibble_permute(x)
    assert [(int(y[0]) >> (4 * j)) & 15 for j in range(8)] == [0, 4, 1, 5, 2, 6, 3, 7]       # kernels/moe_nibble_layout_probe.cu:9-12
    assert int(y[0]) & 0x0f0f0f0f == 0x03020100 and (int(y[0]) >> 4) & 0x0f0f0f0f == 0x07060504
    assert np.array_equal(oracle.nibble_permute(y, inverse=True), x)


def test_stream_layouts_match_the_matrix_instruction_lane_model():
    n, k = 32, 1024
    words = np.arange(n * k // 2, dtype=np.uint32).astype(np.uint8).reshape(n, k // 2) ^ np.arange(n, dtype=np.uint8)[:, None]
    scales = (np.arange(n * k // 32) % 251).astype(np.uint8).reshape(n, k // 32)
    fp8 = (np.arange(n * k) % 253).astype(np.uint8).reshape(n, k)
    sw, ss, s8 = oracle.stream_words(words, n, k), oracle.stream_scales(scales, n, k), oracle.stream_fp8(fp8, n, k)
    sw, ss, s8 = sw.ravel(), ss.ravel(), s8.ravel()
    for nt in range(n // 16):
        for ks in range(k // 128):
            for lane in range(64):
                r, g = nt * 16 + lane % 16, lane // 16
                at = ((nt * (k // 128) + ks) * 64 + lane) * 16
                assert np.array_equal(sw[at:at + 16], words[r, (ks * 128 + 32 * g) // 2:(ks * 128 + 32 * g) // 2 + 16])   # nibbles k = 128 ks + 32 g ..
                assert ss[((nt * (k // 512) + ks // 4) * 64 + lane) * 4 + ks % 4] == scales[r, ks * 4 + g]
                for half in range(2):
                    at8 = (((nt * (k // 128) + ks) * 2 + half) * 64 + lane) * 16
                    lo = ks * 128 + 64 * half + 16 * g
                    assert np.array_equal(s8[at8:at8 + 16], fp8[r, lo:lo + 16])
    assert np.array_equal(oracle.stream_words(sw, n, k, inverse=True).reshape(words.shape), words)
    assert np.array_equal(oracle.stream_scales(ss, n, k, inverse=True).reshape(scales.shape), scales)
    assert np.array_equal(oracle.stream_fp8(s8, n, k, inverse=True).reshape(fp8.shape), fp8)


# ---- whole layer ---------------------------------------------------------------------------------------------------------
def test_zero_input_zero_output_digest_of_the_reference_fixture():
    # runtime/kernels/ffn-global-v1/index.json, case "zero": input and output digests are both the digest of 61,440
    # zero bytes (6 rows x 5120 BF16); with the reference's hidden size and a reduced expert count the oracle reproduces it
    g = geometry(5120, 8, 6, 512, 512, "reference")
    ops = synth.LayerOperands(g, "pin/zero", weight_std=0.02)
    x = torch.zeros((6, 5120), dtype=torch.int16)
    out = oracle_layer(g, ops, x)["out"]
    assert hashlib.sha256(out.tobytes()).hexdigest() == "0693f6bf" + hashlib.sha256(bytes(61440)).hexdigest()[8:]
    assert hashlib.sha256(bytes(61440)).hexdigest().startswith("0693f6bf")


def test_layer_c_function_agrees_with_staged_evaluation_and_float64():
    g = geometry(512, 8, 2, 512, 512, "reference")
    ops = synth.LayerOperands(g, "pin/layer")
    x = synth.activations("pin/layer", 5, 512)
    tokens = np.array([1, 129264, 3, 4, 5], np.int64)
    staged = oracle_layer(g, ops, x, tokens=tokens, live=4)
    whole = oracle.layer(oracle_config(g), u16(x), tokens, 4, u16(ops.gate_w), ops.bias.numpy(), ops.bias_alt.numpy(), ops.w13.numpy(),
                         ops.s13.numpy(), ops.w2.numpy(), ops.s2.numpy(), ops.sh_w13.numpy(), ops.sh_s13.numpy(), ops.sh_w2.numpy(),
                         ops.sh_s2.numpy())
    for name in ["ids", "weights", "h", "hq", "route_out", "shared_up", "shared_act", "shared_down", "routed", "out"]:
        assert np.array_equal(np.asarray(staged[name]).ravel(), np.asarray(whole[name]).ravel()), name
    # float64 evaluation of the same layer from the dequantized operands, with exact (unquantized) intermediates kept
    # in float64: agreement within the quantization noise of the FP8 activations pins signs, operand order and the
    # up / gate row order end to end
    xd = bf(u16(x))
    ids, wts = staged["ids"], staged["weights"]
    ref = np.zeros((5, 512))
    for r in range(4):
        for k in range(2):
            e = ids[r, k]
            w13 = dequant_fp4(ops.w13[e].numpy(), ops.s13[e].numpy())
            w2 = dequant_fp4(ops.w2[e].numpy(), ops.s2[e].numpy())
            p = w13 @ xd[r]
            gate = np.minimum(p[512:], 10)
            hcol = gate / (1 + np.exp(-gate)) * np.clip(p[:512], -10, 10)
            ref[r] += (w2 @ hcol) * wts[r, k]
    s13 = dequant_fp8(ops.sh_w13.numpy(), ops.sh_s13.numpy(), 32, 32)
    s2 = dequant_fp8(ops.sh_w2.numpy(), ops.sh_s2.numpy(), 32, 32)
    for r in range(5):
        p = s13 @ xd[r]
        gate = np.minimum(p[:512], 10)                                               # shared: gate rows first
        ref[r] += s2 @ (gate / (1 + np.exp(-gate)) * np.clip(p[512:], -10, 10))
    got = bf(staged["out"])
    assert np.abs(got - ref).max() <= 0.06 * np.abs(ref).max()
    assert np.corrcoef(got.ravel(), ref.ravel())[0, 1] > 0.995    # FP8 activation noise; a swapped gate / up order or operand gives < 0.9


@pytest.mark.skipif(not oracle.simd_available(), reason="the vectorised oracle loops need AVX2 + FMA")
@pytest.mark.parametrize("mode", ["benchmark", "reference"])
def test_vectorised_projection_loops_against_the_scalar_oracle(mode):
    # the CPU baseline's build of the three projection loops: the same operands and roundings, a block's 32 products summed in
    # eight lanes instead of one chain.  Against the scalar oracle: every BF16 output within one BF16 step (almost all equal),
    # and against float64 on the dequantized operands as close as the scalar oracle is
    import helpers
    g = helpers.geometry(1024, 16, 2, 512, 512, mode)
    ops = helpers.synth.LayerOperands(g, "simd-" + mode, device="cpu")
    x = helpers.synth.activations("simd-" + mode, 12, g.hidden)
    scalar = helpers.oracle_layer(g, ops, x)
    fast = helpers.oracle_layer(g, ops, x, ids_weights=(scalar["ids"], scalar["weights"]), simd=True)
    for name in ["h", "shared_up", "shared_down"]:
        assert helpers.bf16_ulp_distance(fast[name], scalar[name]) <= 1.0, name
        assert np.mean(fast[name] != scalar[name]) < 0.01, name
    # downstream of a BF16 value that moved one step the FP8 codes of its block may move too; given the same codes FC2 agrees
    cfg = helpers.oracle_config(g)
    again = oracle.expert_fc2(cfg, scalar["hq"], scalar["hs"], helpers.np_of(ops.w2), helpers.np_of(ops.s2), scalar["ids"], scalar["weights"], simd=True)
    assert helpers.bf16_ulp_distance(again, scalar["route_out"]) <= 1.0 and np.mean(again != scalar["route_out"]) < 0.01
    r = helpers.error_stats(fast["out"], scalar["out"])
    assert r[0] <= 1e-2 and r[1] <= 1e-3
    # special values of the bit-arithmetic E4M3 decode: every code against the table decode, through a one-hot product
    codes = np.arange(256, dtype=np.uint8)
    k = 512
    wq = np.zeros((256, k), np.uint8)
    wq[np.arange(256), 7] = codes                                  # weight row j holds code j at column 7
    aq = np.zeros((1, k), np.uint8)
    aq[0, 7] = 0x38                                                # 1.0
    ones = np.full((1, k // 32), 127, np.uint8)
    ws = np.full((256 // 32, k // 32), 127, np.uint8)
    a = oracle.fp8_linear(aq, ones, 32, wq, ws, 32, 32)
    b = oracle.fp8_linear(aq, ones, 32, wq, ws, 32, 32, simd=True)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("mode", ["benchmark", "reference"])
def test_layer_against_float64_on_the_same_quantized_operands(mode):
    # the whole layer with every dot product in float64 (torch's matrix products on exactly dequantized operands) and every
    # requantization point kept: the oracle's FP32 chains agree with it to the BF16 boundaries
    import helpers
    g = helpers.geometry(1024, 16, 2, 512, 512, mode)
    ops = helpers.synth.LayerOperands(g, "c1", device="cpu")
    x = helpers.synth.activations("c1", 8, g.hidden)
    want = helpers.oracle_layer(g, ops, x)
    exact = helpers.exact_layer(g, ops, x, want["ids"], want["weights"])
    for name in ["h", "route_out", "shared_up", "shared_down", "out"]:
        assert helpers.bf16_ulp_distance(want[name], exact[name], accumulation=0.0) <= 1.0, name
        assert np.mean(want[name] != exact[name]) <= 1e-3, name
    assert np.array_equal(want["hq"], exact["hq"]) or np.mean(want["hq"] != exact["hq"]) <= 1e-4
    # a transposed operand, a dropped scale or the wrong half of the up / gate rows would move every value: the float64
    # evaluation with up and gate swapped is far from the oracle
    swapped = type("Ops", (), {})()
    for k, v in vars(ops).items():
        setattr(swapped, k, v)
    I = g.intermediate
    swapped.w13 = torch.cat([ops.w13[:, I:], ops.w13[:, :I]], dim=1)
    swapped.s13 = torch.cat([ops.s13[:, I:], ops.s13[:, :I]], dim=1)
    other = helpers.exact_layer(g, swapped, x, want["ids"], want["weights"])
    assert np.mean(other["h"] != want["h"]) > 0.9
