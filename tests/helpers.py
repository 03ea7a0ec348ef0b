"""Shared test harness: benchmark configs, a python driver of the C ABI in the reference's call order
(src/ffn.rs:974-1047), and the stage-by-stage oracle evaluation it is compared with."""
import ctypes
import importlib
import math

import numpy as np
import torch

import oracle

pkg = importlib.import_module("titanic-flash-41_amd")
native = pkg.native
synth = pkg.synth
Geometry = native.Geometry

STREAM_MAX_ROWS = 64
GEMM_TILE_M = 128


def geometry(hidden, experts, topk, inter, shared, mode="benchmark"):
    """mode "benchmark": the benchmark configs' numerics (sigmoid, renormalised, scale 1, 128-wide activation blocks, 128 x 128
    shared weight blocks).  mode "reference": the reference's (sqrt-softplus, x 1.5, 32-wide blocks, 32 x 32, image-token bias)."""
    if mode == "benchmark":
        return Geometry(hidden, experts, topk, inter, shared, 0, 1.0, 128, 128, 128, -1, 10.0)
    return Geometry(hidden, experts, topk, inter, shared, 1, 1.5, 32, 32, 32, 129264, 10.0)


def oracle_config(g):
    return oracle.config(g.hidden, g.experts, g.topk, g.intermediate, g.shared_intermediate, g.scoring, g.route_scale,
                         g.act_block, g.shared_bn, g.shared_bk, g.alt_token, g.swiglu_limit)


CONFIGS = {
    "c1": dict(rows=8, hidden=1024, experts=16, topk=2, inter=512, shared=512),
    "c2": dict(rows=4, hidden=4096, experts=256, topk=6, inter=2048, shared=2048),
    "c3": dict(rows=32, hidden=4096, experts=256, topk=6, inter=2048, shared=2048),
    "c4": dict(rows=4096, hidden=4096, experts=256, topk=6, inter=2048, shared=2048),
    "c5": dict(rows=16384, hidden=4096, experts=256, topk=6, inter=2048, shared=2048),
}


def np_of(t):
    return t.detach().cpu().numpy()


def u16(t):
    return np_of(t).view(np.uint16)


def configure(g):
    lib = native.load()
    status = lib.ca_ffn_configure(ctypes.byref(g))
    assert status == 0, status
    st = ctypes.c_int32(0)
    ctx = lib.ca_primitives_open(ctypes.byref(st))
    assert st.value == 0 and ctx, st.value
    return ctx


class GpuLayer:
    """Drives the C ABI the way LayerFfn::run_quantized_input does (src/ffn.rs:974-1047): gate product, front-end with the
    router's top-k inside (few rows) or top-k kernel + wide plan (many rows), routed experts, shared expert, fused sum."""

    def __init__(self, g, ops, rows, device="cuda"):
        self.g, self.rows, self.dev = g, rows, device
        self.lib = native.load()
        self.ctx = configure(g)
        H, E, K, I, S, B = g.hidden, g.experts, g.topk, g.intermediate, g.shared_intermediate, g.act_block
        d = device
        self.gate_w, self.bias, self.bias_alt = ops.gate_w.to(d), ops.bias.to(d), ops.bias_alt.to(d)
        # load-time preparation (expert_packing::prepare_layer): canonical bytes -> streaming layouts, on the GPU
        self.w13 = self._compact(ops.w13.to(d), "ca_expert_compact_words", E * 2 * I, H, 16, 32)
        self.s13 = self._compact(ops.s13.to(d), "ca_expert_compact_scales", E * 2 * I, H, 1, 32)
        self.w2 = self._compact(ops.w2.to(d), "ca_expert_compact_words", E * H, I, 16, 32)
        self.s2 = self._compact(ops.s2.to(d), "ca_expert_compact_scales", E * H, I, 1, 32)
        self.sh_w13 = self._compact(ops.sh_w13.to(d), "ca_dense_compact_fp8", 2 * S, H, 16, 16, extra=(0,))
        self.sh_w2 = self._compact(ops.sh_w2.to(d), "ca_dense_compact_fp8", H, S, 16, 16, extra=(0,))
        self.sh_s13, self.sh_s2 = ops.sh_s13.to(d), ops.sh_s2.to(d)
        self.tile_m = 16 if rows <= STREAM_MAX_ROWS else GEMM_TILE_M
        pairs = rows * K
        self.max_tiles = -(-pairs // self.tile_m) - 1 + min(E, pairs)
        padded = self.max_tiles * self.tile_m
        z = lambda shape, dt: torch.zeros(shape, dtype=dt, device=d)
        self.logits = z((rows, E), torch.float32)
        self.ids = z((rows, K), torch.int32)
        self.weights = z((rows, K), torch.float32)
        self.xq, self.xs = z((rows, H), torch.uint8), z((rows, H // B), torch.uint8)
        self.xq_min, self.xs_min = z((rows, H), torch.uint8), z((rows, H // B), torch.uint8)
        self.h = z((padded, I), torch.int16)
        self.hq, self.hs = z((padded, I), torch.uint8), z((padded, I // B), torch.uint8)
        self.task_expert = torch.full((self.max_tiles,), -1, dtype=torch.int32, device=d)
        self.task_valid = torch.full((self.max_tiles,), -1, dtype=torch.int32, device=d)
        self.tile_base = torch.full((E + 1,), -1, dtype=torch.int32, device=d)
        self.token_map = torch.full((padded,), -1, dtype=torch.int32, device=d)
        self.token_weights = z((padded,), torch.float32)
        self.route_out = z((rows, K, H), torch.int16)
        waves = (pairs + 63) // 64
        self.plan_scratch = z((waves * E + pairs,), torch.int32)
        self.routed = z((rows, H), torch.int16)
        self.shared_up = z((rows, 2 * S), torch.int16)
        self.shared_act = z((rows, S), torch.int16)
        self.shared_aq, self.shared_as = z((rows, S), torch.uint8), z((rows, S // B), torch.uint8)
        self.shared_down = z((rows, H), torch.int16)
        self.out = z((rows, H), torch.int16)
        self.live = z((1,), torch.int32)
        self.tokens = z((rows,), torch.int64)
        self.padding = torch.full((rows,), -1, dtype=torch.int32, device=d)
        self.sync = z((1024 + 8 * 512,), torch.int32)      # arrival counters + the front-end's logit mailbox

    def _compact(self, src, kernel, n, k, unit_bytes, unit_elems, extra=None):
        src = src.contiguous()
        dst = torch.empty_like(src)
        total = n * (k // unit_elems)
        args = [src, dst, n, k] + (list(extra) if extra is not None else [n])
        native.launch(kernel, (total + 255) // 256, 256, args)
        torch.cuda.synchronize()
        return dst

    def close(self):
        self.lib.ca_primitives_close(ctypes.c_void_p(self.ctx))

    def run(self, x, tokens=None, live=None, padding=None, stream=0, fuse_route=None, fuse_gate=False):
        g, rows = self.g, self.rows
        K = g.topk
        self.x = x.to(self.dev).contiguous()
        self.live.fill_(rows if live is None else live)
        if tokens is not None:
            self.tokens.copy_(torch.as_tensor(tokens, dtype=torch.int64))
        use_padding = padding is not None
        if use_padding:
            self.padding.copy_(torch.as_tensor(padding, dtype=torch.int32))
        torch.cuda.synchronize()
        sp = ctypes.c_void_p(stream)
        fuse = rows * K <= 1024 if fuse_route is None else fuse_route
        fuse_gate = fuse_gate and fuse and rows <= STREAM_MAX_ROWS
        for off in range(0, rows, 16):
            if fuse_gate or (rows > 16 and rows > STREAM_MAX_ROWS):
                break
            n = min(16, rows - off)
            st = self.lib.ca_router_logits(n, ctypes.c_void_p(self.x.data_ptr() + off * g.hidden * 2), native.ptr(self.gate_w),
                                           ctypes.c_void_p(self.logits.data_ptr() + off * g.experts * 4), sp)
            assert st == 0, st
        if rows > STREAM_MAX_ROWS:
            st = self.lib.ca_router_logits_wide(rows, native.ptr(self.x), native.ptr(self.gate_w), native.ptr(self.logits), sp)
            assert st == 0, st
        dyn = [self.x, self.ids, self.weights, self.xq, self.xs, self.xq_min, self.xs_min, self.h, self.hq, self.hs,
               self.task_expert, self.task_valid, self.tile_base, self.token_map, self.token_weights, self.w13, self.s13,
               self.w2, self.s2, self.route_out, self.plan_scratch]
        scalars = [rows, rows, self.max_tiles * self.tile_m, self.max_tiles, self.tile_m, 1]
        if fuse:
            st = native.primitives_launch(self.ctx, 1, dyn + [self.logits, self.bias, self.bias_alt, self.tokens, self.live,
                                                             self.padding if use_padding else None, self.gate_w if fuse_gate else None, self.sync], scalars + [rows], stream)
        else:
            blocks = (rows + 15) // 16
            native.launch("ca_route_topk", blocks, 1024,
                          [self.logits, self.bias, self.bias_alt, self.tokens, self.live, self.padding if (use_padding and blocks == 1) else None,
                           self.ids, self.weights, rows, g.experts, K, g.scoring, float(g.route_scale), ctypes.c_int64(g.alt_token)], stream)
            if use_padding and blocks > 1:
                native.launch("ca_route_padding_rows", (rows * K + 127) // 128, 128, [self.ids, self.weights, self.padding, rows, K], stream)
            st = native.primitives_launch(self.ctx, 0, dyn, scalars, stream)
        assert st == 0, st
        st = native.primitives_launch(self.ctx, 5, [self.xq_min, self.xs_min, self.sh_w13, self.sh_s13, self.sh_w2, self.sh_s2,
                                                    self.shared_act, self.shared_aq, self.shared_as, self.shared_up, self.shared_down],
                                      [rows], stream)
        assert st == 0, st
        n_live = rows if live is None else min(live, rows)
        n = rows * g.hidden
        native.launch("ca_ffn_sum_shared", (n // 8 + 255) // 256, 256,
                      [self.route_out, self.shared_down, self.routed, self.out, n, n_live, K, g.hidden], stream)
        torch.cuda.synchronize()
        return self.taps()

    def taps(self):
        names = ["logits", "ids", "weights", "xq", "xs", "xq_min", "xs_min", "h", "hq", "hs", "task_expert", "task_valid",
                 "tile_base", "token_map", "token_weights", "route_out", "routed", "shared_up", "shared_act", "shared_aq",
                 "shared_as", "shared_down", "out"]
        out = {}
        for n in names:
            a = np_of(getattr(self, n))
            out[n] = a.view(np.uint16) if a.dtype == np.int16 else a
        return out


def oracle_layer(g, ops, x, tokens=None, live=None, padding=None, logits=None, ids_weights=None, simd=False):
    """Stage-by-stage oracle evaluation; routed experts are evaluated on the active experts only (ids remapped), so
    configs with hundreds of experts stay cheap.  `logits` / `ids_weights` substitute the GPU's own upstream results.
    `simd`: the three projection loops in their vectorised form (the CPU baseline; another summation order inside a block)."""
    cfg = oracle_config(g)
    rows = x.shape[0]
    K, I, H, B = g.topk, g.intermediate, g.hidden, g.act_block
    xb = u16(x)
    t = {}
    t["logits"] = oracle.router_logits(xb, u16(ops.gate_w)) if logits is None else logits
    tok = np.zeros(rows, np.int64) if tokens is None else np.asarray(tokens, np.int64)
    if ids_weights is None:
        t["ids"], t["weights"] = oracle.route_topk(cfg, t["logits"], np_of(ops.bias), np_of(ops.bias_alt), tok,
                                                   rows if live is None else live, padding)
    else:
        t["ids"], t["weights"] = ids_weights
    t["xq"], t["xs"] = oracle.quantize_rows(xb, B, 0.0)
    t["xq_min"], t["xs_min"] = oracle.quantize_rows(xb, B, 1e-4)
    active = sorted(set(int(e) for e in t["ids"].ravel() if 0 <= e < g.experts))
    remap = {e: i for i, e in enumerate(active)}
    ids_small = np.array([[remap.get(int(e), -1) for e in row] for row in t["ids"]], np.int32)
    small = oracle.config(H, max(1, len(active)), K, I, g.shared_intermediate, g.scoring, g.route_scale, B, g.shared_bn,
                          g.shared_bk, g.alt_token, g.swiglu_limit)
    pick = torch.as_tensor(active if active else [0], dtype=torch.long)
    w13, s13 = np_of(ops.w13[pick.to(ops.w13.device)]), np_of(ops.s13[pick.to(ops.s13.device)])
    w2, s2 = np_of(ops.w2[pick.to(ops.w2.device)]), np_of(ops.s2[pick.to(ops.s2.device)])
    t["h"] = oracle.expert_fc1(small, t["xq"], t["xs"], w13, s13, ids_small, simd=simd)
    hq, hs = oracle.quantize_rows(t["h"].reshape(rows * K, I), B, 0.0)
    t["hq"], t["hs"] = hq.reshape(rows, K, I), hs.reshape(rows, K, I // B)
    t["route_out"] = oracle.expert_fc2(small, t["hq"], t["hs"], w2, s2, ids_small, t["weights"], simd=simd)
    t["shared_up"] = oracle.fp8_linear(t["xq_min"], t["xs_min"], B, np_of(ops.sh_w13), np_of(ops.sh_s13), g.shared_bn, g.shared_bk, simd=simd)
    t["shared_act"], t["shared_aq"], t["shared_as"] = oracle.shared_swiglu_quant(t["shared_up"], B, g.swiglu_limit)
    t["shared_down"] = oracle.fp8_linear(t["shared_aq"], t["shared_as"], B, np_of(ops.sh_w2), np_of(ops.sh_s2), g.shared_bn, g.shared_bk, simd=simd)
    n_live = rows if live is None else min(live, rows)
    t["routed"], t["out"] = oracle.ffn_sum_shared(t["route_out"], t["shared_down"], n_live)
    return t


def _active_subset(g, ops, ids):
    active = sorted(set(int(e) for e in np.asarray(ids).ravel() if 0 <= e < g.experts))
    remap = {e: i for i, e in enumerate(active)}
    ids_small = np.array([[remap.get(int(e), -1) for e in row] for row in ids], np.int32)
    small = oracle.config(g.hidden, max(1, len(active)), g.topk, g.intermediate, g.shared_intermediate, g.scoring,
                          g.route_scale, g.act_block, g.shared_bn, g.shared_bk, g.alt_token, g.swiglu_limit)
    pick = torch.as_tensor(active if active else [0], dtype=torch.long)
    return small, ids_small, pick


def oracle_fc2_from(g, ops, ids, weights, hq, hs):
    """Oracle FC2 of given quantized intermediates ([rows][K][I] codes, [rows][K][I / block] scales)."""
    small, ids_small, pick = _active_subset(g, ops, ids)
    return oracle.expert_fc2(small, hq, hs, np_of(ops.w2[pick.to(ops.w2.device)]), np_of(ops.s2[pick.to(ops.s2.device)]),
                             ids_small, weights)


def bf16_ulp_distance(got_u16, want_u16, accumulation=1e-4):
    """Largest |got - want| in units of the allowance 2^-7 |want| (one BF16 rounding step) + `accumulation` * max |want|
    (FP32 / matrix-core accumulation-order noise of a dot product, which does not shrink with the result)."""
    gv, wv = bf(got_u16), bf(want_u16)
    if wv.size == 0:          # nothing to compare (no live route)
        return 0.0
    allowance = np.abs(wv) * 2.0 ** -7 + accumulation * np.abs(wv).max() + 1e-300
    return float((np.abs(gv - wv) / allowance).max())


def bf(a):
    return oracle.bf16_to_f32(a).astype(np.float64)


def error_report(got_u16, want_u16, floor=1e-3, bound=1e-2):
    """The layer-output tolerance in both readings.  `max_rel`: max |got - want| over max |want| (relative to the tensor's
    largest magnitude).  `max_elem_rel`: max over elements of |got - want| / max(|want|, floor * max |want|), the per-element
    relative error with an absolute floor below which an element's own magnitude no longer shrinks its allowance;
    `frac_above`: the fraction of elements whose per-element figure exceeds `bound`; `mean_abs`: mean |got - want|."""
    g, w = bf(got_u16), bf(want_u16)
    if w.size == 0:
        return {"max_rel": 0.0, "mean_abs": 0.0, "max_elem_rel": 0.0, "frac_above": 0.0, "elements": 0}
    scale = np.abs(w).max() + 1e-30
    diff = np.abs(g - w)
    elem = diff / np.maximum(np.abs(w), floor * scale)
    return {"max_rel": float(diff.max() / scale), "mean_abs": float(diff.mean()), "max_elem_rel": float(elem.max()),
            "frac_above": float((elem > bound).mean()), "elements": int(w.size)}


def assert_output_tolerance(name, got_u16, want_u16, max_rel=1e-2, mean_abs=1e-3, frac_above=None, max_elem_rel=None):
    """Prints both readings of the tolerance and asserts the stated bounds: max relative error (of the tensor's largest
    magnitude) and mean absolute error always; the per-element figures where the caller states a bound for them."""
    r = error_report(got_u16, want_u16)
    print("  %s: max rel %.3e (bound %.0e), mean abs %.3e (bound %.0e); per element with floor 1e-3 max|want|: max %.3e, above 1e-2: %.3e of %d"
          % (name, r["max_rel"], max_rel, r["mean_abs"], mean_abs, r["max_elem_rel"], r["frac_above"], r["elements"]))
    assert r["max_rel"] <= max_rel and r["mean_abs"] <= mean_abs, (name, r)
    if frac_above is not None:
        assert r["frac_above"] <= frac_above, (name, r)
    if max_elem_rel is not None:
        assert r["max_elem_rel"] <= max_elem_rel, (name, r)
    return r


def error_stats(got_u16, want_u16):
    """(max relative error against the reference's largest magnitude per row, mean absolute error)."""
    g, w = bf(got_u16), bf(want_u16)
    if w.size == 0:
        return 0.0, 0.0
    scale = np.abs(w).max() + 1e-30
    return float(np.abs(g - w).max() / scale), float(np.abs(g - w).mean())


# ---- float64 evaluation of the layer on the same quantized operands ------------------------------------------------------
_E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]


def _lut_e4m3(device):
    return torch.tensor([float(oracle.lib().orc_e4m3_to_f32(i)) for i in range(256)], dtype=torch.float64, device=device)


def dequant_mxfp4(w, s):
    """Packed E2M1 bytes [n][k/2] (low nibble = even column) with UE8M0 scales [n][k/32] -> float64 [n][k] (exact)."""
    lut = torch.tensor(_E2M1, dtype=torch.float64, device=w.device)
    nib = torch.stack([w & 15, w >> 4], dim=-1).reshape(w.shape[0], -1).long()
    scale = torch.pow(torch.tensor(2.0, dtype=torch.float64, device=w.device), s.double() - 127.0)
    return lut[nib] * scale.repeat_interleave(32, dim=1)


def dequant_fp8_blocks(w, s, bn, bk):
    """E4M3 codes [n][k] with UE8M0 block scales [n/bn][k/bk] -> float64 (exact)."""
    scale = torch.pow(torch.tensor(2.0, dtype=torch.float64, device=w.device), s.double() - 127.0)
    return _lut_e4m3(w.device)[w.long()] * scale.repeat_interleave(bn, dim=0).repeat_interleave(bk, dim=1)


def dequant_rows(codes, scales, block, device, zero_marks_zero_block):
    """Activation rows: E4M3 codes [rows][k], UE8M0 scales [rows][k/block] (numpy) -> float64 tensor (exact)."""
    q = torch.from_numpy(np.ascontiguousarray(codes)).to(device).long()
    s = torch.from_numpy(np.ascontiguousarray(scales)).to(device)
    scale = torch.pow(torch.tensor(2.0, dtype=torch.float64, device=device), s.double() - 127.0)
    if zero_marks_zero_block:
        scale = torch.where(s == 0, torch.zeros_like(scale), scale)
    return _lut_e4m3(device)[q] * scale.repeat_interleave(block, dim=1)


def _to_bf16_bits(t64):
    return t64.to(torch.float32).to(torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16)


def exact_layer(g, ops, x, ids, weights, live=None, h_given=None):
    """The layer with every dot product in float64 on the same quantized operands (dequantized exactly) and every
    requantization point of the layer kept (token codes, BF16 intermediate and its codes, BF16 route outputs, BF16 shared
    projections, the shared activation and its codes, the ordered FP32 route sum, the BF16 addition).  What a GPU or oracle
    result differs from it by is its own accumulation error, and what that error does to the FP8 codes downstream.  Runs on
    the operands' device (float64 matrix products of torch, an implementation of its own).  `h_given`: BF16 bits
    [rows][K][I] to continue from instead of the float64 FC1 + SwiGLU (what follows a given activation exactly)."""
    rows = x.shape[0]
    K, I, H, B = g.topk, g.intermediate, g.hidden, g.act_block
    dev = ops.w13.device
    xb = u16(x)
    t = {}
    xq, xs = oracle.quantize_rows(xb, B, 0.0)
    xq_min, xs_min = oracle.quantize_rows(xb, B, 1e-4)
    xr = dequant_rows(xq, xs, B, dev, True)
    h = np.zeros((rows * K, I), np.uint16)
    flat_ids = np.asarray(ids).reshape(-1)
    active = sorted(set(int(e) for e in flat_ids if 0 <= e < g.experts))
    limit = float(g.swiglu_limit)
    for e in active if h_given is None else []:
        routes = np.nonzero(flat_ids == e)[0]
        w = dequant_mxfp4(ops.w13[e], ops.s13[e])
        proj = xr[torch.as_tensor(routes // K, device=dev)] @ w.T
        up, gate = proj[:, :I], proj[:, I:]
        gv = torch.clamp(gate, max=limit)
        uv = torch.clamp(up, min=-limit, max=limit)
        h[routes] = _to_bf16_bits(gv * torch.sigmoid(gv) * uv)
    if h_given is not None:
        h = np.ascontiguousarray(h_given).reshape(rows * K, I).copy()
        h[~((flat_ids >= 0) & (flat_ids < g.experts))] = 0
    hq, hs = oracle.quantize_rows(h, B, 0.0)
    hd = dequant_rows(hq, hs, B, dev, True)
    route_out = np.zeros((rows * K, H), np.uint16)
    wts = torch.from_numpy(np.ascontiguousarray(np.asarray(weights, np.float32).reshape(-1))).to(dev).double()
    for e in active:
        routes = np.nonzero(flat_ids == e)[0]
        at = torch.as_tensor(routes, device=dev)
        w = dequant_mxfp4(ops.w2[e], ops.s2[e])
        route_out[routes] = _to_bf16_bits((hd[at] @ w.T) * wts[at][:, None])
    t["h"], t["hq"], t["hs"] = h.reshape(rows, K, I), hq.reshape(rows, K, I), hs.reshape(rows, K, -1)
    t["route_out"] = route_out.reshape(rows, K, H)
    xm = dequant_rows(xq_min, xs_min, B, dev, False)
    t["shared_up"] = _to_bf16_bits(xm @ dequant_fp8_blocks(ops.sh_w13, ops.sh_s13, g.shared_bn, g.shared_bk).T)
    t["shared_act"], aq, asc = oracle.shared_swiglu_quant(t["shared_up"], B, g.swiglu_limit)
    t["shared_down"] = _to_bf16_bits(dequant_rows(aq, asc, B, dev, False) @ dequant_fp8_blocks(ops.sh_w2, ops.sh_s2, g.shared_bn, g.shared_bk).T)
    n_live = rows if live is None else min(live, rows)
    t["routed"], t["out"] = oracle.ffn_sum_shared(t["route_out"], t["shared_down"], n_live)
    return t


def accuracy_table(name, gpu_out, oracle_out, exact_out, factor=1.5):
    """Both readings of the output error of the GPU and of the oracle against the float64 evaluation; asserts that the GPU is
    as close to exact arithmetic as the oracle is (within `factor`, and an allowance of one part in 10^4 of the largest
    magnitude for outputs where both are that close)."""
    a, b = error_report(gpu_out, exact_out), error_report(oracle_out, exact_out)
    print("  %s vs float64: GPU max rel %.3e, mean abs %.3e, per element max %.3e, above 1e-2 %.3e | oracle max rel %.3e, mean abs %.3e, "
          "per element max %.3e, above 1e-2 %.3e" % (name, a["max_rel"], a["mean_abs"], a["max_elem_rel"], a["frac_above"], b["max_rel"], b["mean_abs"],
                                                   b["max_elem_rel"], b["frac_above"]))
    return a, b
