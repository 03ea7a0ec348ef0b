"""numpy front-end of the CPU oracle (test infrastructure only).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this package: it is the checker the HIP path
is compared with, never part of the product path.  Arrays are plain numpy: bf16 as uint16, e4m3 / e2m1 pairs / ue8m0 as
uint8.
"""
import ctypes
import os

import numpy as np

from . import build as _build

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


class Config(ctypes.Structure):
    _fields_ = [("hidden", ctypes.c_int32), ("experts", ctypes.c_int32), ("topk", ctypes.c_int32),
                ("inter", ctypes.c_int32), ("shared_inter", ctypes.c_int32), ("scoring", ctypes.c_int32),
                ("route_scale", ctypes.c_float), ("act_block", ctypes.c_int32), ("shared_bn", ctypes.c_int32),
                ("shared_bk", ctypes.c_int32), ("alt_token", ctypes.c_int64), ("swiglu_limit", ctypes.c_float)]


class _LayerIn(ctypes.Structure):
    _fields_ = [("x", ctypes.c_void_p), ("tokens", ctypes.c_void_p), ("rows", ctypes.c_int32), ("live", ctypes.c_int32),
                ("padding", ctypes.c_void_p), ("gate_w", ctypes.c_void_p), ("bias", ctypes.c_void_p),
                ("bias_alt", ctypes.c_void_p), ("w13", ctypes.c_void_p), ("s13", ctypes.c_void_p),
                ("w2", ctypes.c_void_p), ("s2", ctypes.c_void_p), ("sh_w13", ctypes.c_void_p),
                ("sh_s13", ctypes.c_void_p), ("sh_w2", ctypes.c_void_p), ("sh_s2", ctypes.c_void_p)]


_TAPS = ["logits", "ids", "weights", "xq_routed", "xs_routed", "xq_shared", "xs_shared", "h", "hq", "hs", "route_out",
         "routed", "shared_up", "shared_act", "shared_aq", "shared_as", "shared_down", "out"]


class _LayerOut(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in _TAPS]


def lib():
    global _lib
    if _lib is None:
        path = _build.build(force=False)
        _lib = ctypes.CDLL(path)
        f32, u8, u16 = ctypes.c_float, ctypes.c_uint8, ctypes.c_uint16
        for name, res, args in [("orc_bf16_to_f32", f32, [u16]), ("orc_f32_to_bf16", u16, [f32]),
                                ("orc_e4m3_to_f32", f32, [u8]), ("orc_f32_to_e4m3", u8, [f32]),
                                ("orc_e2m1_to_f32", f32, [u8]), ("orc_f32_to_e2m1", u8, [f32]),
                                ("orc_ue8m0_to_f32", f32, [u8]), ("orc_exp", f32, [f32]),
                                ("orc_log1p_pos", f32, [f32]), ("orc_logistic", f32, [f32])]:
            getattr(_lib, name).restype = res
            getattr(_lib, name).argtypes = args
        _lib.orc_scale_code1_check.restype = ctypes.c_uint32
        _lib.orc_scale_codes4.restype = ctypes.c_uint32
        _lib.orc_simd_available.restype = ctypes.c_int32
    return _lib


def set_threads(n):
    lib().orc_set_threads(_i32(n))


def config(hidden, experts, topk, inter, shared_inter, scoring=0, route_scale=1.0, act_block=128, shared_bn=128,
           shared_bk=128, alt_token=-1, swiglu_limit=10.0):
    return Config(hidden, experts, topk, inter, shared_inter, scoring, route_scale, act_block, shared_bn, shared_bk,
                  alt_token, swiglu_limit)


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _i32(v):
    return ctypes.c_int32(int(v))


def _i64(v):
    return ctypes.c_int64(int(v))


# ---- scalar maps (vectorised through python loops: small inputs only) -------------------------------------------------
def map_scalar(name, values, out_dtype):
    f = getattr(lib(), name)
    flat = np.asarray(values).ravel()
    return np.array([f(v.item()) for v in flat], dtype=out_dtype).reshape(np.shape(values))


def bf16_to_f32(a):
    return (np.asarray(a, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(a):
    """Round to nearest even (numpy restatement used for building inputs, checked against orc_f32_to_bf16 in the tests)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7fffffff) > 0x7f800000
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


# ---- quantizers for synthetic weights ---------------------------------------------------------------------------------
def quantize_mxfp4(w):
    w = _c(w, np.float32)
    rows, cols = w.shape
    packed = np.empty((rows, cols // 2), np.uint8)
    scales = np.empty((rows, cols // 32), np.uint8)
    lib().orc_quantize_mxfp4(_p(w), _i64(rows), _i64(cols), _p(packed), _p(scales))
    return packed, scales


def quantize_fp8_blocks(w, bn, bk):
    w = _c(w, np.float32)
    rows, cols = w.shape
    codes = np.empty((rows, cols), np.uint8)
    scales = np.empty((rows // bn, cols // bk), np.uint8)
    lib().orc_quantize_fp8_blocks(_p(w), _i64(rows), _i64(cols), _i32(bn), _i32(bk), _p(codes), _p(scales))
    return codes, scales


# ---- router -----------------------------------------------------------------------------------------------------------
def router_logits(x, w):
    x, w = _c(x, np.uint16), _c(w, np.uint16)
    rows, hidden = x.shape
    experts = w.shape[0]
    out = np.empty((rows, experts), np.float32)
    lib().orc_router_logits(_p(x), _p(w), _p(out), _i32(rows), _i32(hidden), _i32(experts))
    return out


def route_topk(cfg, logits, bias, bias_alt=None, tokens=None, live=None, padding=None):
    logits = _c(logits, np.float32)
    rows = logits.shape[0]
    bias = _c(bias, np.float32)
    bias_alt = None if bias_alt is None else _c(bias_alt, np.float32)
    tokens = None if tokens is None else _c(tokens, np.int64)
    padding = None if padding is None else _c(padding, np.int32)
    ids = np.empty((rows, cfg.topk), np.int32)
    weights = np.empty((rows, cfg.topk), np.float32)
    lib().orc_route_topk(ctypes.byref(cfg), _p(logits), _p(bias), _p(bias_alt), _p(tokens),
                         _i32(rows if live is None else live), _p(padding), _p(ids), _p(weights), _i32(rows))
    return ids, weights


def route_padding_rows(ids, weights, source):
    ids, weights = _c(ids, np.int32).copy(), _c(weights, np.float32).copy()
    source = _c(source, np.int32)
    lib().orc_route_padding_rows(_p(ids), _p(weights), _p(source), _i32(ids.shape[0]), _i32(ids.shape[1]))
    return ids, weights


def route_census(ids, live, experts):
    ids = _c(ids, np.int32)
    counts = np.zeros(experts, np.uint32)
    lib().orc_route_census(_p(ids), _i32(live), _i32(ids.shape[0]), _i32(ids.shape[1]), _i32(experts), _p(counts))
    return counts


def plan(ids, weights, experts, groups, tile_m, capacity_tiles=None):
    """Returns the reference's five tables; untouched entries hold -1 (weights: 0)."""
    ids, weights = _c(ids, np.int32), _c(weights, np.float32)
    rows, topk = ids.shape
    pairs = rows * topk
    tiles = capacity_tiles if capacity_tiles is not None else min(pairs, experts + pairs // tile_m)
    base = np.full(experts + 1, -1, np.int32)
    task_expert = np.full(tiles * groups, -1, np.int32)
    task_valid = np.full(tiles * groups, -1, np.int32)
    token_map = np.full(tiles * tile_m, -1, np.int32)
    token_weights = np.zeros(tiles * tile_m, np.float32)
    lib().orc_plan(_p(ids), _p(weights), _i32(rows), _i32(topk), _i32(experts), _i32(groups), _i32(tile_m), _p(base),
                   _p(task_expert), _p(task_valid), _p(token_map), _p(token_weights))
    return base, task_expert, task_valid, token_map, token_weights


# ---- quantizers / shared expert -------------------------------------------------------------------------------------
def quantize_rows(x, block, min_amax=0.0):
    x = _c(x, np.uint16)
    rows, cols = x.shape
    codes = np.empty((rows, cols), np.uint8)
    scales = np.empty((rows, cols // block), np.uint8)
    lib().orc_quantize_rows(_p(x), _i32(rows), _i32(cols), _i32(block), ctypes.c_float(min_amax), _p(codes), _p(scales))
    return codes, scales


def shared_swiglu(x, limit=10.0):
    x = _c(x, np.uint16)
    rows, two = x.shape
    act = np.empty((rows, two // 2), np.uint16)
    lib().orc_shared_swiglu(_p(x), _p(act), _i32(rows), _i32(two // 2), ctypes.c_float(limit))
    return act


def shared_swiglu_quant(x, block, limit=10.0):
    x = _c(x, np.uint16)
    rows, two = x.shape
    inter = two // 2
    act = np.empty((rows, inter), np.uint16)
    codes = np.empty((rows, inter), np.uint8)
    scales = np.empty((rows, inter // block), np.uint8)
    lib().orc_shared_swiglu_quant(_p(x), _p(act), _p(codes), _p(scales), _i32(rows), _i32(inter), _i32(block),
                                  ctypes.c_float(limit))
    return act, codes, scales


def simd_available():
    """Whether the host has AVX2 + FMA, i.e. whether `simd=True` may be passed to the three projection functions."""
    return bool(lib().orc_simd_available())


def _projection(name, simd):
    if simd and not simd_available():
        raise RuntimeError("the vectorised oracle loops need AVX2 + FMA")
    return getattr(lib(), ("orc_simd_" if simd else "orc_") + name)


def fp8_linear(aq, a_scales, act_block, wq, w_scales, bn, bk, simd=False):
    aq, a_scales, wq, w_scales = _c(aq, np.uint8), _c(a_scales, np.uint8), _c(wq, np.uint8), _c(w_scales, np.uint8)
    rows, k = aq.shape
    n = wq.shape[0]
    out = np.empty((rows, n), np.uint16)
    _projection("fp8_linear", simd)(_p(aq), _p(a_scales), _i32(act_block), _p(wq), _p(w_scales), _i32(bn), _i32(bk), _i32(rows),
                         _i32(n), _i32(k), _p(out))
    return out


# ---- routed experts ---------------------------------------------------------------------------------------------------
def expert_fc1(cfg, xq, xs, w13, s13, ids, want_proj=False, simd=False):
    xq, xs, w13, s13, ids = _c(xq, np.uint8), _c(xs, np.uint8), _c(w13, np.uint8), _c(s13, np.uint8), _c(ids, np.int32)
    rows = xq.shape[0]
    h = np.empty((rows, cfg.topk, cfg.inter), np.uint16)
    proj = np.empty((rows, cfg.topk, 2 * cfg.inter), np.float32) if want_proj else None
    _projection("expert_fc1", simd)(ctypes.byref(cfg), _p(xq), _p(xs), _p(w13), _p(s13), _p(ids), _i32(rows), _p(h), _p(proj))
    return (h, proj) if want_proj else h


def expert_fc2(cfg, hq, hs, w2, s2, ids, weights, simd=False):
    hq, hs, w2, s2 = _c(hq, np.uint8), _c(hs, np.uint8), _c(w2, np.uint8), _c(s2, np.uint8)
    ids, weights = _c(ids, np.int32), _c(weights, np.float32)
    rows = ids.shape[0]
    out = np.empty((rows, cfg.topk, cfg.hidden), np.uint16)
    _projection("expert_fc2", simd)(ctypes.byref(cfg), _p(hq), _p(hs), _p(w2), _p(s2), _p(ids), _p(weights), _i32(rows), _p(out))
    return out


# ---- combine ----------------------------------------------------------------------------------------------------------
def topk_sum(routes, live=None, previous=None):
    routes = _c(routes, np.uint16)
    rows, topk, hidden = routes.shape
    routed = np.zeros((rows, hidden), np.uint16) if previous is None else _c(previous, np.uint16).copy()
    lib().orc_topk_sum(_p(routes), _p(routed), _i32(rows), _i32(topk), _i32(hidden), _i32(rows if live is None else live))
    return routed


def ffn_add(a, b):
    a, b = _c(a, np.uint16), _c(b, np.uint16)
    out = np.empty_like(a)
    lib().orc_ffn_add(_p(a), _p(b), _p(out), _i64(a.size))
    return out


def ffn_sum_shared(routes, shared, live=None, previous=None):
    routes, shared = _c(routes, np.uint16), _c(shared, np.uint16)
    rows, topk, hidden = routes.shape
    routed = np.zeros((rows, hidden), np.uint16) if previous is None else _c(previous, np.uint16).copy()
    out = np.empty((rows, hidden), np.uint16)
    lib().orc_ffn_sum_shared(_p(routes), _p(shared), _p(routed), _p(out), _i32(rows), _i32(topk), _i32(hidden),
                             _i32(rows if live is None else live))
    return routed, out


def rmsnorm(x, weight, eps):
    x, weight = _c(x, np.uint16), _c(weight, np.uint16)
    out = np.empty_like(x)
    lib().orc_rmsnorm(_p(x), _p(weight), _p(out), _i32(x.shape[0]), _i32(x.shape[1]), ctypes.c_float(eps))
    return out


def hc_mma_scale_bytes(rows, groups):
    """Size of the MMA-offset scale array for `rows` rows of `groups` 32-wide blocks: whole tiles of 128 rows."""
    return ((rows + 127) // 128) * ((groups + 3) // 4) * 512


def hc_combine_norm_quant(x, pre, weight, block=32, eps=1e-20, mma=True):
    """x [rows][streams][cols] BF16 bits, pre [rows][streams] f32 or None -> (y, q, sr, sm or None)."""
    x, weight = _c(x, np.uint16), _c(weight, np.uint16)
    rows, streams, cols = x.shape
    pre = None if pre is None else _c(pre, np.float32)
    y = np.empty((rows, cols), np.uint16)
    q = np.empty((rows, cols), np.uint8)
    sr = np.empty((rows, cols // block), np.uint8)
    sm = np.zeros(hc_mma_scale_bytes(rows, cols // block), np.uint8) if mma else None
    lib().orc_hc_combine_norm_quant(_p(x), None if pre is None else _p(pre), _p(weight), _p(y), _p(q), _p(sr),
                                    None if sm is None else _p(sm), _i32(rows), _i32(cols), _i32(streams), _i32(block),
                                    ctypes.c_float(eps))
    return y, q, sr, sm


def hc_post(a, residual, post, comb):
    """a [rows][cols], residual [rows][streams][cols] BF16 bits; post [rows][streams], comb [rows][streams][streams] f32."""
    a, residual = _c(a, np.uint16), _c(residual, np.uint16)
    post, comb = _c(post, np.float32), _c(comb, np.float32)
    rows, streams, cols = residual.shape
    y = np.empty_like(residual)
    lib().orc_hc_post(_p(a), _p(residual), _p(post), _p(comb), _p(y), _i32(rows), _i32(cols), _i32(streams))
    return y


def residual_add(a, b):
    a, b = _c(a, np.uint16), _c(b, np.uint16)
    out = np.empty_like(a)
    lib().orc_residual_add(_p(a), _p(b), _p(out), _i64(a.size))
    return out


# ---- whole layer ------------------------------------------------------------------------------------------------------
def layer(cfg, x, tokens, live, gate_w, bias, bias_alt, w13, s13, w2, s2, sh_w13, sh_s13, sh_w2, sh_s2, padding=None):
    """Runs the whole layer; returns a dict of every tap."""
    rows = x.shape[0]
    H, E, K, I, S, B = cfg.hidden, cfg.experts, cfg.topk, cfg.inter, cfg.shared_inter, cfg.act_block
    keep = dict(x=_c(x, np.uint16), tokens=_c(tokens, np.int64), gate_w=_c(gate_w, np.uint16), bias=_c(bias, np.float32),
                bias_alt=_c(bias if bias_alt is None else bias_alt, np.float32), w13=_c(w13, np.uint8),
                s13=_c(s13, np.uint8), w2=_c(w2, np.uint8), s2=_c(s2, np.uint8), sh_w13=_c(sh_w13, np.uint8),
                sh_s13=_c(sh_s13, np.uint8), sh_w2=_c(sh_w2, np.uint8), sh_s2=_c(sh_s2, np.uint8))
    pad = None if padding is None else _c(padding, np.int32)
    lin = _LayerIn(_p(keep["x"]), _p(keep["tokens"]), rows, live, _p(pad), _p(keep["gate_w"]), _p(keep["bias"]),
                   _p(keep["bias_alt"]), _p(keep["w13"]), _p(keep["s13"]), _p(keep["w2"]), _p(keep["s2"]),
                   _p(keep["sh_w13"]), _p(keep["sh_s13"]), _p(keep["sh_w2"]), _p(keep["sh_s2"]))
    taps = dict(logits=np.zeros((rows, E), np.float32), ids=np.zeros((rows, K), np.int32),
                weights=np.zeros((rows, K), np.float32), xq_routed=np.zeros((rows, H), np.uint8),
                xs_routed=np.zeros((rows, H // B), np.uint8), xq_shared=np.zeros((rows, H), np.uint8),
                xs_shared=np.zeros((rows, H // B), np.uint8), h=np.zeros((rows, K, I), np.uint16),
                hq=np.zeros((rows, K, I), np.uint8), hs=np.zeros((rows, K, I // B), np.uint8),
                route_out=np.zeros((rows, K, H), np.uint16), routed=np.zeros((rows, H), np.uint16),
                shared_up=np.zeros((rows, 2 * S), np.uint16), shared_act=np.zeros((rows, S), np.uint16),
                shared_aq=np.zeros((rows, S), np.uint8), shared_as=np.zeros((rows, S // B), np.uint8),
                shared_down=np.zeros((rows, H), np.uint16), out=np.zeros((rows, H), np.uint16))
    lout = _LayerOut(*[_p(taps[n]) for n in _TAPS])
    lib().orc_layer(ctypes.byref(cfg), ctypes.byref(lin), ctypes.byref(lout))
    return taps


# ---- layouts and codes ------------------------------------------------------------------------------------------------
def _stream(name, src, n, k, inverse):
    src = _c(src, np.uint8)
    dst = np.empty_like(src)
    getattr(lib(), name)(_p(src), _p(dst), _i32(n), _i32(k), _i32(1 if inverse else 0))
    return dst


def stream_words(src, n, k, inverse=False):
    return _stream("orc_stream_words", src, n, k, inverse)


def stream_scales(src, n, k, inverse=False):
    return _stream("orc_stream_scales", src, n, k, inverse)


def stream_fp8(src, n, k, inverse=False):
    return _stream("orc_stream_fp8", src, n, k, inverse)


def nibble_permute(words, inverse=False):
    words = _c(words, np.uint32).copy()
    lib().orc_nibble_permute(_p(words), ctypes.c_uint64(words.size), _i32(1 if inverse else 0))
    return words


def scale_code1_layout(experts, hidden, inter):
    out = (ctypes.c_int64 * 6)()
    lib().orc_scale_code1_layout(_i64(experts), _i64(hidden), _i64(inter), out)
    return tuple(out)


def scale_code1(scales, matrices, n, columns):
    scales = _c(scales, np.uint8)
    units = ((n + 127) // 128) * ((columns + 3) // 4)
    code = np.zeros(matrices * units * 16, np.uint32)
    flags = np.zeros(matrices * units * 4, np.uint32)
    bases = np.zeros(matrices, np.uint32)
    lib().orc_scale_code1(_p(scales), _p(code), _p(flags), _p(bases), _i32(matrices), _i32(n), _i32(columns))
    return code, flags, bases


def scale_code1_check(scales, code, flags, bases, matrices, n, columns):
    raw = ctypes.c_uint64(0)
    err = lib().orc_scale_code1_check(_p(_c(scales, np.uint8)), _p(_c(code, np.uint32)), _p(_c(flags, np.uint32)),
                                      _p(_c(bases, np.uint32)), _i32(matrices), _i32(n), _i32(columns), ctypes.byref(raw))
    return err, raw.value


def scale_codes4(source, matrices, n, columns):
    source = _c(source, np.uint8)
    out = np.zeros(matrices * n * columns, np.uint8)
    err = lib().orc_scale_codes4(_p(source), _p(out), _i32(matrices), _i32(n), _i32(columns))
    return out, err


def scale_codes4_decode(coded, matrices, n, columns):
    coded = _c(coded, np.uint8)
    out = np.zeros(matrices * n * columns, np.uint8)
    lib().orc_scale_codes4_decode(_p(coded), _p(out), _i32(matrices), _i32(n), _i32(columns))
    return out


def codec_row_bytes(k):
    return k + (k // 32) * 5


def codec_encode(routed, routed_scales, shared):
    routed, routed_scales, shared = _c(routed, np.uint8), _c(routed_scales, np.uint8), _c(shared, np.uint8)
    rows, k = routed.shape
    packed = np.zeros((rows, codec_row_bytes(k)), np.uint8)
    lib().orc_codec_encode(_p(routed), _p(routed_scales), _p(shared), _p(packed), _i32(rows), _i32(k))
    return packed


def codec_decode(packed, k, mma=False):
    packed = _c(packed, np.uint8)
    rows = packed.shape[0]
    shared = np.empty((rows, k), np.uint8)
    row_scales = np.empty((rows, k // 32), np.uint8)
    mma_scales = np.zeros(rows * (k // 32), np.uint8) if mma else None
    lib().orc_codec_decode(_p(packed), _p(shared), _p(row_scales), _p(mma_scales), _i32(rows), _i32(k))
    return (shared, row_scales, mma_scales) if mma else (shared, row_scales)


def codec_pack_bf16(x):
    x = _c(x, np.uint16)
    rows, k = x.shape
    packed = np.zeros((rows, codec_row_bytes(k)), np.uint8)
    lib().orc_codec_pack_bf16(_p(x), _p(packed), _i32(rows), _i32(k))
    return packed


def codec_local_live(global_live, rows, rank):
    f = lib().orc_codec_local_live
    f.restype = ctypes.c_int32
    return int(f(_i32(global_live), _i32(rows), _i32(rank)))
