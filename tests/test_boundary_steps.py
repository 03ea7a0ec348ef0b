"""The steps either side of the layer at the decoder's FFN boundary (src/decoder.rs:1497-1543, 1654-1656; src/ffn.rs:974-975):
the producer whose output the layer takes instead of quantizing itself -- the reference's `hc_combine_norm_quant`
(runtime/kernels/mhc-norm-quant-v1/mhc-norm-quant.py:15-44: stream combine, RMS norm, MXFP8 codes, row and matrix-instruction
scale bytes) -- and the post step behind the layer, `hc_post_tiles` (runtime/kernels/mhc-post-tiles-v1/mhc-post-tiles.py:11-27),
alone and fused behind the route sum and the shared addition; plus their single-stream forms.  The oracle's restatements are
pinned here on the CPU (float64, crafted cases whose exact answer is known, closed forms, brute force over the scale-byte
offsets); the kernels are compared with the oracle bit for bit on the GPU.  Unpinned against the reference's object code: the
summation order of the squares and its approximate reciprocal root (rsqrt.approx / div.full there)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import bf, geometry, native, np_of, synth, u16


def norm_inputs(rows, cols, name="norm"):
    x = synth.normal(name + "/x", (rows, cols), std=3.0)
    x[0, :] *= 1e-3                      # a row of tiny values: eps matters
    if rows > 2:
        x[2, :] = 0.0                    # a zero row: every block zero
        x[1, 5] = 300.0                  # an outlier
    w = 1.0 + synth.normal(name + "/w", (cols,), std=0.2)
    return u16(synth.to_bf16_bits(x)), u16(synth.to_bf16_bits(w))


@pytest.mark.parametrize("cols", [1024, 4096, 5120, 8192])
def test_rmsnorm_against_float64(cols):
    eps = 1e-6
    x, w = norm_inputs(5, cols)
    got = bf(oracle.rmsnorm(x, w, eps))
    xf, wf = bf(x), bf(w)
    want = xf / np.sqrt((xf * xf).mean(axis=1, keepdims=True) + eps) * wf
    # one BF16 rounding of a value computed with three FP32 roundings before it: within 2^-8 relative + FP32 noise
    assert np.all(np.abs(got - want) <= np.abs(want) * (2.0 ** -8 + 1e-6) + 1e-30)
    assert not got[2].any()
    # a dropped eps, a missing weight or a sum over the wrong length would all fail the bound above; so would a wrong order of
    # the two products by more than rounding.  The summation order itself: permuting the row changes at most the last bits
    perm = np.random.default_rng(1).permutation(cols)
    again = bf(oracle.rmsnorm(x[:, perm], w[perm], eps))
    assert np.all(np.abs(again - got[:, perm]) <= np.abs(got[:, perm]) * 2.0 ** -7)


def hc_inputs(rows, cols, streams=4, name="hc"):
    x = synth.normal(name + "/x", (rows, streams, cols), std=2.0)
    if rows > 2:
        x[2] = 0.0                       # a zero row: every block at the quantizer's floor
        x[1, 0, 5] = 300.0               # an outlier
    pre = synth.normal(name + "/pre", (rows, streams), std=0.4, mean=0.5)          # asymmetric over the streams
    w = 1.0 + synth.normal(name + "/w", (cols,), std=0.2)
    return u16(synth.to_bf16_bits(x)), pre.numpy().copy(), u16(synth.to_bf16_bits(w))


def bf16_round(v64):
    return bf(oracle.f32_to_bf16(v64.astype(np.float32)))


@pytest.mark.parametrize("cols", [1024, 4096, 5120])
def test_hc_combine_norm_quant_against_float64(cols):
    rows = 6
    x, pre, w = hc_inputs(rows, cols)
    y, q, sr, sm = oracle.hc_combine_norm_quant(x, pre, w)
    value = bf16_round((bf(x) * pre[:, :, None].astype(np.float64)).sum(axis=1))       # the BF16 combine boundary
    want = value / np.sqrt((value * value).mean(axis=1, keepdims=True) + 1e-20) * bf(w)
    got = bf(y)
    err = np.abs(got - want)
    # one BF16 rounding of a value with three FP32 roundings before it.  Where the FP32 chain and float64 land on different sides
    # of a BF16 tie of the combine (a handful of elements in 30,000) the input of the norm is one BF16 step off
    one_step = np.abs(want) * (2.0 ** -8 + 1e-6) + 1e-30
    assert np.mean(err > one_step) < 2e-3 and np.all(err <= 3 * one_step)
    assert not got[2].any()
    # a transposed coefficient table (pre[c][row]), a dropped stream or a stream order that matters would fail the bound: the
    # coefficients differ per stream and row
    swapped = pre.copy()
    swapped[:, [0, 1]] = swapped[:, [1, 0]]
    other = bf(oracle.hc_combine_norm_quant(x, swapped, w)[0])
    assert np.mean(np.abs(other - want) > one_step) > 0.5
    # the codes and the scale bytes are the shared-flavour quantizer's of the normalized row (32-wide blocks, amax floored at 1e-4)
    codes, scales = oracle.quantize_rows(y, 32, 1e-4)
    assert np.array_equal(q, codes) and np.array_equal(sr, scales)
    assert np.all(sr[2] == 105) and not q[2].any()                # 1e-4 / 448 rounded up to a power of two: 2^-22
    assert sr.min() >= 105


def test_hc_combine_keeps_the_bf16_boundary_and_fuses_the_products():
    cols = 5120
    w = u16(synth.to_bf16_bits(torch.ones(cols)))
    # (a) the BF16 boundary behind the combine.  One column holds 64, every other column 1 + 0.49 * 2^-7, which the boundary
    # rounds to 1: mean square (4096 + 5119) / 5120 with it, (4096 + 5119 * 1.00767) / 5120 without; 64 / rms = 47.705 against
    # 47.604, i.e. 47.75 against 47.5 in BF16 (steps of 0.25 there)
    x = np.zeros((1, 4, cols), np.float32)
    x[0, 0, :] = 1.0
    x[0, 0, 7] = 64.0
    pre = np.array([[1.0 + 0.49 * 2.0 ** -7, 0.0, 0.0, 0.0]], np.float32)
    x[0, 1, 7] = 64.0                                               # the big column: 64 * pre0 + 64 * pre1 = 64 exactly
    pre[0, 1] = 1.0 - pre[0, 0]
    y = bf(oracle.hc_combine_norm_quant(u16(synth.to_bf16_bits(torch.from_numpy(x))), pre, w)[0])
    assert y[0, 7] == 47.75 and np.all(np.delete(y[0], 7) == 0.74609375)          # 1 / rms = 0.74540 -> BF16 0.74609375
    # (b) fused multiply-adds.  value = fma(x1, pre1, fma(x0, pre0, 0)) with x0 = -(1 + 2^-7), pre0 = 1, x1 = 1 + 2^-7,
    # pre1 = 1 + 2^-23: the exact second product is 1 + 2^-7 + 2^-23 + 2^-30, so the fused chain leaves 2^-23 (1 + 2^-7), a
    # separately rounded product 2^-23.  Every other column is 1, so 1 / rms = 1.0000977 and the BF16 result keeps the difference
    x = np.zeros((1, 4, cols), np.float32)
    x[0, 0, :] = 1.0
    x[0, 0, 3], x[0, 1, 3] = -(1.0 + 2.0 ** -7), 1.0 + 2.0 ** -7
    pre = np.array([[1.0, 1.0 + 2.0 ** -23, 0.0, 0.0]], np.float32)
    y = bf(oracle.hc_combine_norm_quant(u16(synth.to_bf16_bits(torch.from_numpy(x))), pre, w)[0])
    assert y[0, 3] == 2.0 ** -23 * (1.0 + 2.0 ** -7) and y[0, 0] == 1.0
    # (c) the order of the streams: fma(c, 1, fma(b, 1, fma(a, 1, 0))) with a = 2^30, b = -2^30, c = 1 gives 1; any other order loses it
    x = np.zeros((1, 4, cols), np.float32)
    x[0, 3, :] = 1.0
    x[0, 0, 9], x[0, 1, 9], x[0, 3, 9] = 2.0 ** 30, -2.0 ** 30, 0.0
    x[0, 2, 9] = 1.0
    ones = np.ones((1, 4), np.float32)
    y = bf(oracle.hc_combine_norm_quant(u16(synth.to_bf16_bits(torch.from_numpy(x))), ones, w)[0])
    assert y[0, 9] == 1.0
    x[0, 0, 9], x[0, 2, 9] = 1.0, 2.0 ** 30                         # 1 first: lost against 2^30
    y = bf(oracle.hc_combine_norm_quant(u16(synth.to_bf16_bits(torch.from_numpy(x))), ones, w)[0])
    assert y[0, 9] == 0.0


def test_hc_scale_byte_offsets_by_brute_force():
    # sm[(row % 32) * 16 + ((row / 32) % 4) * 4 + (row / 128) * 20480 + (group / 4) * 512 + group % 4] at 5,120 columns
    # (mhc-norm-quant.py:44): a bijection of (row, group) onto whole 128-row tiles of 160 groups, with the reference's constants
    rows, cols = 300, 5120
    groups = cols // 32
    x, pre, w = hc_inputs(rows, cols, name="hc-offsets")
    y, q, sr, sm = oracle.hc_combine_norm_quant(x, pre, w)
    assert sm.size == 3 * 20480 == oracle.hc_mma_scale_bytes(rows, groups)
    seen = np.zeros(sm.size, bool)
    for row in range(rows):
        for group in range(groups):
            at = (row % 32) * 16 + ((row // 32) % 4) * 4 + (row // 128) * 20480 + (group // 4) * 512 + group % 4
            assert not seen[at] and sm[at] == sr[row, group]
            seen[at] = True
    assert seen.sum() == rows * groups and not sm[~seen].any()      # the offsets of absent rows stay as they were
    # the row codec's decoder writes the same bytes at the same offsets from a second source of the reference
    # (moe-dual-quant-codec-fast.cu:69-74), for the rows of whole tiles
    packed = oracle.codec_pack_bf16(y[:256])
    shared, row_scales, mma = oracle.codec_decode(packed, cols, mma=True)
    assert np.array_equal(shared, q[:256]) and np.array_equal(row_scales, sr[:256]) and np.array_equal(mma, sm[:2 * 20480])


def test_single_stream_is_the_plain_norm():
    x, w = norm_inputs(5, 4096, "single")
    for eps in (1e-20, 1e-6):
        y = oracle.hc_combine_norm_quant(x[:, None, :], None, w, eps=eps, mma=False)[0]
        assert np.array_equal(y, oracle.rmsnorm(x, w, eps))
    ones = np.ones((5, 1), np.float32)
    assert np.array_equal(oracle.hc_combine_norm_quant(x[:, None, :], ones, w, eps=1e-6, mma=False)[0], oracle.rmsnorm(x, w, 1e-6))


def post_inputs(rows, cols, name="post"):
    a = u16(synth.to_bf16_bits(synth.normal(name + "/a", (rows, cols), std=1.5)))
    r = u16(synth.to_bf16_bits(synth.normal(name + "/r", (rows, 4, cols), std=2.0)))
    post = synth.normal(name + "/post", (rows, 4), std=0.5, mean=0.8).numpy().copy()
    comb = synth.normal(name + "/comb", (rows, 4, 4), std=0.5, mean=0.25).numpy().copy()      # not symmetric
    return a, r, post, comb


def test_hc_post_against_float64_and_special_cases():
    rows, cols = 7, 1024
    a, r, post, comb = post_inputs(rows, cols)
    got = bf(oracle.hc_post(a, r, post, comb))
    # y[row][c] = post[c] a + sum_s comb[s][c] r_s
    want = post[:, :, None].astype(np.float64) * bf(a)[:, None, :] + np.einsum("rsc,rsh->rch", comb.astype(np.float64), bf(r))
    scale = np.abs(post[:, :, None]) * np.abs(bf(a))[:, None, :] + np.einsum("rsc,rsh->rch", np.abs(comb).astype(np.float64), np.abs(bf(r)))
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + scale * 4e-7)       # one BF16 rounding + four FP32 roundings
    transposed = bf(oracle.hc_post(a, r, post, np.ascontiguousarray(comb.transpose(0, 2, 1))))
    assert np.mean(np.abs(transposed - want) > np.abs(want) * 2.0 ** -8 + scale * 4e-7) > 0.5
    # identity mix and no post term: the streams come back bit for bit; post 1 and no mix: every stream is the layer's output
    eye = np.broadcast_to(np.eye(4, dtype=np.float32), (rows, 4, 4)).copy()
    zero4, one4 = np.zeros((rows, 4), np.float32), np.ones((rows, 4), np.float32)
    assert np.array_equal(oracle.hc_post(a, r, zero4, eye), r)
    assert np.array_equal(oracle.hc_post(a, r, one4, np.zeros_like(eye)), np.broadcast_to(a[:, None, :], r.shape))
    # stream s goes to output c through comb[s][c]: a single one at [1][3] moves stream 1 to output 3 alone
    single = np.zeros_like(eye)
    single[:, 1, 3] = 1.0
    moved = oracle.hc_post(a, r, zero4, single)
    assert np.array_equal(moved[:, 3], r[:, 1]) and not (moved[:, [0, 1, 2]] & 0x7fff).any()


def test_residual_add_against_float64():
    rng = np.random.default_rng(2)
    a = rng.integers(0, 1 << 16, 200000).astype(np.uint16)
    b = rng.integers(0, 1 << 16, 200000).astype(np.uint16)
    finite = np.isfinite(bf(a)) & np.isfinite(bf(b)) & (np.abs(bf(a)) < 1e30) & (np.abs(bf(b)) < 1e30)
    a, b = a[finite], b[finite]
    got = oracle.residual_add(a, b)
    exact = bf(a) + bf(b)                                   # exact in float64
    want = oracle.f32_to_bf16(exact.astype(np.float32))     # the same two roundings (FP32, then BF16)
    assert np.array_equal(got, want)
    # against the once-rounded sum: equal but for double rounding, and never more than one BF16 step away
    err = np.abs(bf(got) - exact)
    ulp = np.maximum(np.abs(exact), 2.0 ** -126) * 2.0 ** -7
    assert np.all(err <= ulp)
    # unlike the shared addition (flush to zero) subnormal sums survive
    tiny = np.array([0x0001], np.uint16)
    assert oracle.residual_add(tiny, tiny)[0] == 0x0002 and oracle.ffn_add(tiny, tiny)[0] == 0


@pytest.mark.gpu
@pytest.mark.parametrize("mode,hidden,rows", [("benchmark", 4096, 4), ("reference", 5120, 6), ("reference", 1024, 40), ("benchmark", 8192, 3)])
def test_norm_quant_kernel_bit_exact(mode, hidden, rows):
    g = geometry(hidden, 16, 2, 512, 512, mode)
    lib = native.load()
    ctx = native.open_context(g)
    x, w = norm_inputs(rows, hidden, "gpu-norm")
    xd, wd = torch.from_numpy(x.view(np.int16)).cuda(), torch.from_numpy(w.view(np.int16)).cuda()
    B = g.act_block
    normed = torch.zeros((rows, hidden), dtype=torch.int16, device="cuda")
    codes, scales = torch.zeros((rows, hidden), dtype=torch.uint8, device="cuda"), torch.zeros((rows, hidden // B), dtype=torch.uint8, device="cuda")
    codes_min, scales_min = torch.zeros_like(codes), torch.zeros_like(scales)
    eps = 1e-6
    st = lib.ca_ffn_norm_quant(ctypes.c_void_p(ctx), rows, native.ptr(xd), native.ptr(wd), eps, native.ptr(normed), native.ptr(codes),
                               native.ptr(scales), native.ptr(codes_min), native.ptr(scales_min), None)
    torch.cuda.synchronize()
    assert st == 0
    want = oracle.rmsnorm(x, w, eps)
    assert np.array_equal(np_of(normed).view(np.uint16), want)
    q, s = oracle.quantize_rows(want, B, 0.0)
    assert np.array_equal(np_of(codes), q) and np.array_equal(np_of(scales), s)
    q, s = oracle.quantize_rows(want, B, 1e-4)
    assert np.array_equal(np_of(codes_min), q) and np.array_equal(np_of(scales_min), s)
    # one flavour alone, and the argument checks
    codes.zero_()
    assert lib.ca_ffn_norm_quant(ctypes.c_void_p(ctx), rows, native.ptr(xd), native.ptr(wd), eps, native.ptr(normed), None, None,
                                 native.ptr(codes_min), native.ptr(scales_min), None) == 0
    torch.cuda.synchronize()
    assert not np_of(codes).any()
    assert lib.ca_ffn_norm_quant(ctypes.c_void_p(ctx), rows, native.ptr(xd), native.ptr(wd), eps, native.ptr(normed), native.ptr(codes), None,
                                 None, None, None) == -1
    assert lib.ca_ffn_norm_quant(None, rows, native.ptr(xd), native.ptr(wd), eps, native.ptr(normed), None, None, None, None, None) == -1
    lib.ca_primitives_close(ctypes.c_void_p(ctx))


def dev(a):
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    return torch.from_numpy(a).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("mode,hidden,rows", [("reference", 5120, 6), ("reference", 5120, 16), ("reference", 5120, 128), ("reference", 5120, 300),
                                              ("benchmark", 4096, 4), ("reference", 1024, 40), ("benchmark", 8192, 3)])
def test_hc_combine_norm_quant_kernel_bit_exact(mode, hidden, rows):
    g = geometry(hidden, 16, 2, 512, 512, mode)
    lib = native.load()
    ctx = native.open_context(g)
    B, groups = g.act_block, hidden // g.act_block
    x, pre, w = hc_inputs(rows, hidden, name="gpu-hc")
    xd, pd, wd = dev(x), dev(pre), dev(w)
    normed = torch.zeros((rows, hidden), dtype=torch.int16, device="cuda")
    q, sr = torch.zeros((rows, hidden), dtype=torch.uint8, device="cuda"), torch.zeros((rows, groups), dtype=torch.uint8, device="cuda")
    routed_q, routed_s = torch.zeros_like(q), torch.zeros_like(sr)
    sm = torch.full((oracle.hc_mma_scale_bytes(rows, groups),), 0x55, dtype=torch.uint8, device="cuda") if B == 32 else None
    st = lib.ca_hc_combine_norm_quant(ctypes.c_void_p(ctx), rows, 4, native.ptr(xd), native.ptr(pd), native.ptr(wd), native.ptr(normed), native.ptr(q),
                                      native.ptr(sr), native.ptr(sm) if sm is not None else None, native.ptr(routed_q), native.ptr(routed_s), None)
    torch.cuda.synchronize()
    assert st == 0
    want_y, want_q, want_sr, want_sm = oracle.hc_combine_norm_quant(x, pre, w, block=B, mma=B == 32)
    assert np.array_equal(np_of(normed).view(np.uint16), want_y)
    assert np.array_equal(np_of(q), want_q) and np.array_equal(np_of(sr), want_sr)
    codes, scales = oracle.quantize_rows(want_y, B, 0.0)
    assert np.array_equal(np_of(routed_q), codes) and np.array_equal(np_of(routed_s), scales)
    if sm is not None:
        written = np.zeros(want_sm.size, bool)
        for row in range(rows):
            for group in range(groups):
                written[(row % 32) * 16 + ((row // 32) % 4) * 4 + (row // 128) * ((groups + 3) // 4 * 512) + (group // 4) * 512 + group % 4] = True
        got = np_of(sm)
        assert np.array_equal(got[written], want_sm[written]) and np.all(got[~written] == 0x55)      # absent rows' bytes are left alone
    # single stream, no coefficients: the plain norm's bits at the reference's eps (the buffer read as [rows][1][hidden])
    one = torch.zeros_like(normed)
    assert lib.ca_hc_combine_norm_quant(ctypes.c_void_p(ctx), rows, 1, native.ptr(xd), None, native.ptr(wd), native.ptr(one), None, None, None, None,
                                        None, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(np_of(one).view(np.uint16), oracle.rmsnorm(np.ascontiguousarray(x.reshape(rows * 4, hidden)[:rows]), w, 1e-20))
    # argument checks: a pair given by half, scale bytes at matrix-instruction offsets for another block width, no context
    assert lib.ca_hc_combine_norm_quant(ctypes.c_void_p(ctx), rows, 4, native.ptr(xd), native.ptr(pd), native.ptr(wd), native.ptr(normed), native.ptr(q),
                                        None, None, None, None, None) == -1
    if B != 32:
        assert lib.ca_hc_combine_norm_quant(ctypes.c_void_p(ctx), rows, 4, native.ptr(xd), native.ptr(pd), native.ptr(wd), native.ptr(normed),
                                            native.ptr(q), native.ptr(sr), native.ptr(q), None, None, None) == -1
    assert lib.ca_hc_combine_norm_quant(None, rows, 4, native.ptr(xd), native.ptr(pd), native.ptr(wd), native.ptr(normed), None, None, None, None, None,
                                        None) == -1
    lib.ca_primitives_close(ctypes.c_void_p(ctx))


@pytest.mark.gpu
@pytest.mark.parametrize("hidden,rows", [(5120, 6), (4096, 37), (1024, 300)])
def test_hc_post_kernel_bit_exact(hidden, rows):
    g = geometry(hidden, 16, 2, 512, 512, "reference")
    lib = native.load()
    ctx = native.open_context(g)
    a, r, post, comb = post_inputs(rows, hidden, "gpu-post")
    ad, rd, pd, cd = dev(a), dev(r), dev(post), dev(comb)
    y = torch.zeros_like(rd)
    assert lib.ca_hc_post(ctypes.c_void_p(ctx), rows, native.ptr(ad), native.ptr(rd), native.ptr(pd), native.ptr(cd), native.ptr(y), None) == 0
    torch.cuda.synchronize()
    want = oracle.hc_post(a, r, post, comb)
    assert np.array_equal(np_of(y).view(np.uint16), want)
    # in place
    assert lib.ca_hc_post(ctypes.c_void_p(ctx), rows, native.ptr(ad), native.ptr(rd), native.ptr(pd), native.ptr(cd), native.ptr(rd), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(rd, y)
    assert lib.ca_hc_post(ctypes.c_void_p(ctx), rows, native.ptr(ad), native.ptr(rd), None, native.ptr(cd), native.ptr(y), None) == -1
    lib.ca_primitives_close(ctypes.c_void_p(ctx))


@pytest.mark.gpu
def test_the_layer_between_the_reference_boundary_operators():
    # hc_combine_norm_quant -> Layer.run_quantized (the layer skips its own quantizer: src/ffn.rs:974-975) -> sum + shared + hc_post in one
    # pass, at the reference's numerics (32-wide blocks).  The layer's output from the producer's codes equals its output from the
    # normalized rows alone, and the fused pass equals the oracle's sum, addition and post step.
    from helpers import pkg
    g = geometry(1024, 16, 2, 512, 512, "reference")
    ops = synth.LayerOperands(g, "c1", device="cpu")
    rows, live = 8, 6
    lib = native.load()
    ctx = native.open_context(g)
    x, pre, w = hc_inputs(rows, g.hidden, name="chain-hc")
    x[2] = x[3]                                             # no zero row in the chain
    xd, pd, wd = dev(x), dev(pre), dev(w)
    groups = g.hidden // 32
    normed = torch.zeros((rows, g.hidden), dtype=torch.int16, device="cuda")
    q, sr = torch.zeros((rows, g.hidden), dtype=torch.uint8, device="cuda"), torch.zeros((rows, groups), dtype=torch.uint8, device="cuda")
    sm = torch.zeros(oracle.hc_mma_scale_bytes(rows, groups), dtype=torch.uint8, device="cuda")
    assert lib.ca_hc_combine_norm_quant(ctypes.c_void_p(ctx), rows, 4, native.ptr(xd), native.ptr(pd), native.ptr(wd), native.ptr(normed), native.ptr(q),
                                        native.ptr(sr), native.ptr(sm), None, None, None) == 0
    torch.cuda.synchronize()
    layer = pkg.host.Layer(g, ops, rows)
    layer.set_tokens()
    layer.run(normed)
    plain = layer.taps()
    layer.run_quantized(normed, q, sr)
    fed = layer.taps()
    assert np.array_equal(fed["out"], plain["out"]) and np.array_equal(fed["route_out"], plain["route_out"])
    a_unused, r, post, comb = post_inputs(rows, g.hidden, "chain-post")
    routes, shared = dev(plain["route_out"]), dev(plain["shared_down"])
    routed = dev(plain["routed"]).clone()
    routed[live:] = 0x3c00                                  # rows past the live ones keep what the buffer holds
    before = np_of(routed).view(np.uint16).copy()
    rd, pod, cd = dev(r), dev(post), dev(comb)
    ffn, y = torch.zeros((rows, g.hidden), dtype=torch.int16, device="cuda"), torch.zeros_like(rd)
    assert lib.ca_ffn_sum_hc_post(ctypes.c_void_p(ctx), rows, live, native.ptr(routes), native.ptr(shared), native.ptr(rd), native.ptr(pod),
                                  native.ptr(cd), native.ptr(routed), native.ptr(ffn), native.ptr(y), None) == 0
    torch.cuda.synchronize()
    want_routed, want_ffn = oracle.ffn_sum_shared(plain["route_out"], plain["shared_down"], live, previous=before)
    assert np.array_equal(np_of(routed).view(np.uint16), want_routed) and np.array_equal(np_of(ffn).view(np.uint16), want_ffn)
    assert np.array_equal(np_of(y).view(np.uint16), oracle.hc_post(want_ffn, r, post, comb))
    assert np.array_equal(want_ffn[:live], plain["out"][:live])
    layer.close()
    lib.ca_primitives_close(ctypes.c_void_p(ctx))


@pytest.mark.gpu
def test_the_layer_takes_the_producers_rows_and_the_residual_follows():
    # producer -> Layer.run_quantized (the layer skips its own quantizer: src/ffn.rs:974-975) -> sum + shared + residual in one
    # pass.  The layer's output from the producer's codes equals its output from the normalized BF16 rows (the producer's codes
    # are the layer's own quantizer's codes of those rows), and the fused residual equals the oracle's addition.
    from helpers import pkg
    g = geometry(1024, 16, 2, 512, 512, "benchmark")
    ops = synth.LayerOperands(g, "c1", device="cpu")
    rows = 8
    lib = native.load()
    ctx = native.open_context(g)
    x, w = norm_inputs(rows, g.hidden, "chain")
    x[2, :] = x[3, :]                                       # no zero row in the chain
    xd, wd = torch.from_numpy(x.view(np.int16)).cuda(), torch.from_numpy(w.view(np.int16)).cuda()
    normed = torch.zeros((rows, g.hidden), dtype=torch.int16, device="cuda")
    codes = torch.zeros((rows, g.hidden), dtype=torch.uint8, device="cuda")
    scales = torch.zeros((rows, g.hidden // g.act_block), dtype=torch.uint8, device="cuda")
    codes_min, scales_min = torch.zeros_like(codes), torch.zeros_like(scales)
    assert lib.ca_ffn_norm_quant(ctypes.c_void_p(ctx), rows, native.ptr(xd), native.ptr(wd), 1e-6, native.ptr(normed), native.ptr(codes),
                                 native.ptr(scales), native.ptr(codes_min), native.ptr(scales_min), None) == 0
    torch.cuda.synchronize()
    layer = pkg.host.Layer(g, ops, rows)
    layer.set_tokens()
    layer.run(normed)
    plain = layer.taps()
    layer.run_quantized(normed, codes_min, scales_min)
    fed = layer.taps()
    assert np.array_equal(fed["out"], plain["out"]) and np.array_equal(fed["route_out"], plain["route_out"])
    residual = torch.from_numpy(u16(synth.activations("chain/residual", rows, g.hidden)).view(np.int16)).cuda()
    routes = torch.from_numpy(plain["route_out"].view(np.int16)).cuda()
    shared = torch.from_numpy(plain["shared_down"].view(np.int16)).cuda()
    live = 6
    routed = torch.from_numpy(plain["routed"].view(np.int16)).cuda().clone()
    routed[live:] = 0x3c00                                  # rows past the live ones keep what the buffer holds
    before = np_of(routed).view(np.uint16).copy()
    ffn = torch.zeros_like(residual)
    after = torch.zeros_like(residual)
    assert lib.ca_ffn_sum_residual(ctypes.c_void_p(ctx), rows, live, native.ptr(routes), native.ptr(shared), native.ptr(residual), native.ptr(routed),
                                   native.ptr(ffn), native.ptr(after), None) == 0
    torch.cuda.synchronize()
    want_routed, want_ffn = oracle.ffn_sum_shared(plain["route_out"], plain["shared_down"], live, previous=before)
    assert np.array_equal(np_of(routed).view(np.uint16), want_routed) and np.array_equal(np_of(ffn).view(np.uint16), want_ffn)
    assert np.array_equal(np_of(after).view(np.uint16), oracle.residual_add(want_ffn, np_of(residual).view(np.uint16)))
    assert np.array_equal(want_ffn[:live], plain["out"][:live])
    # in place, without the intermediate
    assert lib.ca_ffn_sum_residual(ctypes.c_void_p(ctx), rows, live, native.ptr(routes), native.ptr(shared), native.ptr(residual), native.ptr(routed),
                                   None, native.ptr(residual), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(residual, after)
    layer.close()
    lib.ca_primitives_close(ctypes.c_void_p(ctx))
