"""The steps either side of the layer at the decoder's FFN boundary (src/decoder.rs:1497-1543, 1654-1656; src/ffn.rs:974-975):
the RMS-norm + MXFP8 producer whose output the layer takes instead of quantizing itself, and the residual addition fused
behind the route sum and the shared addition.  The reference's own boundary operators are binaries, so parity with them is
unpinned; the oracle's definitions are pinned against float64 here (CPU), and the kernels against the oracle (GPU)."""
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
