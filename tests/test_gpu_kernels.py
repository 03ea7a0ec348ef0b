"""GPU parity of the individual kernels reached by name (ca_kernel_launch) and of the fixed-signature entry points."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import configure, geometry, native, np_of, oracle_config, synth, u16

pytestmark = pytest.mark.gpu


def dev(a, dtype=None):
    t = torch.as_tensor(a)
    if dtype is not None:
        t = t.view(dtype) if t.element_size() == torch.empty((), dtype=dtype).element_size() else t.to(dtype)
    return t.cuda().contiguous()


@pytest.mark.parametrize("hidden,experts", [(1024, 16), (4096, 256)])
@pytest.mark.parametrize("rows", [1, 3, 16])
def test_router_logits_bit_exact(hidden, experts, rows):
    g = geometry(hidden, experts, 2, 512, 512)
    configure(g)
    x = synth.activations("logits", rows, hidden)
    w = synth.to_bf16_bits(synth.normal("logits/w", (experts, hidden), std=hidden ** -0.5))
    out = torch.zeros((rows, experts), dtype=torch.float32, device="cuda")
    dx, dw = x.cuda(), w.cuda()
    st = native.load().ca_router_logits(rows, native.ptr(dx), native.ptr(dw), native.ptr(out), None)
    assert st == 0
    torch.cuda.synchronize()
    want = oracle.router_logits(u16(x), u16(w))
    assert np.array_equal(np_of(out).view(np.uint32), want.view(np.uint32))
    assert native.load().ca_router_logits(17, native.ptr(dx), native.ptr(dw), native.ptr(out), None) == -1
    assert native.load().ca_router_logits(0, native.ptr(dx), native.ptr(dw), native.ptr(out), None) == -1


def test_many_row_router_logits_both_tile_heights():
    # the many-row gate product runs 64-row workgroup tiles below 256 workgroups and 128-row tiles from there on; every logit is
    # the same sum in the same order either way: 32,805 rows (128-row tiles, ragged last tile) must hold, bit for bit, what its
    # first 1,000 rows give on their own (64-row tiles), and a sample of rows is held to the oracle's fixed-order product
    hidden, experts = 512, 320                     # two expert groups of 256: the second one ragged
    g = geometry(hidden, experts, 2, 512, 512)
    configure(g)
    rows = 32805
    x = synth.activations("logits-wide", rows, hidden).cuda()
    w = synth.to_bf16_bits(synth.normal("logits-wide/w", (experts, hidden), std=hidden ** -0.5)).cuda()
    lib = native.load()
    big = torch.full((rows, experts), float("nan"), dtype=torch.float32, device="cuda")
    small = torch.full((1000, experts), float("nan"), dtype=torch.float32, device="cuda")
    assert lib.ca_router_logits_wide(rows, native.ptr(x), native.ptr(w), native.ptr(big), None) == 0
    assert lib.ca_router_logits_wide(1000, native.ptr(x), native.ptr(w), native.ptr(small), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(big[:1000].view(torch.int32), small.view(torch.int32))
    assert not torch.isnan(big).any()
    sample = np.unique(np.concatenate([np.arange(0, rows, 1999), [63, 64, 127, 128, 999, rows - 38, rows - 37, rows - 1]]))
    want = oracle.router_logits(u16(x[torch.as_tensor(sample).cuda()].cpu()), u16(w.cpu()))
    got = np_of(big)[sample]
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max() + 1e-6


@pytest.mark.parametrize("mode,experts,topk", [("benchmark", 256, 6), ("reference", 384, 6), ("reference", 128, 3), ("benchmark", 16, 2)])
def test_route_topk_bit_exact(mode, experts, topk):
    g = geometry(1024, experts, topk, 512, 512, mode)
    cfg = oracle_config(g)
    rows = 40
    logits = synth.normal("topk/logits", (rows, experts), std=2.0)
    logits[3, 5] = float("nan")
    logits[4, :] = 0.25          # every score ties: lowest ids win, in order
    logits[5, 7] = 30.0          # past the softplus switch
    bias = synth.normal("topk/bias", (experts,), std=0.1)
    bias_alt = synth.normal("topk/bias_alt", (experts,), std=0.1)
    tokens = torch.arange(rows, dtype=torch.int64)
    tokens[2] = 129264
    live = 37
    ids = torch.zeros((rows, topk), dtype=torch.int32, device="cuda")
    weights = torch.zeros((rows, topk), dtype=torch.float32, device="cuda")
    native.launch("ca_route_topk", (rows + 15) // 16, 1024,
                  [logits.cuda(), bias.cuda(), bias_alt.cuda(), tokens.cuda(), torch.tensor([live], dtype=torch.int32).cuda(), None, ids,
                   weights, rows, experts, topk, g.scoring, float(g.route_scale), ctypes.c_int64(g.alt_token)])
    torch.cuda.synchronize()
    want_ids, want_w = oracle.route_topk(cfg, logits.numpy(), bias.numpy(), bias_alt.numpy(), tokens.numpy(), live)
    assert np.array_equal(np_of(ids), want_ids)
    assert np.array_equal(np_of(weights).view(np.uint32), want_w.view(np.uint32))
    # census of the routed slots of live rows
    counts = torch.zeros(experts, dtype=torch.int32, device="cuda")
    native.launch("ca_route_census", (rows * topk + 255) // 256, 256,
                  [ids, torch.tensor([live], dtype=torch.int32).cuda(), rows, topk, counts, experts])
    torch.cuda.synchronize()
    assert np.array_equal(np_of(counts).astype(np.uint32), oracle.route_census(want_ids, live, experts))


@pytest.mark.parametrize("rows,experts,topk,tile_m", [(4096, 256, 6, 128), (300, 16, 2, 16), (1000, 384, 6, 128)])
def test_wide_plan_bit_exact(rows, experts, topk, tile_m):
    rng = np.random.default_rng(7)
    # skewed routing: expert popularity ~ rank^-1.1, distinct ids per row, a few inactive routes
    p = np.arange(1, experts + 1, dtype=np.float64) ** -1.1
    p /= p.sum()
    ids = np.stack([rng.choice(experts, size=topk, replace=False, p=p) for _ in range(rows)]).astype(np.int32)
    ids[rows - 3:] = -1
    weights = rng.random((rows, topk), dtype=np.float32)
    pairs = rows * topk
    waves = (pairs + 63) // 64
    max_tiles = -(-pairs // tile_m) - 1 + min(experts, pairs)
    d_ids, d_w = dev(ids), dev(weights)
    wave_counts = torch.zeros(waves * experts, dtype=torch.int32, device="cuda")
    local_rank = torch.zeros(pairs, dtype=torch.int32, device="cuda")
    base = torch.full((experts + 1,), -1, dtype=torch.int32, device="cuda")
    te = torch.full((max_tiles,), -1, dtype=torch.int32, device="cuda")
    tv = torch.full((max_tiles,), -1, dtype=torch.int32, device="cuda")
    tmap = torch.full((max_tiles * tile_m,), -1, dtype=torch.int32, device="cuda")
    tw = torch.zeros(max_tiles * tile_m, dtype=torch.float32, device="cuda")
    native.launch("ca_plan_wave_counts", (waves + 3) // 4, 256, [d_ids, pairs, experts, wave_counts, local_rank])
    native.launch("ca_plan_scan", experts, 256, [wave_counts, waves, experts, base])
    native.launch("ca_plan_tiles", 1, 512, [experts, 1, tile_m, base, te, tv])
    native.launch("ca_plan_scatter", (pairs + 255) // 256, 256, [d_ids, d_w, wave_counts, local_rank, base, pairs, experts, tile_m, tmap, tw])
    torch.cuda.synchronize()
    want = oracle.plan(ids, weights, experts, 1, tile_m, capacity_tiles=max_tiles)
    for got, exp in zip([base, te, tv, tmap], want[:4]):
        assert np.array_equal(np_of(got), exp)
    assert np.array_equal(np_of(tw).view(np.uint32), want[4].view(np.uint32))


@pytest.mark.parametrize("block", [32, 128])
def test_quantize_rows_bit_exact_incl_edge_values(block):
    g = geometry(1024, 16, 2, 512, 512, "reference" if block == 32 else "benchmark")
    ctx = configure(g)
    rows, cols = 33, 1024
    x = synth.normal("quant/x", (rows, cols), std=1.0)
    x[0] = 0.0                       # zero blocks: scale byte 0 (routed) / floor 1e-4 (shared)
    x[1] *= 1e-6                     # tiny blocks
    x[2] *= 3e4                      # large blocks
    x[3, :64] = 448.0                # exactly representable maxima
    x[4, :32] = torch.tensor([2.0 ** -k for k in range(32)])
    x[5] *= 1e-30                    # blocks whose scale underflows towards denormals
    xb = synth.to_bf16_bits(x).cuda()
    outs = [torch.zeros((rows, cols), dtype=torch.uint8, device="cuda"), torch.zeros((rows, cols // block), dtype=torch.uint8, device="cuda"),
            torch.zeros((rows, cols), dtype=torch.uint8, device="cuda"), torch.zeros((rows, cols // block), dtype=torch.uint8, device="cuda")]
    st = native.primitives_launch(ctx, 3, [xb] + outs, [rows, cols, 0])
    assert st == 0
    torch.cuda.synchronize()
    for flavour, (codes, scales) in [(0.0, outs[:2]), (1e-4, outs[2:])]:
        wq, ws = oracle.quantize_rows(u16(xb), block, flavour)
        assert np.array_equal(np_of(codes), wq) and np.array_equal(np_of(scales), ws)


def test_shared_swiglu_and_add_entry_points():
    g = geometry(1024, 16, 2, 512, 512, "reference")
    configure(g)
    rows, inter = 6, 512
    x = synth.normal("swiglu/x", (rows, 2 * inter), std=4.0)
    x[0, :8] = torch.tensor([11.0, -11.0, 10.0, -10.0, 1e-3, 0.0, 50.0, -50.0])
    xb = synth.to_bf16_bits(x).cuda()
    act = torch.zeros((rows, inter), dtype=torch.int16, device="cuda")
    assert native.load().ca_shared_swiglu(rows, native.ptr(xb), native.ptr(act), None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(u16(act), oracle.shared_swiglu(u16(xb)))
    for block in (32, 128):
        act2 = torch.zeros_like(act)
        codes = torch.zeros((rows, inter), dtype=torch.uint8, device="cuda")
        scales = torch.zeros((rows, inter // block), dtype=torch.uint8, device="cuda")
        native.launch("ca_shared_swiglu_quant", 8, 256, [xb, act2, codes, scales, rows, inter, block, 10.0])
        torch.cuda.synchronize()
        wa, wq, ws = oracle.shared_swiglu_quant(u16(xb), block)
        assert np.array_equal(u16(act2), wa) and np.array_equal(np_of(codes), wq) and np.array_equal(np_of(scales), ws)
    a = synth.to_bf16_bits(synth.normal("add/a", (rows, 1024)))
    b = synth.to_bf16_bits(synth.normal("add/b", (rows, 1024)))
    a.view(-1)[:4] = torch.from_numpy(np.array([1, 0x8001, 0x0040, 0], np.uint16).view(np.int16))      # denormal inputs are flushed
    out = torch.zeros((rows, 1024), dtype=torch.int16, device="cuda")
    da, db = a.cuda(), b.cuda()
    assert native.load().ca_ffn_add(rows, native.ptr(da), native.ptr(db), native.ptr(out), None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(u16(out), oracle.ffn_add(u16(a), u16(b)))


def test_topk_sum_entry_takes_its_live_rows_from_active_m_alone():
    # entry 2 (moe.w4a16.topk_sum): rows below the scalar active_m are summed, the others keep the buffer's contents; the third
    # pointer is bound to the output buffer by the contracts (as the reference binds its node's spare pointers) and is never read
    # as a live count -- BF16 bits there must not change the result
    import ctypes
    from helpers import geometry
    g = geometry(1024, 16, 6, 512, 512, "benchmark")
    ctx = native.open_context(g)
    lib = native.load()
    rows, live = 8, 5
    routes = synth.to_bf16_bits(synth.normal("entry2/routes", (rows, g.topk, g.hidden))).cuda()
    out = torch.full((rows, g.hidden), 0x3c00, dtype=torch.int16, device="cuda")
    pointers = (ctypes.c_uint64 * 3)(routes.data_ptr(), out.data_ptr(), out.data_ptr())
    scalars = (ctypes.c_int32 * 3)(live, 0, 0)
    assert lib.ca_primitives_launch(ctypes.c_void_p(ctx), 2, pointers, 3, scalars, 3, None) == 0
    torch.cuda.synchronize()
    want = oracle.topk_sum(u16(routes), live=live, previous=np.full((rows, g.hidden), 0x3c00, np.uint16))
    assert np.array_equal(u16(out), want) and np.all(u16(out)[live:] == 0x3c00)
    pointers = (ctypes.c_uint64 * 3)(routes.data_ptr(), out.data_ptr(), 0)          # a null third pointer is as good
    scalars = (ctypes.c_int32 * 3)(rows, 0, 0)
    assert lib.ca_primitives_launch(ctypes.c_void_p(ctx), 2, pointers, 3, scalars, 3, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(u16(out), oracle.topk_sum(u16(routes)))
    lib.ca_primitives_close(ctypes.c_void_p(ctx))


def test_group_sum_rows_layout():
    hidden, topk, quarter, per, group, live = 1024, 6, 8, 4, 1, 27
    routes = synth.to_bf16_bits(synth.normal("group/routes", (32, topk, hidden)))
    out = torch.full((4, per, hidden), 0x7fc0, dtype=torch.int16, device="cuda")
    n = 4 * per * hidden // 8
    native.launch("ca_moe_group_sum_rows", (n + 255) // 256, 256, [routes.cuda(), out, quarter, per, group, live, topk, hidden])
    torch.cuda.synchronize()
    summed = oracle.topk_sum(u16(routes))
    got = u16(out)
    for c in range(4):
        for j in range(per):
            row = c * quarter + group * per + j
            if row < live:
                assert np.array_equal(got[c, j], summed[row])
            else:
                assert (got[c, j] == 0x7fc0).all()


def test_prepared_layouts_codes_and_permutation_round_trip():
    n, k = 256, 1024
    rng = np.random.default_rng(3)
    words = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    scales = rng.choice(np.array([118, 119, 119, 119, 120, 121, 131], np.uint8), (n, k // 32))
    fp8 = rng.integers(0, 256, (n, k), dtype=np.uint8)
    for kernel, inverse, src, want, unit in [
        ("ca_expert_compact_words", "ca_expert_expand_words", words, oracle.stream_words(words, n, k), 32),
        ("ca_expert_compact_scales", "ca_expert_expand_scales", scales, oracle.stream_scales(scales, n, k), 32)]:
        d_src = dev(src)
        d_dst = torch.zeros_like(d_src)
        total = n * (k // unit) if src is not scales else n * (k // 32)
        native.launch(kernel, (total + 255) // 256, 256, [d_src, d_dst, n, k, n])
        back = torch.zeros_like(d_src)
        native.launch(inverse, (total + 255) // 256, 256, [d_dst, back, n, k])
        torch.cuda.synchronize()
        assert np.array_equal(np_of(d_dst).ravel(), want.ravel()) and np.array_equal(np_of(back), src)
    d_src = dev(fp8)
    d_dst, back = torch.zeros_like(d_src), torch.zeros_like(d_src)
    total = n * (k // 16)
    native.launch("ca_dense_compact_fp8", (total + 255) // 256, 256, [d_src, d_dst, n, k, 0])
    native.launch("ca_dense_compact_fp8", (total + 255) // 256, 256, [d_dst, back, n, k, 1])
    torch.cuda.synchronize()
    assert np.array_equal(np_of(d_dst).ravel(), oracle.stream_fp8(fp8, n, k).ravel()) and np.array_equal(np_of(back), fp8)
    # nibble permutation entry point (involutive pair)
    w32 = rng.integers(0, 2 ** 32, 4096, dtype=np.uint32)
    d = dev(w32.view(np.int32))
    assert native.load().ca_moe_nibble_permute(native.ptr(d), w32.nbytes, 0, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(np_of(d).view(np.uint32), oracle.nibble_permute(w32))
    assert native.load().ca_moe_nibble_permute(native.ptr(d), w32.nbytes, 1, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(np_of(d).view(np.uint32), w32)
    assert native.load().ca_moe_nibble_permute(native.ptr(d), 6, 0, None) == -1
    # one-bit scale code on the prepared scale bytes + GPU self check + census
    # matrix 0, 1: the commonest byte is the base; matrix 2: the byte below the commonest is more common than the byte above and
    # becomes the base (kernels/expert_scale_codes.cuh:49-51)
    matrices, columns = 3, k // 32
    mixes = [[119, 119, 119, 120, 120, 117], [119, 119, 119, 120, 120, 117], [120, 120, 120, 119, 119, 117]]
    prepared = np.stack([oracle.stream_scales(rng.choice(np.array(mixes[m], np.uint8), (n, columns)), n, k) for m in range(matrices)])
    units = (n // 128) * (columns // 4)
    code = torch.zeros(matrices * units * 16, dtype=torch.int32, device="cuda")
    flags = torch.zeros(matrices * units * 4, dtype=torch.int32, device="cuda")
    bases = torch.zeros(matrices, dtype=torch.int32, device="cuda")
    error = torch.zeros(1, dtype=torch.int32, device="cuda")
    counts = torch.zeros(1, dtype=torch.int64, device="cuda")
    d_sc = dev(prepared)
    native.launch("ca_expert_scale_code1", matrices, 256, [d_sc, code, flags, bases, n, columns])
    native.launch("ca_expert_scale_code1_check", ((units * 128 + 255) // 256, matrices, 1), 256, [d_sc, code, flags, bases, error, n, columns])
    native.launch("ca_expert_scale_code1_census", (flags.numel() + 255) // 256, 256, [flags, counts, ctypes.c_size_t(flags.numel())])
    torch.cuda.synchronize()
    wc, wf, wb = oracle.scale_code1(prepared, matrices, n, columns)
    assert np.array_equal(np_of(code).view(np.uint32), wc) and np.array_equal(np_of(flags).view(np.uint32), wf)
    assert np.array_equal(np_of(bases).view(np.uint32), wb) and int(error.item()) == 0
    assert [int(v) & 255 for v in wb] == [119, 119, 119]
    err, raw_rows = oracle.scale_code1_check(prepared, wc, wf, wb, matrices, n, columns)
    assert err == 0 and raw_rows == int(counts.item()) and raw_rows > 0
    # four-bit row deltas
    plain = rng.choice(np.arange(112, 126, dtype=np.uint8), (matrices, n, columns))
    out4 = torch.zeros(matrices * n * columns, dtype=torch.uint8, device="cuda")
    error.zero_()
    native.launch("ca_expert_scale_codes4", ((n + 3) // 4, matrices, 1), 256, [dev(plain), out4, error, matrices, n, columns])
    torch.cuda.synchronize()
    want4, err4 = oracle.scale_codes4(plain, matrices, n, columns)
    assert err4 == 0 and int(error.item()) == 0 and np.array_equal(np_of(out4), want4)
    assert np.array_equal(oracle.scale_codes4_decode(np_of(out4), matrices, n, columns).reshape(plain.shape), plain)


def test_error_conventions():
    lib = native.load()
    g = geometry(1024, 16, 2, 512, 512)
    ctx = configure(g)
    assert lib.ca_ffn_abi() == 1 and lib.ca_primitives_abi() == 1
    assert native.primitives_launch(ctx, 99, [None], [0]) == -3
    assert native.primitives_launch(ctx, 2, [None, None], [0, 0, 0]) == -2
    assert native.primitives_launch(ctx, 2, [None, None, None], [1, 0, 0]) == -1
    bad = geometry(1000, 16, 2, 512, 512)
    assert lib.ca_ffn_configure(ctypes.byref(bad)) == -4
    # profiling marks: none, five or seven events
    dummy = (ctypes.c_void_p * 7)(*[1] * 7)
    assert lib.ca_primitives_marks(ctypes.c_void_p(ctx), dummy, 6) == -1
    dummy[6] = None
    assert lib.ca_primitives_marks(ctypes.c_void_p(ctx), dummy, 7) == -1
    assert lib.ca_primitives_marks(ctypes.c_void_p(ctx), None, 0) == 0
    with pytest.raises(RuntimeError):
        native.launch("no_such_kernel", 1, 64, [])


def test_code_object_loads_and_resolves_every_kernel_by_name():
    # the reference resolves its kernels by name from a code module (src/cuda.rs:199-226 Module::function / Function::launch);
    # the same names must resolve from titanic_moe_gfx950.hsaco through the HIP module interface, and a launch through it
    # must give the library's own result
    import ctypes
    import os
    hip = ctypes.CDLL("libamdhip64.so")
    assert os.path.exists(native.CODE_OBJECT), "build the package first (python -m __graft_entry__ or build.py)"
    torch.cuda.init()
    torch.zeros(1, device="cuda")
    module = ctypes.c_void_p()
    assert hip.hipModuleLoad(ctypes.byref(module), native.CODE_OBJECT.encode()) == 0
    lib = native.load()
    lib.ca_kernel_name.restype = ctypes.c_char_p
    functions = {}
    for i in range(lib.ca_kernel_count()):
        name = lib.ca_kernel_name(i)
        f = ctypes.c_void_p()
        assert hip.hipModuleGetFunction(ctypes.byref(f), module, name) == 0, name
        functions[name.decode()] = f
    assert {"ca_route_padding_rows", "ca_ffn_sum_shared", "ca_moe_frontend", "ca_moe_route_frontend", "ca_route_topk",
            "ca_expert_compact_words", "ca_expert_compact_scales", "ca_expert_scale_code1"} <= set(functions)
    n = 8 * 1024
    a = synth.activations("module/a", 8, 1024).cuda()
    b = synth.activations("module/b", 8, 1024).cuda()
    out = torch.zeros_like(a)
    args = (ctypes.c_void_p * 4)()
    held = [ctypes.c_void_p(a.data_ptr()), ctypes.c_void_p(b.data_ptr()), ctypes.c_void_p(out.data_ptr()), ctypes.c_longlong(n // 8)]
    for i, v in enumerate(held):
        args[i] = ctypes.cast(ctypes.pointer(v), ctypes.c_void_p)
    hip.hipModuleLaunchKernel.argtypes = [ctypes.c_void_p] + [ctypes.c_uint] * 7 + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    assert hip.hipModuleLaunchKernel(functions["ca_ffn_add_rows"], (n // 8 + 255) // 256, 1, 1, 256, 1, 1, 0, None, args, None) == 0
    assert hip.hipDeviceSynchronize() == 0
    want = oracle.ffn_add(u16(a), u16(b))
    assert np.array_equal(u16(out), want)
    assert hip.hipModuleUnload(module) == 0


def test_format_conversions_match_the_oracle_on_every_rounding_boundary():
    # every sign / exponent / leading-mantissa pattern with the low-bit patterns around each rounding boundary of both formats
    # (E4M3 keeps 3 mantissa bits, BF16 keeps 7), the saturation range of E4M3, specials, and a million random bit patterns
    hi = np.arange(1 << 16, dtype=np.uint32) << 16                       # sign, exponent, 7 mantissa bits
    lows = np.array([0, 1, 0x7fff, 0x8000, 0x8001, 0xffff], np.uint32)
    bits = [(hi[:, None] | lows[None, :]).ravel()]
    top = np.arange(1 << 12, dtype=np.uint32) << 20                      # sign, exponent, 3 mantissa bits
    low20 = np.array([0, 1, 0x7ffff, 0x80000, 0x80001, 0xfffff], np.uint32)
    bits.append((top[:, None] | low20[None, :]).ravel())
    around_448 = np.frombuffer(np.arange(440.0, 500.0, 0.125, dtype=np.float32).tobytes(), np.uint32)
    bits += [around_448, around_448 | np.uint32(0x80000000)]
    bits.append(np.random.default_rng(7).integers(0, 1 << 32, size=1 << 20, dtype=np.uint64).astype(np.uint32))
    bits = np.concatenate(bits)
    bits = bits[: len(bits) // 4 * 4]
    values = bits.view(np.float32)
    d_in = torch.from_numpy(values.copy()).cuda()
    d8 = torch.zeros(len(bits), dtype=torch.uint8, device="cuda")
    d16 = torch.zeros(len(bits), dtype=torch.int16, device="cuda")
    native.launch("ca_convert_formats", 1024, 256, [d_in, d8, d16, ctypes.c_int64(len(bits))])
    torch.cuda.synchronize()
    L = oracle.lib()
    want8 = np.array([L.orc_f32_to_e4m3(float(v)) if v == v else 0x7f for v in values[: 1 << 16]], np.uint8)
    assert np.array_equal(np_of(d8)[: 1 << 16], want8)
    # the whole set against numpy restatements of the two roundings (checked against the oracle on the first 65,536 above)
    def e4m3_np(u):
        sign, a = (u >> 24) & 0x80, u & 0x7fffffff
        normal = np.minimum(((a.astype(np.uint64) + 0x7ffff + ((a >> 20) & 1)) >> 20).astype(np.int64) - 960, 0x7e)
        tiny = (np.abs(u.view(np.float32)).astype(np.float32) + np.float32(24576.0)).view(np.uint32).astype(np.int64) - 0x46c00000
        q = np.where(a < 0x3c800000, tiny, normal)
        return np.where(a > 0x7f800000, 0x7f, sign | q).astype(np.uint8)
    def bf16_np(u):
        nan = (u & 0x7fffffff) > 0x7f800000
        r = ((u.astype(np.uint64) + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint32)
        return np.where(nan, (u >> 16) | 0x40, r).astype(np.uint16)
    assert np.array_equal(e4m3_np(bits[: 1 << 16]), want8)
    assert np.array_equal(np_of(d8), e4m3_np(bits))
    assert np.array_equal(np_of(d16).view(np.uint16), bf16_np(bits))
    want16 = np.array([L.orc_f32_to_bf16(float(v)) for v in values[: 1 << 16] if v == v], np.uint16)
    assert np.array_equal(np_of(d16).view(np.uint16)[: 1 << 16][values[: 1 << 16] == values[: 1 << 16]], want16)
