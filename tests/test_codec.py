"""The wire row "dual_quant_rows_v1" (reference: runtime/kernels/moe-input-codec-coalesced-v1/moe-dual-quant-codec-fast.cu).

CPU part: pins the oracle's restatement against things other than its own formula -- the property the format exists for
(decode(pack(x)) is the shared quantizer's output, exactly, for every block), the rescaling step evaluated in exact
rational arithmetic over every code and scale, the documented row size (5,920 bytes for 5,120 columns:
runtime/kernels/moe-input-codec-coalesced-v1/manifest.json "numerical_contract"), hand-built rows.
GPU part: the C entry points (ca_pack_bf16, ca_encode, ca_decode, ca_local_live) against the oracle, bit for bit, at the
reference's row width among others, their argument checks, and the full-size property on the device.
"""
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle
from helpers import synth, u16


def e4m3_fraction(code):
    e, m = (code >> 3) & 15, code & 7
    v = Fraction(m, 512) if e == 0 else Fraction(8 + m, 8) * Fraction(2) ** (e - 7)
    return -v if code & 0x80 else v


FINITE = [c for c in range(256) if (c & 0x7f) != 0x7f]
GRID = sorted((e4m3_fraction(c), c) for c in range(0x7f))          # non-negative codes by value


def e4m3_round(value):
    """Round-to-nearest-even of an exact rational onto the E4M3 grid, saturating at 448 (the conversion the codec names)."""
    sign = 0x80 if value < 0 else 0
    a = abs(value)
    best = None
    for v, c in GRID:
        d = abs(v - a)
        if best is None or d < best[0] or (d == best[0] and (c & 1) == 0 and (best[1] & 1) == 1):
            best = (d, c)
    return sign | best[1]


def rows_with_small_blocks(tag, rows, k):
    """BF16 rows whose 32-wide blocks span ordinary, tiny (amax below the shared quantizer's floor of 1e-4), zero and
    mixed-sign cases."""
    x = synth.normal(tag, (rows, k), std=1.0).numpy().astype(np.float32).reshape(rows, k // 32, 32)
    kind = np.arange(rows * (k // 32)).reshape(rows, k // 32) % 7
    scale = np.select([kind == 0, kind == 1, kind == 2, kind == 3, kind == 4], [1.0, 3e-5, 2e-6, 1e-7, 9e-5], default=4e-5)
    x = x * scale[:, :, None]
    x[kind == 6] = 0.0
    x[0, 0, :] = -0.0
    return u16(synth.to_bf16_bits(torch.from_numpy(x.reshape(rows, k))))


def test_row_size_matches_the_reference_manifest():
    assert oracle.codec_row_bytes(5120) == 5920 == 5120 * 37 // 32
    x = rows_with_small_blocks("codec/size", 2, 5120)
    assert oracle.codec_pack_bf16(x).shape == (2, 5920)


def test_rescaled_code_matches_exact_arithmetic_for_every_code_and_scale():
    # one row; per scale byte below the floor eight blocks holding every finite code: with the expected shared codes every
    # correction word must be zero, with any other code every bit must be set
    scales = list(range(0, 105))
    codes = np.array(FINITE + [0, 0], dtype=np.uint8)                      # 256 = eight blocks
    routed = np.tile(codes, len(scales)).reshape(1, -1)
    k = routed.shape[1]
    assert k % 128 == 0
    groups = k // 32
    row_scales = np.repeat(np.array(scales, np.uint8), 8).reshape(1, -1)
    want = np.zeros_like(routed)
    for i, s in enumerate(scales):
        for j, c in enumerate(codes):
            c = int(c)
            want[0, i * 256 + j] = (c & 0x80) | e4m3_round(abs(e4m3_fraction(c)) * Fraction(2) ** (s - 105))
    packed = oracle.codec_encode(routed, row_scales, want)
    assert not packed[0, k + groups:].any()
    assert np.array_equal(packed[0, :k], routed[0]) and np.array_equal(packed[0, k:k + groups], row_scales[0])
    other = oracle.codec_encode(routed, row_scales, want ^ 1)
    assert (np.ascontiguousarray(other[0, k + groups:]).view(np.uint32) == 0xffffffff).all()
    # blocks at or above the floor carry no correction whatever the shared codes say
    high = oracle.codec_encode(routed, np.full_like(row_scales, 105), want ^ 1)
    assert not high[0, k + groups:].any()


def test_correction_steps_towards_the_rescaled_magnitude():
    # hand-built row: 0x09 (1.125 * 2^-6) under scale 104 rescales to 9 * 2^-10 = 4.5 * 2^-9: a tie between codes 4 and 5,
    # rounded to even (4); with the bit set the decoder must move up to 5 (|scaled| > |value(4)|).
    k = 128
    groups = k // 32
    row = np.zeros(oracle.codec_row_bytes(k), np.uint8)
    row[0] = 0x09
    row[1] = 0x89          # the same, negative: 0x84 -> 0x85
    row[2] = 0x0b          # 11 * 2^-10 = 5.5 * 2^-9: tie between 5 and 6 -> 6; bit set: |scaled| < |value(6)| -> 5
    row[k:k + groups] = [104, 127, 127, 127]
    row[k + groups: k + groups + 4] = [0b111, 0, 0, 0]
    shared, scales = oracle.codec_decode(row.reshape(1, -1), k)
    assert list(shared[0, :4]) == [5, 0x85, 5, 0]
    assert list(scales[0]) == [105, 127, 127, 127]
    row[k + groups] = 0
    shared, _ = oracle.codec_decode(row.reshape(1, -1), k)
    assert list(shared[0, :4]) == [4, 0x84, 6, 0]
    # correction words are little-endian: bit 9 of block 1 is bit 1 of that word's second byte
    routed = np.zeros((1, k), np.uint8)
    routed[0, 32 + 9] = 0x09
    want = routed.copy()
    want[0, 32 + 9] = 5
    packed = oracle.codec_encode(routed, np.array([[127, 104, 127, 127]], np.uint8), want)
    assert list(packed[0, k + groups + 4: k + groups + 8]) == [0, 0x02, 0, 0]


@pytest.mark.parametrize("rows,k", [(96, 128), (24, 1024), (6, 5120)])
def test_decode_of_pack_is_the_shared_quantizer(rows, k):
    x = rows_with_small_blocks("codec/roundtrip/%d" % k, rows, k)
    packed = oracle.codec_pack_bf16(x)
    routed_codes, routed_scales = oracle.quantize_rows(x, 32, 0.0)
    shared_codes, shared_scales = oracle.quantize_rows(x, 32, 1e-4)
    groups = k // 32
    assert np.array_equal(packed[:, :k], routed_codes) and np.array_equal(packed[:, k:k + groups], routed_scales)
    words = np.ascontiguousarray(packed[:, k + groups:]).view(np.uint32)
    assert words.any(), "the inputs must exercise the correction path"
    assert not words[routed_scales >= 105].any()
    got_codes, got_scales = oracle.codec_decode(packed, k)
    assert np.array_equal(got_scales, shared_scales)
    assert np.array_equal(got_codes, shared_codes)


def test_mma_scale_offsets_are_a_permutation_of_the_row_major_scales():
    rows, k = 256, 512
    x = rows_with_small_blocks("codec/mma", rows, k)
    packed = oracle.codec_pack_bf16(x)
    _, row_scales, mma = oracle.codec_decode(packed, k, mma=True)
    groups = k // 32
    # the reference's layout: 128-row panels, inside a panel 512 bytes per four scale columns, 16 bytes per row of a
    # 32-row band, 4 bytes per band (moe-dual-quant-codec-fast.cu:69-74)
    panel = mma.reshape(rows // 128, groups // 4, 32, 4, 4)          # [panel][col / 4][row % 32][row / 32 % 4][col % 4]
    back = panel.transpose(0, 3, 2, 1, 4).reshape(rows, groups)
    assert np.array_equal(back, row_scales)


def test_local_live_rows_of_a_sharded_batch():
    assert [oracle.codec_local_live(10, 4, r) for r in range(4)] == [4, 4, 2, 0]
    assert [oracle.codec_local_live(0, 4, r) for r in range(4)] == [0, 0, 0, 0]
    assert [oracle.codec_local_live(99, 4, r) for r in range(4)] == [4, 4, 4, 4]


# ---- GPU ------------------------------------------------------------------------------------------------------------
def _native():
    from helpers import native
    return native


def _np(t):
    return t.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,k", [(128, 128), (256, 1024), (128, 5120), (384, 4096)])
def test_gpu_codec_matches_oracle_bit_for_bit(rows, k):
    native = _native()
    lib = native.load()
    x = rows_with_small_blocks("codec/gpu/%d/%d" % (rows, k), rows, k)
    dx = torch.from_numpy(x.view(np.int16)).cuda()
    stride, groups = oracle.codec_row_bytes(k), k // 32
    packed = torch.zeros((rows, stride), dtype=torch.uint8, device="cuda")
    print("ca_pack_bf16", rows, k, flush=True)
    assert lib.ca_pack_bf16(native.ptr(dx), native.ptr(packed), rows, k, None) == 0
    torch.cuda.synchronize()
    want = oracle.codec_pack_bf16(x)
    assert np.array_equal(_np(packed), want)
    # the encoder from the two quantizers' separate outputs
    routed_codes, routed_scales = oracle.quantize_rows(x, 32, 0.0)
    shared_codes, shared_scales = oracle.quantize_rows(x, 32, 1e-4)
    packed2 = torch.zeros_like(packed)
    print("ca_encode", rows, k, flush=True)
    assert lib.ca_encode(native.ptr(torch.from_numpy(routed_codes).cuda()), native.ptr(torch.from_numpy(routed_scales).cuda()),
                         native.ptr(torch.from_numpy(shared_codes).cuda()), native.ptr(packed2), rows, k, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(_np(packed2), want)
    # the decoder
    shared = torch.zeros((rows, k), dtype=torch.uint8, device="cuda")
    scales = torch.zeros((rows, groups), dtype=torch.uint8, device="cuda")
    mma = torch.zeros(rows * groups, dtype=torch.uint8, device="cuda")
    print("ca_decode", rows, k, flush=True)
    assert lib.ca_decode(native.ptr(packed), native.ptr(shared), native.ptr(scales), native.ptr(mma), rows, k, None) == 0
    torch.cuda.synchronize()
    want_codes, want_scales, want_mma = oracle.codec_decode(want, k, mma=True)
    assert np.array_equal(_np(shared), want_codes) and np.array_equal(_np(shared), shared_codes)
    assert np.array_equal(_np(scales), want_scales) and np.array_equal(_np(mma), want_mma)
    shared.zero_()
    assert lib.ca_decode(native.ptr(packed), native.ptr(shared), native.ptr(scales), None, rows, k, None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(_np(shared), want_codes)


@pytest.mark.gpu
def test_gpu_codec_argument_checks_and_local_live():
    native = _native()
    lib = native.load()
    a = torch.zeros(128 * 160, dtype=torch.uint8, device="cuda")
    p = native.ptr(a)
    assert lib.ca_pack_bf16(p, p, 0, 128, None) == -1 and lib.ca_pack_bf16(p, p, 1, 96, None) == -1 and lib.ca_pack_bf16(None, p, 1, 128, None) == -1
    assert lib.ca_encode(p, p, p, p, 1, 64, None) == -1 and lib.ca_encode(p, p, p, p, -1, 128, None) == -1
    assert lib.ca_decode(p, p, p, p, 64, 128, None) == -1 and lib.ca_decode(p, p, p, p, 128, 100, None) == -1
    glob = torch.tensor([10], dtype=torch.int32, device="cuda")
    local = torch.zeros(4, dtype=torch.int32, device="cuda")
    for rank in range(4):
        assert lib.ca_local_live(native.ptr(glob), native.ptr(local[rank:]), 4, rank, None) == 0
    torch.cuda.synchronize()
    assert local.tolist() == [4, 4, 2, 0]
    assert lib.ca_local_live(native.ptr(glob), native.ptr(local), 4, 4, None) == -1 and lib.ca_local_live(native.ptr(glob), native.ptr(local), 0, 0, None) == -1


@pytest.mark.gpu
def test_gpu_codec_full_size_round_trip_is_the_shared_quantizer():
    """16,384 rows of 5,120 columns (a prefill chunk at the reference's width), checked on the device: routed codes and scales sit in
    the row as the routed quantizer kernel writes them, and decode returns the shared quantizer kernel's codes and scales."""
    native = _native()
    lib = native.load()
    rows, k = 16384, 5120
    gen = torch.Generator(device="cuda").manual_seed(20261125)
    x = torch.randn((rows, k), generator=gen, device="cuda", dtype=torch.float32)
    kind = (torch.arange(rows * (k // 32), device="cuda") % 5).reshape(rows, k // 32, 1)
    x = (x.reshape(rows, k // 32, 32) * torch.where(kind == 0, 1.0, torch.where(kind == 1, 3e-5, torch.where(kind == 2, 1e-6, torch.where(kind == 3, 0.0, 8e-5))))).reshape(rows, k).to(torch.bfloat16)
    groups, stride = k // 32, oracle.codec_row_bytes(k)
    packed = torch.zeros((rows, stride), dtype=torch.uint8, device="cuda")
    assert lib.ca_pack_bf16(native.ptr(x), native.ptr(packed), rows, k, None) == 0
    codes = [torch.zeros((rows, k), dtype=torch.uint8, device="cuda") for _ in range(3)]
    scales = [torch.zeros((rows, groups), dtype=torch.uint8, device="cuda") for _ in range(3)]
    native.launch("ca_quantize_rows", 4096, 256, [x, codes[0], scales[0], codes[1], scales[1], ctypes_i64(rows), k, 32])
    assert lib.ca_decode(native.ptr(packed), native.ptr(codes[2]), native.ptr(scales[2]), None, rows, k, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(packed[:, :k], codes[0]) and torch.equal(packed[:, k:k + groups], scales[0])
    assert torch.equal(codes[2], codes[1]) and torch.equal(scales[2], scales[1])
    assert int(packed[:, k + groups:].max()) > 0


def ctypes_i64(v):
    import ctypes
    return ctypes.c_int64(v)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,hidden", [(128, 1024), (512, 1024), (128, 5120)])
def test_gpu_row_transport_pass_equals_the_ordinary_pass(rows, hidden):
    """The one-rank row transport (pack -> routed experts from the wire rows, shared expert from the decoded codes) must give the
    ordinary pass's output bit for bit: both quantizers are reproduced exactly, everything downstream is the same kernels.
    Reference numerics (32-wide blocks), the small parity geometry at many rows (grouped-GEMM regime), and the reference's
    token width (wire rows of 5,920 bytes: src/moe.rs:512-583)."""
    from helpers import geometry, pkg, synth
    from test_gpu_layer import check_layer, make
    host = pkg.host
    if hidden == 1024:
        g, ops, x, rows = make("c1", "reference", "cuda", rows=rows, seed_name="codec/transport/%d" % rows)
    else:
        g = geometry(hidden, 16, 6, 512, 512, "reference")
        ops = synth.LayerOperands(g, "codec/transport/wide", device="cuda")
        x = synth.activations("codec/transport/wide", rows, hidden, device="cuda")
        assert oracle.codec_row_bytes(hidden) == 5920
    layer = host.Layer(g, ops, rows, overlap=False, sum_shared=False)
    layer.set_tokens()
    print("ordinary pass", rows, flush=True)
    layer.run(x)
    want = layer.taps()
    check_layer(g, ops, x, want, exact_logits=False, max_rel=2e-2)
    stride = oracle.codec_row_bytes(g.hidden)
    packed = torch.zeros((rows, stride), dtype=torch.uint8, device="cuda")
    print("row transport pass", rows, flush=True)
    layer.run_row_transport(x, packed)
    got = layer.taps()
    assert np.array_equal(packed.cpu().numpy(), oracle.codec_pack_bf16(u16(x.cpu())))
    for name in ["ids", "weights", "xq", "xs", "token_map", "hq", "hs", "route_out", "routed", "shared_aq", "shared_as", "shared_down", "out"]:
        assert np.array_equal(np.ascontiguousarray(got[name]).view(np.uint8), np.ascontiguousarray(want[name]).view(np.uint8)), name
    layer.close()
    # a geometry with 128-wide blocks has no wire row
    g2, ops2, x2, _ = make("c1", "benchmark", "cuda", rows=128)
    other = host.Layer(g2, ops2, 128, overlap=False)
    other.set_tokens()
    with pytest.raises(host.HostError, match="packed MoE transport requires the wide sequential profile"):
        other.run_row_transport(x2)
    other.close()
