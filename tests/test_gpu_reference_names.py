"""The kernels the reference resolves by name and launches with fixed argument lists (its own layer: hidden 5,120, 384
experts, top 6, a shared-expert shard of 576 columns), launched here exactly so: hipModuleGetFunction on the reference-layer
code object, hipModuleLaunchKernel with the reference's argument list, grid and block (src/ffn.rs:1041-1044, 1099-1102,
1228-1230; src/moe.rs:212-218, kernels/moe_frontend.cuh:154-266; src/blockscaled.rs:54, 375; src/mhc.rs:79), and checked
against the oracle."""
import ctypes
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import geometry, native, np_of, oracle_config, synth, u16

pytestmark = pytest.mark.gpu

H, E, K, IS, IS_PAD = 5120, 384, 6, 576, 640


class Module:
    def __init__(self, path):
        self.hip = ctypes.CDLL("libamdhip64.so")
        assert os.path.exists(path), "build the package first"
        torch.zeros(1, device="cuda")
        self.module = ctypes.c_void_p()
        assert self.hip.hipModuleLoad(ctypes.byref(self.module), path.encode()) == 0
        self.hip.hipModuleLaunchKernel.argtypes = [ctypes.c_void_p] + [ctypes.c_uint] * 7 + [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]

    def function(self, name):
        f = ctypes.c_void_p()
        assert self.hip.hipModuleGetFunction(ctypes.byref(f), self.module, name.encode()) == 0, name
        return f

    def launch(self, name, grid, block, args, shared=0):
        """args: tensors (pointers), None (null pointer), python ints (int32)."""
        held = []
        for a in args:
            if a is None:
                held.append(ctypes.c_void_p(0))
            elif isinstance(a, torch.Tensor):
                held.append(ctypes.c_void_p(a.data_ptr()))
            else:
                held.append(ctypes.c_int32(a))
        argv = (ctypes.c_void_p * len(held))(*[ctypes.cast(ctypes.pointer(h), ctypes.c_void_p) for h in held])
        gx, gy = grid if isinstance(grid, tuple) else (grid, 1)
        assert self.hip.hipModuleLaunchKernel(self.function(name), gx, gy, 1, block, 1, 1, shared, None, argv, None) == 0, name
        assert self.hip.hipDeviceSynchronize() == 0, name

    def close(self):
        assert self.hip.hipModuleUnload(self.module) == 0


@pytest.fixture(scope="module")
def module():
    m = Module(native.REFERENCE_LAYER_OBJECT)
    yield m
    m.close()


def test_every_name_resolves(module):
    for name in ["ca_ffn_sum_shared", "ca_shared_swiglu_quant128", "ca_shared_swiglu_quant64", "ca_shared_swiglu_quant16_64", "ca_moe_frontend",
                 "ca_moe_route_frontend", "ca_route_topk", "ca_tail_gate", "ca_block_scales_mma", "ca_pad_fp8_columns", "_router_triton_kernel",
                 "ca_moe_group_sum_rows", "hc_combine_norm_quant", "hc_post_tiles"]:
        module.function(name)


def test_ffn_sum_shared_six_arguments(module):
    rows, live = 6, 4
    routes = synth.activations("names/routes", rows * K, H).reshape(rows, K, H).cuda()
    shared = synth.activations("names/shared", rows, H).cuda()
    previous = synth.activations("names/previous", rows, H).cuda()
    routed, out = previous.clone(), torch.zeros_like(shared)
    n = rows * H
    module.launch("ca_ffn_sum_shared", (n + 127) // 128, 128, [routes, shared, routed, out, n, live])
    want_routed, want_out = oracle.ffn_sum_shared(u16(routes), u16(shared), live, previous=u16(previous))
    assert np.array_equal(u16(routed), want_routed) and np.array_equal(u16(out), want_out)
    assert np.array_equal(u16(routed)[live:], u16(previous)[live:])            # rows past the live ones keep the buffer's contents


@pytest.mark.parametrize("name,grid,block,rows", [("ca_shared_swiglu_quant128", 8, 128, 6), ("ca_shared_swiglu_quant16_64", 40, 64, 16),
                                                    ("ca_shared_swiglu_quant64", 8, 64, 3)])
def test_shared_swiglu_quant_of_the_576_column_shard(module, name, grid, block, rows):
    x = synth.normal("names/up", (rows, 2 * IS), std=3.0)
    x[0, :8] = 0.0                       # a block of zeros: floored scale
    x[1, 5] = 40.0                       # past the clamp
    xb = synth.to_bf16_bits(x).cuda()
    a = torch.zeros((rows, IS), dtype=torch.int16, device="cuda")
    q = torch.full((rows, IS_PAD), 0x55, dtype=torch.uint8, device="cuda")
    sr = torch.full((rows, IS_PAD // 32), 0x55, dtype=torch.uint8, device="cuda")
    sm = torch.full((5 * 512,), 0x55, dtype=torch.uint8, device="cuda")
    module.launch(name, grid, block, [xb, a, q, sr, sm, rows])
    act, aq, asc = oracle.shared_swiglu_quant(u16(xb), 32, 10.0)
    assert np.array_equal(u16(a), act)
    assert np.array_equal(np_of(q)[:, :IS], aq) and not np_of(q)[:, IS:].any()
    assert np.array_equal(np_of(sr)[:, :IS // 32], asc) and not np_of(sr)[:, IS // 32:].any()
    want_sm = np.full(5 * 512, 0x55, np.uint8)
    for row in range(rows):
        for block_index in range(IS_PAD // 32):
            want_sm[row * 16 + block_index % 4 + (block_index // 4) * 512] = np_of(sr)[row, block_index]
    assert np.array_equal(np_of(sm), want_sm)


def reference_inputs(rows):
    g = geometry(H, E, K, 2304, 2304, "reference")
    logits = synth.normal("names/logits", (rows, E), std=2.0)
    bias = synth.normal("names/bias", (E,), std=0.1)
    bias_alt = synth.normal("names/bias_alt", (E,), std=0.1)
    tokens = torch.arange(rows, dtype=torch.int64)
    tokens[1] = 129264
    return g, logits, bias, bias_alt, tokens


def test_route_topk_nine_arguments(module):
    rows, live = 16, 14
    g, logits, bias, bias_alt, tokens = reference_inputs(rows)
    padding = torch.full((rows,), -1, dtype=torch.int32)
    padding[15] = 2
    ids = torch.zeros((rows, K), dtype=torch.int32, device="cuda")
    weights = torch.zeros((rows, K), dtype=torch.float32, device="cuda")
    module.launch("ca_route_topk", 1, 512, [logits.cuda(), bias.cuda(), bias_alt.cuda(), tokens.cuda(), torch.tensor([live], dtype=torch.int32).cuda(),
                                           padding.cuda(), ids, weights, rows])
    want_ids, want_w = oracle.route_topk(oracle_config(g), logits.numpy(), bias.numpy(), bias_alt.numpy(), tokens.numpy(), live, padding.numpy())
    assert np.array_equal(np_of(ids), want_ids) and np.array_equal(np_of(weights).view(np.uint32), want_w.view(np.uint32))


def test_router_operator_symbol_with_the_operator_launchers_argument_list(module):
    # src/triton_ops.rs:129-166: one block a row, the manifest's eight arguments as 64-bit words plus two zero words
    rows, live = 6, 5
    g, logits, bias, bias_alt, tokens = reference_inputs(rows)
    ids = torch.zeros((rows, K), dtype=torch.int32, device="cuda")
    weights = torch.zeros((rows, K), dtype=torch.float32, device="cuda")
    tensors = [logits.cuda(), bias.cuda(), bias_alt.cuda(), tokens.cuda(), torch.tensor([live], dtype=torch.int32).cuda(), weights, ids]
    words = [ctypes.c_uint64(t.data_ptr()) for t in tensors] + [ctypes.c_uint64(rows), ctypes.c_uint64(0), ctypes.c_uint64(0)]
    argv = (ctypes.c_void_p * len(words))(*[ctypes.cast(ctypes.pointer(w), ctypes.c_void_p) for w in words])
    assert module.hip.hipModuleLaunchKernel(module.function("_router_triton_kernel"), rows, 1, 1, 128, 1, 1, 0, None, argv, None) == 0
    assert module.hip.hipDeviceSynchronize() == 0
    want_ids, want_w = oracle.route_topk(oracle_config(g), logits.numpy(), bias.numpy(), bias_alt.numpy(), tokens.numpy(), live)
    assert np.array_equal(np_of(ids), want_ids) and np.array_equal(np_of(weights).view(np.uint32), want_w.view(np.uint32))


def plan_buffers(rows, groups, tile_m):
    pairs = rows * K
    tiles = min(pairs, E + pairs // tile_m)
    d = "cuda"
    return dict(token_map=torch.full((tiles * tile_m,), -1, dtype=torch.int32, device=d), token_weights=torch.zeros(tiles * tile_m, device=d),
                task_expert=torch.full((tiles * groups,), -1, dtype=torch.int32, device=d),
                task_valid=torch.full((tiles * groups,), -1, dtype=torch.int32, device=d),
                base=torch.full((E + 1,), -1, dtype=torch.int32, device=d)), tiles


def check_plan(b, tiles, ids, weights, groups, tile_m):
    base, te, tv, tmap, tw = oracle.plan(ids, weights, E, groups, tile_m, capacity_tiles=tiles)
    assert np.array_equal(np_of(b["base"]), base)
    n = int(base[-1])
    assert np.array_equal(np_of(b["task_expert"])[:n * groups], te[:n * groups]) and np.array_equal(np_of(b["task_valid"])[:n * groups], tv[:n * groups])
    occupied = tmap >= 0
    assert np.array_equal(np_of(b["token_map"])[occupied], tmap[occupied])
    assert np.array_equal(np_of(b["token_weights"]).view(np.uint32)[occupied], tw.view(np.uint32)[occupied])


def test_moe_frontend_sixteen_arguments(module):
    rows, groups, tile_m = 6, 4, 16
    g, logits, bias, bias_alt, tokens = reference_inputs(rows)
    ids, weights = oracle.route_topk(oracle_config(g), logits.numpy(), bias.numpy(), bias_alt.numpy(), tokens.numpy(), rows)
    x = synth.activations("names/x", rows, H).cuda()
    packed = torch.zeros((rows, H), dtype=torch.uint8, device="cuda")
    scales = torch.zeros((rows, H // 32), dtype=torch.uint8, device="cuda")
    b, tiles = plan_buffers(rows, groups, tile_m)
    module.launch("ca_moe_frontend", 8, 512, [x, torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda(), packed, scales, b["token_map"],
                                              b["token_weights"], b["task_expert"], b["task_valid"], b["base"], rows, K, E, H, groups, tile_m])
    check_plan(b, tiles, ids, weights, groups, tile_m)
    codes, sc = oracle.quantize_rows(u16(x), 32, 0.0)
    assert np.array_equal(np_of(packed), codes) and np.array_equal(np_of(scales), sc)


def test_moe_route_frontend_twenty_three_arguments(module):
    owner_rows, rows, live, groups, tile_m = 8, 6, 5, 4, 16
    g, logits, bias, bias_alt, tokens = reference_inputs(owner_rows)
    padding = torch.full((owner_rows,), -1, dtype=torch.int32)
    padding[5] = 0
    x = synth.activations("names/x8", owner_rows, H).cuda()
    ids = torch.zeros((owner_rows, K), dtype=torch.int32, device="cuda")
    weights = torch.zeros((owner_rows, K), dtype=torch.float32, device="cuda")
    packed = torch.zeros((rows, H), dtype=torch.uint8, device="cuda")
    scales = torch.zeros((rows, H // 32), dtype=torch.uint8, device="cuda")
    b, tiles = plan_buffers(rows, groups, tile_m)
    module.launch("ca_moe_route_frontend", 9, 512,
                  [x, ids, weights, packed, scales, b["token_map"], b["token_weights"], b["task_expert"], b["task_valid"], b["base"], logits.cuda(),
                   bias.cuda(), bias_alt.cuda(), tokens.cuda(), torch.tensor([live], dtype=torch.int32).cuda(), padding.cuda(), rows, K, E, H, groups,
                   tile_m, owner_rows])
    want_ids, want_w = oracle.route_topk(oracle_config(g), logits.numpy(), bias.numpy(), bias_alt.numpy(), tokens.numpy(), live, padding.numpy())
    assert np.array_equal(np_of(ids), want_ids) and np.array_equal(np_of(weights).view(np.uint32), want_w.view(np.uint32))
    check_plan(b, tiles, want_ids[:rows], want_w[:rows], groups, tile_m)
    codes, sc = oracle.quantize_rows(u16(x)[:rows], 32, 0.0)
    assert np.array_equal(np_of(packed), codes) and np.array_equal(np_of(scales), sc)


def test_group_sum_rows_six_arguments(module):
    # kernels/ffn_sum_shared.cuh:35-58 as src/decoder.rs:1000-1008 launches it: one group of a sequence-parallel chunk's route sums,
    # laid out [destination rank][row of the group][5120]
    rows, groups = 32, 2
    quarter, per = rows // 4, rows // 4 // groups
    live = 27
    routes = synth.activations("names/group-routes", rows * K, H).reshape(rows, K, H).cuda()
    summed = oracle.topk_sum(u16(routes))
    for group in range(groups):
        out = torch.full((4, per, H), 0x3c00, dtype=torch.int16, device="cuda")
        threads = 4 * per * (H // 8)
        module.launch("ca_moe_group_sum_rows", (threads + 255) // 256, 256, [routes, out, quarter, per, group, live])
        got = u16(out)
        for c in range(4):
            for j in range(per):
                row = c * quarter + group * per + j
                if row < live:
                    assert np.array_equal(got[c, j], summed[row]), (group, c, j)
                else:
                    assert np.all(got[c, j] == 0x3c00)             # rows at or past the live count are not written


@pytest.mark.parametrize("rows,parts", [(6, 4), (16, 2), (128, 4)])
def test_boundary_producer_by_the_operator_launchers_list(module, rows, parts):
    # `hc_norm_quant_p4` / `_p2` (src/mhc.rs:606-614, 981-990): grid (rows, PARTS), 256 threads, X P W Y Q SR SM + the launcher's two
    # scratch words (src/triton_ops.rs:141-142)
    from test_boundary_steps import dev, hc_inputs
    x, pre, w = hc_inputs(rows, H, name="names/hc")
    y = torch.zeros((rows, H), dtype=torch.int16, device="cuda")
    q, sr = torch.zeros((rows, H), dtype=torch.uint8, device="cuda"), torch.zeros((rows, H // 32), dtype=torch.uint8, device="cuda")
    sm = torch.zeros(20480, dtype=torch.uint8, device="cuda")
    module.launch("hc_combine_norm_quant", (rows, parts), 256, [dev(x), dev(pre), dev(w), y, q, sr, sm, None, None])
    want_y, want_q, want_sr, want_sm = oracle.hc_combine_norm_quant(x, pre, w)
    assert np.array_equal(u16(y), want_y) and np.array_equal(np_of(q), want_q) and np.array_equal(np_of(sr), want_sr)
    assert np.array_equal(np_of(sm), want_sm)


def test_boundary_post_step_by_the_operator_launchers_list(module):
    # `hc_post_b128_w1` (src/mhc.rs:1223-1234): grid (rows, 40), A R POST C Y + two scratch words; any block
    from test_boundary_steps import dev, post_inputs
    rows = 6
    a, r, post, comb = post_inputs(rows, H, "names/post")
    want = oracle.hc_post(a, r, post, comb)
    for block in (32, 64, 256):
        y = torch.zeros((rows, 4, H), dtype=torch.int16, device="cuda")
        module.launch("hc_post_tiles", (rows, 40), block, [dev(a), dev(r), dev(post), dev(comb), y, None, None])
        assert np.array_equal(u16(y), want), block


def test_tail_gate_scale_spread_and_column_padding(module):
    module.launch("ca_tail_gate", 1, 32, [], shared=47 * 1024)
    n, k, padded_k = 200, 576, 640
    source = torch.randint(100, 140, (((n + 31) // 32), k // 32), dtype=torch.uint8, generator=torch.Generator().manual_seed(5))
    total = ((n + 127) // 128) * 128 * (padded_k // 32)
    out = torch.zeros(total, dtype=torch.uint8, device="cuda")
    module.launch("ca_block_scales_mma", (total + 255) // 256, 256, [source.cuda(), out, n, k, padded_k])
    want = np.full(total, 127, np.uint8)
    k_tiles = padded_k // 128
    for nt in range((n + 127) // 128):
        for kt in range(k_tiles):
            for rl in range(32):
                for rh in range(4):
                    for kg in range(4):
                        row, block = nt * 128 + rh * 32 + rl, kt * 4 + kg
                        if row < n and block < k // 32:
                            want[((nt * k_tiles + kt) * 32 + rl) * 16 + rh * 4 + kg] = source[row // 32, block]
    assert np.array_equal(np_of(out), want)
    weights = torch.randint(0, 255, (n, k), dtype=torch.uint8, generator=torch.Generator().manual_seed(6))
    padded = torch.full((n, padded_k), 0x55, dtype=torch.uint8, device="cuda")
    module.launch("ca_pad_fp8_columns", (n * padded_k + 255) // 256, 256, [weights.cuda(), padded, n, k, padded_k])
    assert np.array_equal(np_of(padded)[:, :k], weights.numpy()) and not np_of(padded)[:, k:].any()
