"""GPU parity of the C++ host mirror (LayerFfn / Router / Workspace / prepare_layer over the C ABI) against the CPU oracle,
in every schedule the reference has (dual-stream shared branch, fused or separate sum, top-k inside or before the
front-end), eager and as a replayed graph."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from helpers import pkg, synth
from test_gpu_layer import check_layer, make

pytestmark = pytest.mark.gpu
host = pkg.host


@pytest.mark.parametrize("overlap,sum_shared,route_front,fold", [(True, True, True, False), (False, False, False, False), (False, True, True, False),
                                                                  (True, False, False, False), (False, True, True, True), (True, True, False, True)])
def test_c1_schedules(overlap, sum_shared, route_front, fold):
    g, ops, x, rows = make("c1", "benchmark", "cpu")
    layer = host.Layer(g, ops, rows, overlap=overlap, sum_shared=sum_shared, route_front=route_front, fold_shared=fold)
    layer.set_tokens()
    layer.run(x.cuda())
    taps = layer.taps()
    if overlap and not fold:   # the branch quantized the input itself; the routed front-end emitted no shared-flavour codes
        taps["xq_min"], taps["xs_min"] = oracle.quantize_rows(x.numpy().view(np.uint16), g.act_block, 1e-4)
    check_layer(g, ops, x, taps)
    layer.close()


def test_reference_mode_tokens_live_padding_and_errors():
    g, ops, x, rows = make("c1", "reference", "cpu")
    layer = host.Layer(g, ops, rows, overlap=False)
    tokens = [5, 129264, 7, 129264, 1, 2, 3, 4]
    padding = [-1, -1, -1, -1, 0, 2, -1, -1]
    layer.set_tokens(tokens, live=4, padding=padding)
    layer.run(x.cuda())
    check_layer(g, ops, x, layer.taps(), tokens=tokens, live=4, padding=np.array(padding, np.int32), max_rel=2e-2)
    assert layer.census().sum() == 4 * g.topk
    with pytest.raises(host.HostError, match="padding route sources must name live rows"):
        layer.set_tokens(tokens, live=4, padding=[-1, -1, -1, -1, 6, -1, -1, -1])
    with pytest.raises(host.HostError, match="router token metadata domain"):
        layer.set_tokens([129280] * 8)
    layer.close()


def test_scale_code_and_prepared_layout_report():
    g, ops, x, rows = make("c1", "benchmark", "cpu")
    layer = host.Layer(g, ops, rows, code_scales=True)
    info = layer.info()
    E, H, I = g.experts, g.hidden, g.intermediate
    assert info["expert_bytes"] == E * (3 * H * I // 2 + 3 * H * I // 32)
    assert info["scale_code_bytes"] == oracle.scale_code1_layout(E, H, I)[5] * 4
    assert info["coded_rows"] == E * (2 * (I // 128) * (H // 128) + (H // 128) * (I // 128)) * 128 and info["raw_rows"] < info["coded_rows"]
    # the scratch arena has one size, whoever computes it: the host mirror, the library, the contract writer
    import ctypes
    from helpers import configure, native
    ctx = configure(g)
    contract = pkg.contracts.scratch_layout(dict(hidden=g.hidden, experts=g.experts, topk=g.topk, intermediate=g.intermediate,
                                                 act_block=g.act_block), rows)
    assert info["scratch_bytes"] == native.load().ca_primitives_scratch_bytes(ctx, 0, rows) == contract[1]
    assert info["max_tiles"] == contract[3] and info["tile_m"] == contract[2]
    layer.close()


@pytest.mark.parametrize("config", ["c2", "c3"])
def test_graph_replay_matches_eager_and_oracle(config):
    g, ops, x, rows = make(config, "benchmark", "cuda")
    layer = host.Layer(g, ops, rows)
    layer.set_tokens()
    xs = [x, synth.activations(config + "/second", rows, g.hidden, device="cuda")]
    graphs = [layer.capture(t) for t in xs]
    for which in (0, 1, 0):       # replays with other work between them must not see stale scratch
        layer.time([graphs[which]], 0, 1)
        taps = layer.taps()
        check_layer(g, ops, xs[which], taps)
        layer.run(xs[1 - which])
    layer.close()


def test_paired_owners_pool_into_one_launch():
    # Paired::run (src/paired_ffn.rs:65-120): two owners of one layer, different live prefixes; every owner's live rows must
    # come out exactly as when the owner runs alone (a row's arithmetic does not depend on which tile row it occupies)
    g, ops, xa, rows = make("c1", "reference", "cpu")
    xb = synth.activations("c1-paired-b", rows, g.hidden)
    tokens_a, tokens_b = [5, 129264, 7, 9, 1, 2, 3, 4], [11, 12, 129264, 14, 15, 16, 17, 18]
    live_a, live_b = 5, 3
    layer = host.Layer(g, ops, rows, overlap=False, sum_shared=False, route_front=False, fold_shared=False)
    alone = []
    for x, tokens, live in [(xa, tokens_a, live_a), (xb, tokens_b, live_b)]:
        layer.set_tokens(tokens, live=live)
        layer.run(x.cuda())
        alone.append(layer.tap("out").reshape(rows, g.hidden).copy())
    xa_d, xb_d = xa.cuda(), xb.cuda()
    out_a, out_b = layer.pair_run(xa_d, tokens_a, live_a, xb_d, tokens_b, live_b)
    assert np.array_equal(out_a[:live_a], alone[0][:live_a]), "owner A differs from its own run"
    assert np.array_equal(out_b[:live_b], alone[1][:live_b]), "owner B differs from its own run"
    # the shared expert once over the pooled rows (the reference pools the owners' shared up-projection, src/paired_ffn.rs:91-102):
    # the same bits again
    pool_a, pool_b = layer.pair_run(xa_d, tokens_a, live_a, xb_d, tokens_b, live_b, pool_shared=True)
    assert np.array_equal(pool_a[:live_a], alone[0][:live_a]) and np.array_equal(pool_b[:live_b], alone[1][:live_b]), "pooled shared expert"
    # and against the oracle, like any other schedule
    from helpers import assert_output_tolerance, oracle_layer
    want = oracle_layer(g, ops, xb, tokens_b, live_b)["out"]
    assert_output_tolerance("owner B's output", out_b[:live_b], want[:live_b], max_rel=2e-2, mean_abs=1e-3)
    with pytest.raises(host.HostError, match="paired FFN needs two live prefixes"):
        layer.pair_run(xa_d, tokens_a, 0, xb_d, tokens_b, live_b)
    layer.close()


@pytest.mark.parametrize("overlap", [False, True])
def test_prequantized_shared_input(overlap):
    # LayerFfn::run_quantized_input (src/ffn.rs:974-1047, 1053-1065): the boundary hands over the rows' codes in the shared
    # expert's quantizer flavour; the result is the one the layer computes when it quantizes the rows itself
    g, ops, x, rows = make("c1", "reference", "cpu")
    layer = host.Layer(g, ops, rows, overlap=overlap)
    layer.set_tokens()
    layer.run(x.cuda())
    want = layer.taps()
    codes, scales = oracle.quantize_rows(x.numpy().view(np.uint16), g.act_block, 1e-4)
    layer.run_quantized(x.cuda(), torch.from_numpy(codes).cuda(), torch.from_numpy(scales).cuda())
    got = layer.taps()
    for name in ["shared_up", "shared_act", "shared_down", "route_out", "out"]:
        assert np.array_equal(got[name], want[name]), name
    with pytest.raises(host.HostError, match="prequantized normalized shared input requires both operands"):
        layer.lib.tfh_layer_run_quantized.argtypes = None
        layer._check(layer.lib.tfh_layer_run_quantized(layer.h, ctypes.c_uint64(x.cuda().data_ptr()), ctypes.c_uint64(0), ctypes.c_uint64(0), layer._err, 512))
    layer.close()


def test_verify_rows_permutation_equivariance_through_the_folded_entry():
    # the 32 rows of the verify configuration in another order: every row's routes, routed sum and layer output are the same
    # bits (the rows share expert tiles in another arrangement, the shared expert's row tiles hold other rows)
    g, ops, x, rows = make("c3", "benchmark", "cuda")
    layer = host.Layer(g, ops, rows)
    layer.set_tokens()
    layer.run(x)
    first = layer.taps()
    perm = torch.randperm(rows, generator=torch.Generator().manual_seed(7))
    layer.run(x[perm.cuda()].contiguous())
    second = layer.taps()
    layer.close()
    order = perm.numpy()
    for name in ["ids", "weights", "xq", "xs", "route_out", "routed", "shared_down", "out"]:
        assert np.array_equal(np.ascontiguousarray(second[name]).view(np.uint8), np.ascontiguousarray(first[name][order]).view(np.uint8)), name
