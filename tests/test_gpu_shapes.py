"""GPU parity over the shapes between and around the benchmark configurations, through the C++ host mirror: one row (the
reference's 1-row micro plan), the 64 / 65-row boundary between the streaming and the grouped-GEMM paths, every supported
contraction length class (multiples of 512 up to 4,096; token widths up to 8,192), top-1 and top-8, the reference's expert count, live prefixes and padding rows on the many-row path.
Same checks as the benchmark shapes (bit-exact routing, plan, codes; staged tolerance behind the matrix cores)."""
import numpy as np
import pytest

from helpers import geometry, pkg, synth
from test_gpu_layer import check_layer

pytestmark = pytest.mark.gpu
host = pkg.host


def run_case(rows, hidden, experts, topk, inter, shared, mode, live=None, padding=None, tokens=None, alt_token=None, **options):
    g = geometry(hidden, experts, topk, inter, shared, mode)
    if alt_token is not None:
        g.alt_token = alt_token
    name = "shape-%d-%d-%d-%d-%d-%d" % (rows, hidden, experts, topk, inter, shared)
    ops = synth.LayerOperands(g, name, device="cuda")
    x = synth.activations(name, rows, hidden)
    layer = host.Layer(g, ops, rows, **options)
    layer.set_tokens(tokens, live=live, padding=padding)
    layer.run(x.cuda())
    taps = layer.taps()
    # gate products of more than 16 rows run on the matrix cores (another summation order than the oracle's)
    stats = check_layer(g, ops, x, taps, tokens=tokens, live=live, padding=None if padding is None else np.array(padding, np.int32),
                        exact_logits=rows <= 16, max_rel=2e-2)
    layer.close()
    return taps, stats


@pytest.mark.parametrize("rows,hidden,experts,topk,inter,shared,mode", [
    (1, 512, 8, 2, 512, 512, "reference"),          # one row, the smallest contraction
    (1, 4096, 256, 6, 2048, 2048, "benchmark"),     # one row at the benchmark geometry
    (3, 4096, 16, 1, 2048, 2048, "benchmark"),      # top-1
    (16, 2048, 64, 8, 1024, 512, "benchmark"),      # top-8, H 2048 / I 1024, another shared width
    (6, 1024, 384, 6, 512, 1024, "reference"),      # the reference's expert count and row count
    (40, 2048, 64, 6, 1024, 1024, "reference"),     # three row tiles, the last partly filled: the shared expert's items take the rows' codes from the quantizer blocks of their launch
    (64, 1024, 32, 4, 512, 512, "reference"),       # the last row count of the streaming path
    (65, 1024, 32, 4, 512, 512, "benchmark"),       # the first of the grouped-GEMM path
    (130, 2048, 16, 2, 1024, 1024, "reference"),    # a second, partly filled row tile; K 1024 in FC2
    (64, 1024, 8, 8, 512, 512, "benchmark"),        # every row to every expert: four full 16-row tiles an expert, 512 routes in the one-block plan
    (200, 1024, 8, 8, 512, 512, "reference"),       # the same at many rows: two 128-row tiles an expert, the second partly filled
    (6, 5120, 32, 6, 2560, 2560, "reference"),      # the reference's token width (src/ffn.rs:65-66): eight-wave FC1 launch, five k-steps a wave
    (40, 5120, 64, 6, 1536, 512, "benchmark"),      # the same with three row tiles; K 1536 in FC2 (three k-steps a wave: scale words straddled)
    (130, 5120, 32, 2, 1024, 512, "reference"),     # many rows at that width: 160 activation scale bytes a row, staged in two passes
    (5, 1536, 16, 2, 3072, 3584, "benchmark"),      # three, six and seven k-steps a wave
    (70, 6144, 16, 2, 512, 512, "reference"),       # many rows, K 6,144
    (3, 8192, 8, 2, 1024, 1024, "benchmark"),       # the widest token row
    (130, 8192, 8, 2, 512, 512, "reference"),       # the same at many rows: 256 activation scale bytes a row, the table's capacity
    (4, 512, 512, 2, 512, 512, "reference"),        # as many experts as the plan block has threads: the tile total is written by the last expert's thread
    (600, 512, 512, 2, 512, 512, "benchmark"),      # the same through the many-route plan kernels
    (1100, 1024, 8, 2, 512, 512, "benchmark"),      # two plan tiles an expert and more: the grouped GEMM's 256-row units; FC2 with one round of k-steps
    (1100, 1024, 8, 2, 512, 512, "reference"),      # the same with 32-wide activation blocks
    (700, 2048, 4, 1, 1024, 512, "benchmark"),      # 256-row units whose last unit of an expert is a single, partly filled plan tile
])
def test_shape(rows, hidden, experts, topk, inter, shared, mode):
    run_case(rows, hidden, experts, topk, inter, shared, mode)


def test_one_live_row_of_a_wider_owner():
    taps, _ = run_case(8, 1024, 16, 2, 512, 512, "reference", live=1)
    assert (taps["ids"][1:] == -1).all() and not taps["weights"][1:].any()


@pytest.mark.parametrize("rows", [8, 40, 130])
def test_no_live_row(rows):
    # live = 0 (src/ffn.rs:121-126 admits it): no route is active, the plan has no tile, the expert launches have no item; the
    # routed output is zero and the layer output is the shared expert's rows past the live prefix as the oracle defines them
    taps, _ = run_case(rows, 1024, 16, 2, 512, 512, "reference", live=0)
    assert np.all(taps["ids"] < 0) or np.all(taps["ids"] >= 16)
    assert not np.any(taps["routed"] & 0x7fff)


def test_many_rows_with_a_live_prefix_and_padding_rows():
    rows = 200
    padding = [-1] * rows
    padding[150], padding[151] = 3, 7           # two padding rows repeat live rows' experts with zero weights
    taps, _ = run_case(rows, 1024, 16, 2, 512, 512, "benchmark", live=152, padding=padding, route_front=False)
    assert np.array_equal(taps["ids"][150], taps["ids"][3]) and np.array_equal(taps["ids"][151], taps["ids"][7])
    assert not taps["weights"][150:152].any() and (taps["ids"][152:] == -1).all()


def test_drafter_parameter_set():
    # the reference's drafter layers: 128 experts, top-3, no image-token bias (src/layer_id.rs:39-47): a row whose token id is
    # the main model's image token must be routed with the ordinary bias
    tokens = [129264, 1, 2, 3, 4, 5]
    taps, _ = run_case(6, 1024, 128, 3, 512, 512, "reference", tokens=tokens, alt_token=-1)
    again, _ = run_case(6, 1024, 128, 3, 512, 512, "reference", tokens=[7, 1, 2, 3, 4, 5], alt_token=-1)
    assert np.array_equal(taps["ids"], again["ids"]) and np.array_equal(taps["out"], again["out"])


@pytest.mark.parametrize("rows,experts,inter,shared", [(6, 16, 576, 576), (40, 8, 2304, 2304), (130, 8, 576, 2304)])
def test_reference_expert_widths_run_zero_padded(rows, experts, inter, shared):
    # the reference's expert widths (2,304; 576 a tensor-parallel rank: src/expert_packing.rs:64-66) are no multiples of 512:
    # the host mirror uploads them with zero weight rows / columns up to the next multiple and the layer runs at that width.
    # The oracle runs the unpadded operands; every tap must match on the real columns and be zero on the added ones.
    g = geometry(5120, experts, 6, inter, shared, "reference")
    name = "padded-%d-%d-%d-%d" % (rows, experts, inter, shared)
    ops = synth.LayerOperands(g, name, device="cuda")
    x = synth.activations(name, rows, g.hidden)
    layer = host.Layer(g, ops, rows)
    run = layer.run_geometry()
    assert (run.intermediate, run.shared_intermediate) == ((inter + 511) // 512 * 512, (shared + 511) // 512 * 512)
    layer.set_tokens()
    layer.run(x.cuda())
    taps = layer.taps()
    layer.close()
    B, I, S, Sp = g.act_block, inter, shared, run.shared_intermediate
    for key, width in (("h", I), ("hq", I), ("hs", I // B), ("shared_act", S), ("shared_aq", S), ("shared_as", S // B)):
        extra = taps[key][:, width:]
        if key in ("hs", "shared_as"):     # scale bytes of all-zero blocks: 0 (routed flavour), the 1e-4 floor's byte (shared flavour)
            assert np.all(extra == (0 if key == "hs" else 105)), key
        else:
            assert not np.any(extra & (0x7fff if extra.dtype == np.uint16 else 0x7f)), key
        taps[key] = np.ascontiguousarray(taps[key][:, :width])
    up = taps["shared_up"]
    assert not np.any(up[:, S:Sp] & 0x7fff) and not np.any(up[:, Sp + S:] & 0x7fff)
    taps["shared_up"] = np.ascontiguousarray(np.concatenate([up[:, :S], up[:, Sp:Sp + S]], axis=1))
    check_layer(g, ops, x, taps, exact_logits=rows <= 16, max_rel=2e-2)
