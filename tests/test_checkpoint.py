"""The host mirror's safetensors scanner and layer-operand loader (src/checkpoint.rs:104-215, src/layout.rs:247-275,
src/weights.rs:276-356, 538-542): operands written with the reference's tensor names come back in the atlas order, and
every malformed checkpoint the reference rejects is rejected with the reference's reason.  CPU only, except the last test."""
import json
import os

import numpy as np
import pytest
import torch

from helpers import geometry, pkg, synth, u16

host = pkg.host


@pytest.fixture(scope="module")
def written(tmp_path_factory):
    g = geometry(512, 4, 2, 512, 512, "reference")
    ops = synth.LayerOperands(g, "checkpoint", device="cpu")
    root = str(tmp_path_factory.mktemp("checkpoint"))
    synth.write_checkpoint(ops, root, prefix="layers.3", shards=3)
    return g, ops, root


def test_operands_come_back_in_atlas_order(written):
    g, ops, root = written
    arrays, tensors, shards = host.checkpoint_layer(g, root, "layers.3")
    assert tensors == 6 * g.experts + 9 and shards == 3
    assert np.array_equal(arrays["gate_w"], u16(ops.gate_w))
    for name in ["bias", "bias_alt", "w13", "s13", "w2", "s2", "sh_w13", "sh_s13", "sh_w2", "sh_s2"]:
        assert np.array_equal(arrays[name], getattr(ops, name).numpy()), name      # up before gate (routed), gate before up (shared)


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layout_names.json")


def table_from_fixture(prefix, hidden, experts, width):
    """The reference's name table (tests/golden/layout_names.json, read out of src/layout.rs:247-275) for a layer of these
    dimensions: {(name, dtype, shape)}."""
    f = json.load(open(GOLDEN))
    dims = {"H": hidden, "E": experts, "I": width}

    def shape(entry):
        out = []
        for d in entry["dims"]:
            head, _, div = d.partition("/")
            out.append((dims[head] if head in dims else int(head)) // (int(div) if div else 1))
        return tuple(out)
    rows = set()
    for entry in f["per_expert"]:
        for e in range(experts):
            rows.add((entry["name"].replace("{p}", prefix).replace("{e}", str(e)), entry["dtype"], shape(entry)))
    for entry in f["per_layer"]:
        rows.add((entry["name"].replace("{p}", prefix), entry["dtype"], shape(entry)))
    return f, rows


def test_the_loader_requires_exactly_the_references_name_table():
    # the reference's own model: hidden 5120, 384 experts, the unpadded expert width 2304, 32 x 32 shared weight blocks
    f, want = table_from_fixture("layers.17", 5120, 384, 2304)
    assert (f["hidden"], f["experts"], f["expert_width"]) == (5120, 384, 2304)
    for entry in f["per_expert"] + f["per_layer"]:        # the symbolic shapes reproduce the numbers read from the reference
        assert tuple(entry["shape"]) == next(s for n, d, s in want if n == entry["name"].replace("{p}", "layers.17").replace("{e}", "0")), entry
    g = geometry(5120, 384, 6, 2304, 2304, "reference")
    got = host.checkpoint_contract(g, "layers.17")
    assert len(got) == len(set(got)) == 6 * 384 + 9
    assert set(got) == want
    # and a small layer's table, the one the tests below write and load
    g = geometry(512, 4, 2, 512, 512, "reference")
    assert set(host.checkpoint_contract(g, "layers.3")) == table_from_fixture("layers.3", 512, 4, 512)[1]


def test_every_tensor_of_the_table_is_required_and_no_other_is_read(written, tmp_path):
    g, ops, root = written
    _, table = table_from_fixture("layers.3", 512, 4, 512)
    index = json.load(open(os.path.join(root, "model.safetensors.index.json")))
    assert set(index["weight_map"]) == {name for name, _, _ in table}       # the writer follows the same table
    # dropping any one kind of tensor from the index and its shard header is noticed by name
    for victim in ["layers.3.ffn.experts.2.w3.scale", "layers.3.ffn.shared_experts.w2.scale", "layers.3.ffn.gate.bias_vl"]:
        bad = copy_of(root, tmp_path / victim.replace(".", "_"))
        path = os.path.join(bad, "model.safetensors.index.json")
        idx = json.load(open(path))
        shard = idx["weight_map"].pop(victim)
        json.dump(idx, open(path, "w"))
        def drop(header, body, victim=victim):
            header.pop(victim)
            return header, body
        rewrite(bad, shard, drop)
        with pytest.raises(host.HostError, match="missing tensor " + victim.replace(".", r"\.") + "|unindexed|hole|gap|disagree"):
            host.checkpoint_layer(g, bad, "layers.3")
    # a wrong dtype for a tensor of the right byte size
    bad = copy_of(root, tmp_path / "dtype")
    victim = "layers.3.ffn.experts.1.w2.weight"
    shard = index["weight_map"][victim]
    def retype(header, body):
        header[victim]["dtype"] = "F8_E4M3"
        return header, body
    rewrite(bad, shard, retype)
    with pytest.raises(host.HostError, match="tensor contract mismatch: " + victim):
        host.checkpoint_layer(g, bad, "layers.3")


def rewrite(root, shard, edit):
    path = os.path.join(root, shard)
    data = open(path, "rb").read()
    n = int.from_bytes(data[:8], "little")
    header = json.loads(data[8:8 + n])
    body = data[8 + n:]
    header, body = edit(header, body)
    text = json.dumps(header).encode()
    open(path, "wb").write(len(text).to_bytes(8, "little") + text + body)


def copy_of(root, tmp_path):
    import shutil
    target = str(tmp_path / "copy")
    shutil.copytree(root, target)
    return target


def first_shard(root):
    return sorted(f for f in os.listdir(root) if f.endswith(".safetensors"))[0]


def test_rejections(written, tmp_path):
    g, ops, root = written
    with pytest.raises(host.HostError, match="missing tensor layers.4"):
        host.checkpoint_layer(g, root, "layers.4")
    wrong = geometry(512, 4, 2, 1024, 512, "reference")
    with pytest.raises(host.HostError, match="tensor contract mismatch"):
        host.checkpoint_layer(wrong, root, "layers.3")

    bad = copy_of(root, tmp_path / "a")
    def hole(header, body):
        key = next(k for k in header if k != "__metadata__" and header[k]["data_offsets"][0] > 0)
        header[key]["shape"][0] -= 1                      # fewer bytes than the offsets say
        return header, body
    rewrite(bad, first_shard(bad), hole)
    with pytest.raises(host.HostError, match="tensor bytes disagree with its shape"):
        host.checkpoint_layer(g, bad, "layers.3")

    bad = copy_of(root, tmp_path / "b")
    rewrite(bad, first_shard(bad), lambda header, body: (header, body + b"\0" * 16))
    with pytest.raises(host.HostError, match="unindexed trailing data"):
        host.checkpoint_layer(g, bad, "layers.3")

    bad = copy_of(root, tmp_path / "c")
    def stranger(header, body):
        header["layers.3.unlisted"] = {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}
        return header, body
    rewrite(bad, first_shard(bad), stranger)
    with pytest.raises(host.HostError, match="index/header disagreement"):
        host.checkpoint_layer(g, bad, "layers.3")

    bad = copy_of(root, tmp_path / "d")
    index = json.load(open(os.path.join(bad, "model.safetensors.index.json")))
    key = next(iter(index["weight_map"]))
    index["weight_map"][key] = "../escape.safetensors"
    json.dump(index, open(os.path.join(bad, "model.safetensors.index.json"), "w"))
    with pytest.raises(host.HostError, match="unsafe shard file name"):
        host.checkpoint_layer(g, bad, "layers.3")

    bad = copy_of(root, tmp_path / "e")
    path = os.path.join(bad, first_shard(bad))
    data = open(path, "rb").read()
    open(path, "wb").write((1 << 40).to_bytes(8, "little") + data[8:])
    with pytest.raises(host.HostError, match="invalid header size"):
        host.checkpoint_layer(g, bad, "layers.3")


def test_expert_scale_bytes_past_the_lossless_range_are_refused(tmp_path):
    g = geometry(512, 4, 2, 512, 512, "reference")
    ops = synth.LayerOperands(g, "checkpoint", device="cpu")
    ops.s2[2, 5, 1] = 248                                  # src/weights.rs:538-542: bytes above 247 cannot be coded losslessly
    root = str(tmp_path / "scales")
    synth.write_checkpoint(ops, root, prefix="layers.0", shards=1)
    with pytest.raises(host.HostError, match="canonical expert scale exceeds lossless conversion range: layers.0.ffn.experts.2.w2.scale"):
        host.checkpoint_layer(g, root, "layers.0")


@pytest.mark.gpu
def test_layer_from_a_checkpoint_equals_the_layer_from_the_operands(tmp_path):
    g = geometry(1024, 16, 2, 512, 512, "benchmark")
    ops = synth.LayerOperands(g, "c1", device="cpu")
    x = synth.activations("c1", 8, g.hidden).cuda()
    root = str(tmp_path / "c1")
    synth.write_checkpoint(ops, root, prefix="layers.11", shards=2)
    direct = host.Layer(g, ops, 8)
    direct.set_tokens()
    direct.run(x)
    want = direct.tap("out").copy()
    direct.close()
    loaded = host.Layer.from_checkpoint(g, root, "layers.11", 8)
    loaded.set_tokens()
    loaded.run(x)
    assert np.array_equal(loaded.tap("out"), want)
    # and the loaded layer against the oracle, tap by tap, like a layer built from the operands
    from test_gpu_layer import check_layer
    check_layer(g, ops, x.cpu(), loaded.taps())
    loaded.close()
