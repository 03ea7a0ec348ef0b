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
    loaded.close()
