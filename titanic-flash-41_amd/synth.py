"""Seeded synthetic operands for the MoE FFN layer (torch, any device).

Generator: SplitMix64 of (stream id + counter) -> two 53-bit uniforms -> Box-Muller in float64 -> float32.  A tensor's
stream id is FNV-1a of "<config>/<tensor>" plus the base seed, so every tensor of every config is reproducible on its
own.  Quantizers follow OCP Microscaling: MXFP4 (E2M1, 32-element blocks along K, UE8M0 scales, low nibble = even
element) for routed experts, E4M3 with UE8M0 block scales for the shared expert.
"""
import math

import torch

BASE_SEED = 20261125
_M64 = (1 << 64) - 1


def fnv1a(text):
    h = 0xcbf29ce484222325
    for b in text.encode():
        h = ((h ^ b) * 0x100000001b3) & _M64
    return h


def _wrap(v):
    v &= _M64
    return v - (1 << 64) if v >= (1 << 63) else v


def _lsr(x, s):
    return (x >> s) & ((1 << (64 - s)) - 1)


def _splitmix(z):
    z = (z ^ _lsr(z, 30)) * _wrap(0xbf58476d1ce4e5b9)
    z = (z ^ _lsr(z, 27)) * _wrap(0x94d049bb133111eb)
    return z ^ _lsr(z, 31)


def normal(name, shape, std=1.0, mean=0.0, device="cpu", seed=BASE_SEED):
    """float32 tensor ~ N(mean, std) for the named stream."""
    n = 1
    for s in shape:
        n *= s
    stream = _wrap(fnv1a(name) + seed * 0x9e3779b97f4a7c15)
    idx = torch.arange(n, dtype=torch.int64, device=device)
    a = _splitmix(idx * 2 * _wrap(0x9e3779b97f4a7c15) + stream)
    b = _splitmix((idx * 2 + 1) * _wrap(0x9e3779b97f4a7c15) + stream)
    u1 = (_lsr(a, 11).to(torch.float64) + 1.0) * (1.0 / 9007199254740992.0)      # (0, 1]
    u2 = _lsr(b, 11).to(torch.float64) * (1.0 / 9007199254740992.0)
    z = torch.sqrt(-2.0 * torch.log(u1)) * torch.cos(2.0 * math.pi * u2)
    return (z * std + mean).to(torch.float32).reshape(shape)


def to_bf16_bits(x):
    """float32 -> BF16 bit patterns (int16 storage), round to nearest even."""
    return x.to(torch.bfloat16).view(torch.int16)


def _floor_log2(a):
    """floor(log2(a)) for positive normal float32 a, from the exponent field."""
    return ((a.view(torch.int32) >> 23) & 255) - 127


def quantize_e2m1(v):
    """float32 -> E2M1 code (uint8, bit 3 = sign), round to nearest even on {0, .5, 1, 1.5, 2, 3, 4, 6}, saturating."""
    a = v.abs()
    q = torch.zeros_like(a, dtype=torch.uint8)
    # thresholds with ties to the even code
    q = torch.where(a > 0.25, torch.full_like(q, 1), q)
    q = torch.where(a >= 0.75, torch.full_like(q, 2), q)
    q = torch.where(a > 1.25, torch.full_like(q, 3), q)
    q = torch.where(a >= 1.75, torch.full_like(q, 4), q)
    q = torch.where(a > 2.5, torch.full_like(q, 5), q)
    q = torch.where(a >= 3.5, torch.full_like(q, 6), q)
    q = torch.where(a > 5.0, torch.full_like(q, 7), q)
    sign = (v.view(torch.int32) < 0).to(torch.uint8) << 3
    return q | sign


def quantize_mxfp4(w):
    """w [rows][cols] float32 -> (packed uint8 [rows][cols/2], scales uint8 [rows][cols/32])."""
    rows, cols = w.shape
    blocks = w.reshape(rows, cols // 32, 32)
    amax = blocks.abs().amax(dim=2)
    e = torch.where(amax >= 1.17549435e-38, _floor_log2(amax.clamp_min(1.17549435e-38)) - 2 + 127, torch.full_like(amax, 127, dtype=torch.int32))
    e = e.clamp(1, 247).to(torch.int32)
    inv = ((254 - e) << 23).view(torch.float32)
    codes = quantize_e2m1(blocks * inv.unsqueeze(2)).reshape(rows, cols // 2, 2)
    packed = codes[:, :, 0] | (codes[:, :, 1] << 4)
    return packed.contiguous(), e.to(torch.uint8).contiguous()


def quantize_fp8_blocks(w, bn, bk):
    """w [rows][cols] float32 -> (E4M3 codes uint8 [rows][cols], scales uint8 [rows/bn][cols/bk])."""
    rows, cols = w.shape
    blocks = w.reshape(rows // bn, bn, cols // bk, bk)
    amax = blocks.abs().amax(dim=(1, 3))
    e = torch.where(amax >= 1.17549435e-38, _floor_log2(amax.clamp_min(1.17549435e-38)) - 8 + 127, torch.full_like(amax, 127, dtype=torch.int32))
    e = e.clamp(1, 247).to(torch.int32)
    inv = ((254 - e) << 23).view(torch.float32)
    scaled = blocks * inv.reshape(rows // bn, 1, cols // bk, 1)
    codes = scaled.reshape(rows, cols).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)   # saturating
    return codes.contiguous(), e.to(torch.uint8).contiguous()


class LayerOperands:
    """Canonical (checkpoint-layout) operands of one layer, all torch tensors on one device."""

    def __init__(self, geometry, config_name, device="cpu", weight_std=0.02, seed=BASE_SEED, experts_subset=None):
        g = geometry
        H, E, I, S = g.hidden, g.experts, g.intermediate, g.shared_intermediate
        self.geometry = g
        name = config_name
        self.gate_w = to_bf16_bits(normal(name + "/gate.weight", (E, H), std=1.0 / math.sqrt(H), device=device, seed=seed))
        self.bias = normal(name + "/gate.bias", (E,), std=0.1, device=device, seed=seed)
        self.bias_alt = normal(name + "/gate.bias_alt", (E,), std=0.1, device=device, seed=seed)
        # routed experts, expert-major: [E][2][I][H/2] (up rows then gate rows), [E][H][I/2]
        self.w13 = torch.empty((E, 2 * I, H // 2), dtype=torch.uint8, device=device)
        self.s13 = torch.empty((E, 2 * I, H // 32), dtype=torch.uint8, device=device)
        self.w2 = torch.empty((E, H, I // 2), dtype=torch.uint8, device=device)
        self.s2 = torch.empty((E, H, I // 32), dtype=torch.uint8, device=device)
        for e in range(E) if experts_subset is None else experts_subset:
            w = normal("%s/experts.%d.w13" % (name, e), (2 * I, H), std=weight_std, device=device, seed=seed)
            self.w13[e], self.s13[e] = quantize_mxfp4(w)
            w = normal("%s/experts.%d.w2" % (name, e), (H, I), std=weight_std, device=device, seed=seed)
            self.w2[e], self.s2[e] = quantize_mxfp4(w)
        w = normal(name + "/shared.w13", (2 * S, H), std=weight_std, device=device, seed=seed)
        self.sh_w13, self.sh_s13 = quantize_fp8_blocks(w, g.shared_bn, g.shared_bk)
        w = normal(name + "/shared.w2", (H, S), std=weight_std, device=device, seed=seed)
        self.sh_w2, self.sh_s2 = quantize_fp8_blocks(w, g.shared_bn, g.shared_bk)


def zipf_bias(experts, s=1.1, strength=1.0, device="cpu"):
    """Per-expert bias whose popularity follows rank^-s (strength scales the spread of the bias)."""
    rank = torch.arange(1, experts + 1, dtype=torch.float32, device=device)
    pop = rank.pow(-s)
    return strength * torch.log(pop / pop.mean())


def activations(config_name, rows, hidden, device="cpu", step=0, seed=BASE_SEED):
    return to_bf16_bits(normal("%s/x.%d" % (config_name, step), (rows, hidden), device=device, seed=seed))


def write_checkpoint(ops, root, prefix="layers.0", shards=2):
    """Writes one layer's canonical operands as a safetensors checkpoint directory with the reference's tensor names, dtypes
    and shapes (src/layout.rs:247-275): per expert w1 (gate) / w3 (up) / w2 packed FP4 (I8 [n][k/2]) with F8_E8M0 scales
    [n][k/32]; shared expert w1 / w3 / w2 F8_E4M3 with F8_E8M0 block scales; gate weight BF16, bias and bias_vl F32.
    Plain file writing (8-byte little-endian header length, JSON header, tensor bytes): nothing of the format needs a library."""
    import json
    import os
    import numpy as np
    g = ops.geometry
    I, S = g.intermediate, g.shared_intermediate
    def raw(t):
        return t.detach().cpu().contiguous().view(-1).view(dtype=torch.uint8).numpy().tobytes()
    tensors = []
    for e in range(g.experts):
        x = "%s.ffn.experts.%d." % (prefix, e)
        tensors += [(x + "w1.weight", "I8", ops.w13[e, I:]), (x + "w1.scale", "F8_E8M0", ops.s13[e, I:]),
                    (x + "w3.weight", "I8", ops.w13[e, :I]), (x + "w3.scale", "F8_E8M0", ops.s13[e, :I]),
                    (x + "w2.weight", "I8", ops.w2[e]), (x + "w2.scale", "F8_E8M0", ops.s2[e])]
    sh = prefix + ".ffn.shared_experts."
    rows13 = ops.sh_s13.shape[0] // 2
    tensors += [(sh + "w1.weight", "F8_E4M3", ops.sh_w13[:S]), (sh + "w1.scale", "F8_E8M0", ops.sh_s13[:rows13]),
                (sh + "w3.weight", "F8_E4M3", ops.sh_w13[S:]), (sh + "w3.scale", "F8_E8M0", ops.sh_s13[rows13:]),
                (sh + "w2.weight", "F8_E4M3", ops.sh_w2), (sh + "w2.scale", "F8_E8M0", ops.sh_s2),
                (prefix + ".ffn.gate.weight", "BF16", ops.gate_w), (prefix + ".ffn.gate.bias", "F32", ops.bias),
                (prefix + ".ffn.gate.bias_vl", "F32", ops.bias_alt)]
    os.makedirs(root, exist_ok=True)
    weight_map = {}
    per = -(-len(tensors) // shards)
    for k in range(shards):
        part = tensors[k * per:(k + 1) * per]
        if not part:
            continue
        name = "model-%05d-of-%05d.safetensors" % (k + 1, shards)
        header, at, blobs = {"__metadata__": {"format": "pt"}}, 0, []
        for key, dtype, t in part:
            b = raw(t)
            header[key] = {"dtype": dtype, "shape": list(t.shape), "data_offsets": [at, at + len(b)]}
            at += len(b)
            blobs.append(b)
            weight_map[key] = name
        text = json.dumps(header).encode()
        with open(os.path.join(root, name), "wb") as f:
            f.write(len(text).to_bytes(8, "little"))
            f.write(text)
            for b in blobs:
                f.write(b)
    with open(os.path.join(root, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f)
