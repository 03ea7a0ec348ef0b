#!/usr/bin/env python3
"""Writes the golden fixtures of this directory.  Run from the repository root: python tests/golden/make_fixtures.py

reference_contract_capacities.json
    Data the reference's own runtime contracts hold for this path: the capacity scalars of the routed-experts node
    (runtime/kernels/moe-runtime-*/runtime-contract.json: num_tokens, max_rows, rows_padded, max_tasks, max_phys_tiles),
    which src/moe.rs:1253-1257 checks at load time.  Only written when the reference checkout is present.

c1_<mode>.npz
    The smallest benchmark configuration (8 rows, H 1024, 16 experts, top-2, I 512, one shared expert) in both numerics
    modes: the seeded inputs that are cheap to store (token rows, token ids, live count, padding sources), digests of the
    seeded weights (which tests regenerate from the same seeds), and every tap of the layer as the CPU oracle computes
    it.  The oracle is pinned elsewhere (tests/test_oracle.py); these files pin it, and the generator, against drift and
    give the GPU tests a committed expectation to compare with.
"""
import glob
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
REFERENCE = "/root/reference"


def contract_capacities():
    rows = []
    for d in sorted(glob.glob(os.path.join(REFERENCE, "runtime/kernels/moe-runtime-*"))):
        f = os.path.join(d, "runtime-contract.json")
        if not os.path.exists(f):
            continue
        contract = json.load(open(f))
        for node in contract.get("nodes", []):
            sc = node.get("scalars", {})
            if "max_phys_tiles" in sc:
                drafter = "dspark" in os.path.basename(d)      # drafter layers: 128 experts, top-3 (src/layer_id.rs:39-47)
                rows.append({"contract": os.path.basename(d), "experts": 128 if drafter else 384, "topk": 3 if drafter else 6,
                             **{k: sc[k] for k in ("num_tokens", "max_rows", "rows_padded", "max_tasks", "max_phys_tiles")}})
                break
    return rows


def digest(t):
    return hashlib.sha256(t.detach().cpu().contiguous().view(-1).view(dtype=__import__("torch").uint8).numpy().tobytes()).hexdigest()


def c1_case(mode):
    import helpers
    from helpers import CONFIGS, geometry, oracle_layer, synth, u16
    import oracle
    c = CONFIGS["c1"]
    g = geometry(c["hidden"], c["experts"], c["topk"], c["inter"], c["shared"], mode)
    ops = synth.LayerOperands(g, "c1", device="cpu")
    x = synth.activations("c1/golden", c["rows"], c["hidden"])
    tokens = np.arange(c["rows"], dtype=np.int64)
    if mode == "reference":
        tokens[3] = 129264                                   # one image-token row: takes bias_alt
    live, padding = 7, np.array([-1, -1, -1, -1, -1, -1, 2, -1], np.int32)   # row 6 repeats row 2's experts with zero weights; row 7 is not live
    taps = oracle_layer(g, ops, x, tokens, live, padding)
    base, te, tv, tmap, tw = oracle.plan(taps["ids"], taps["weights"], g.experts, 1, 16)
    out = {"x": u16(x), "tokens": tokens, "live": np.int32(live), "padding": padding,
           "tile_base": base, "task_expert": te, "task_valid": tv, "token_map": tmap, "token_weights": tw}
    out.update({k: v for k, v in taps.items()})
    names = ["gate_w", "bias", "bias_alt", "w13", "s13", "w2", "s2", "sh_w13", "sh_s13", "sh_w2", "sh_s2"]
    out["weight_digests"] = np.array(json.dumps({n: digest(getattr(ops, n)) for n in names}))
    return out


def main():
    if os.path.isdir(REFERENCE):
        with open(os.path.join(HERE, "reference_contract_capacities.json"), "w") as f:
            json.dump(contract_capacities(), f, indent=1)
    for mode in ("benchmark", "reference"):
        np.savez_compressed(os.path.join(HERE, "c1_%s.npz" % mode), **c1_case(mode))


if __name__ == "__main__":
    main()
