#!/usr/bin/env python3
"""Writes tests/golden/layout_names.json: the tensor names, dtypes and shapes the reference requires for the FFN part of
one layer, read out of the text of the reference's contract (src/layout.rs:247-275, `validate_target_weights`): the
`c.require(&format!(...), Dtype::X, &[...])` calls whose name contains ".ffn.", inside their `for e in 0..N` and
`for (name, n, k) in [...]` loops.  The reference is read as text, nothing of it is run.  The fixture holds data only:
name templates ({p} = layer prefix, {e} = expert number), the safetensors dtype strings (src/checkpoint.rs:15-26) and
the shapes both as numbers (the reference's model: hidden 5120, 384 experts, expert width 2304) and as expressions in
H (hidden), E (experts), I (expert width), from which a test builds the table of a smaller layer.

    python tests/golden/make_layout_names.py [/root/reference]
"""
import json
import os
import re
import sys

DTYPES = {"F32": "F32", "Bf16": "BF16", "Fp8": "F8_E4M3", "E8m0": "F8_E8M0", "PackedFp4": "I8"}     # src/checkpoint.rs:15-26
HIDDEN = 5120            # config.text_config.hidden_size of the reference's model (runtime/model/config.json)


def number(expr, bindings):
    """A shape entry `name` or `name / digits` (a loop variable or a literal, optionally divided) as an integer; anything else
    in the reference's text is refused, nothing of it is evaluated."""
    m = re.fullmatch(r"(\w+)(?:\s*/\s*(\d+))?", expr.strip())
    if not m:
        raise ValueError("unexpected shape expression in the reference's contract: %r" % expr)
    head, div = m.group(1), m.group(2)
    base = bindings[head] if head in bindings else int(head)
    return base // int(div) if div else base


def symbolic(expr, value, bindings):
    """A shape entry as an expression in H, E, I: loop variables by their value's meaning, literals by their value."""
    names = {HIDDEN: "H", 384: "E", 2304: "I"}
    expr = expr.strip()
    m = re.fullmatch(r"(\w+)(?:\s*/\s*(\d+))?", expr)
    head, div = m.group(1), m.group(2)
    base = bindings[head] if head in bindings else int(head)
    text = names.get(base, str(base))
    return text + ("/" + div if div else "")


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    lines = open(os.path.join(root, "src", "layout.rs")).read().split("\n")
    start = next(i for i, l in enumerate(lines) if "fn validate_target_weights" in l)
    text = "\n".join(lines[start:start + 80])
    text = text[:text.index("engram_layer_ids")]
    entries = []
    # walk the text: remember the innermost tuple loop and whether an expert loop is open (by indentation)
    tuple_loop = None
    for m in re.finditer(r"for \((\w+), (\w+), (\w+)\) in \[(.*?)\]\s*\{|c\.require\(\s*&format!\(\"([^\"]+)\"\),\s*Dtype::(\w+),\s*&\[([^\]]*)\],?\s*\)", text, re.S):
        if m.group(1):
            rows = re.findall(r"\(\"(\w+)\",\s*([\w]+),\s*([\w]+)\)", m.group(4))
            tuple_loop = [(r[0], r[1], r[2]) for r in rows]
            continue
        name, dtype, shape = m.group(5), m.group(6), m.group(7)
        if ".ffn." not in name:
            continue
        dims = [d for d in shape.split(",") if d.strip()]
        variants = tuple_loop if "{name}" in name else [(None, None, None)]
        for tname, n, k in variants:
            bind = {"d": HIDDEN}
            if tname is not None:
                bind["n"] = HIDDEN if n == "d" else int(n)
                bind["k"] = HIDDEN if k == "d" else int(k)
            numbers = [number(d, bind) for d in dims]
            entries.append({"name": name.replace("{name}", tname) if tname else name, "dtype": DTYPES[dtype], "shape": numbers,
                            "dims": [symbolic(d, None, bind) for d in dims]})
    experts = int(re.search(r"for e in 0\.\.(\d+)", text).group(1))
    out = {"source": "src/layout.rs:247-275 (validate_target_weights, the .ffn. tensors of one layer)", "hidden": HIDDEN, "experts": experts,
           "expert_width": 2304, "per_expert": [e for e in entries if "{e}" in e["name"]], "per_layer": [e for e in entries if "{e}" not in e["name"]]}
    target = os.path.join(os.path.dirname(os.path.abspath(__file__)), "layout_names.json")
    with open(target, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(target, len(out["per_expert"]), "per expert,", len(out["per_layer"]), "per layer")


if __name__ == "__main__":
    main()
