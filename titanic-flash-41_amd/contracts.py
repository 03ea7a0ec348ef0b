"""Writes the operator contracts of the kernel library in the reference's schema:

  contracts/bindings.json                  entries {index, name, kernel_id, pointers[], i32_scalars[]}  (src/primitives.rs:10-36)
  contracts/runtime-contract-m<rows>.json  nodes [{entry, kernel_id, pointers {name: {role, offset}}, scalars {}}], scratch_bytes,
                                           scratch_initializer, abi, deterministic, swiglu_limit  (src/moe.rs:34-68, 343-367)
  contracts/runtime-contract-micro-m4.json the micro sequence (quantize, both projections with FP32 projections kept, route sum; src/moe.rs:379-393)
  contracts/native.json                    the libcanada_ffn.so-style contract (src/ffn.rs:28-41)

Run:  python -m titanic-flash-41_amd.contracts   (from the repository root, after the build)
"""
import hashlib
import importlib
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "contracts")

DYN_POINTERS = ["a_ptr", "topk_ids_ptr", "topk_weights_ptr", "packed_a_storage_ptr", "scale_storage_ptr", "shared_a_storage_ptr",
                "shared_scale_storage_ptr", "intermediate_ptr", "intermediate_codes_ptr", "intermediate_scales_ptr", "task_expert_ptr",
                "task_valid_rows_ptr", "expert_tile_base", "token_map_ptr", "token_weights_ptr", "b_w13", "sfb_w13_ptr", "b_down",
                "sfb_down_ptr", "scatter_ptr", "plan_scratch_ptr"]
ROUTE_POINTERS = ["logits_ptr", "bias_ptr", "bias_alt_ptr", "input_ids_ptr", "num_token_non_padded_ptr", "padding_sources_ptr",
                  "gate_weight_ptr", "sync_ptr"]
SHARED_POINTERS = ["shared_w13", "shared_sfb_w13", "shared_w2", "shared_sfb_w2", "shared_activation_ptr", "shared_activation_codes_ptr",
                   "shared_activation_scales_ptr", "shared_up_ptr", "shared_output_ptr"]
MICRO_POINTERS = ["packed_a_ptr", "a_scales_ptr", "w13_ptr", "w13_scales_ptr", "intermediate_ptr", "projections_ptr", "token_weights_ptr",
                  "topk_ids_ptr", "alpha1_ptr", "input_scale_ptr", "w2_ptr", "w2_scales_ptr", "route_output_ptr", "alpha2_ptr", "down_scale_ptr",
                  "task_expert_ptr", "task_valid_rows_ptr", "expert_tile_base", "token_map_ptr", "tile_weights_ptr"]
QUANT_POINTERS = ["source_ptr", "values_ptr", "scale_rows_ptr", "scale_mma_ptr"]
DYN_SCALARS = ["num_tokens", "max_rows", "rows_padded", "max_phys_tiles", "tile_m", "groups"]

ENTRIES = [
    ("kernel_000", "integration.tp_moe.dynamic", DYN_POINTERS, DYN_SCALARS),
    ("kernel_001", "integration.tp_moe.dynamic", DYN_POINTERS + ROUTE_POINTERS, DYN_SCALARS + ["owner_rows"]),
    ("kernel_002", "moe.w4a16.topk_sum", ["fc2_ptr", "output_ptr", "num_token_non_padded_ptr"], ["active_m", "weight_num_experts", "route_num_experts"]),
    ("kernel_003", "gemm.mxfp8_quant_cute", ["input_ptr", "values_ptr", "scales_ptr", "values_min_ptr", "scales_min_ptr"], ["m", "k", "reserved"]),
    ("kernel_004", "gemm.dense", ["a_ptr", "sfa_ptr", "b_ptr", "sfb_ptr", "output_ptr"], ["m", "n", "k"]),
    ("kernel_005", "ffn.shared_expert", ["a_ptr", "sfa_ptr"] + SHARED_POINTERS, ["m"]),
    ("kernel_006", "moe.w4a8.phase1", DYN_POINTERS, DYN_SCALARS),
    ("kernel_007", "moe.w4a8.phase2", DYN_POINTERS, DYN_SCALARS),
    ("kernel_008", "moe.front_end", DYN_POINTERS, DYN_SCALARS),
    ("kernel_009", "ffn.experts_with_shared", DYN_POINTERS + ROUTE_POINTERS + SHARED_POINTERS, DYN_SCALARS + ["owner_rows"]),
    # entry 0 with a_ptr holding wire rows "dual_quant_rows_v1" (the reference's packed contract: src/moe.rs:512-583)
    ("kernel_010", "integration.tp_moe.dynamic", DYN_POINTERS, DYN_SCALARS),
    # the reference's micro sequence (src/moe.rs:379-393): its operand lists, then this library's plan tables
    ("kernel_011", "moe.w4a8.compact_micro", MICRO_POINTERS, ["num_pairs", "max_active_clusters"]),
    ("kernel_012", "gemm.mxfp8_quant_cute", QUANT_POINTERS, ["m", "source_k", "grid_x"]),       # no amax floor (routed experts)
    ("kernel_013", "gemm.mxfp8_quant_cute", QUANT_POINTERS, ["m", "source_k", "grid_x"]),       # amax floored at 1e-4 (shared expert)
]

ROLE = {"a_ptr": "input", "topk_ids_ptr": "ids", "topk_weights_ptr": "routing_weights", "b_w13": "w13", "sfb_w13_ptr": "s13",
        "b_down": "w2", "sfb_down_ptr": "s2"}


def align256(n):
    return (n + 255) // 256 * 256


def max_phys_tiles(pairs, tile_m, experts):
    """Tile capacity of a launch, as the reference's contracts state it (runtime-contract.json `max_phys_tiles`;
    src/moe.rs:1253-1257 checks it): min(E, pairs) experts open a tile each, the other routes fill ceil(pairs / tile_m) - 1 more."""
    return -(-pairs // tile_m) - 1 + min(experts, pairs)


def scratch_layout(g, rows):
    """The Workspace's scratch regions (same order and formulas as tf::Workspace in host/ffn_host.cpp)."""
    tile_m = 16 if rows <= 64 else 128
    pairs = rows * g["topk"]
    tiles = max_phys_tiles(pairs, tile_m, g["experts"])
    padded = tiles * tile_m
    H, I, B = g["hidden"], g["intermediate"], g["act_block"]
    sizes = [("packed_a_storage_ptr", rows * H), ("scale_storage_ptr", rows * H // B), ("shared_a_storage_ptr", rows * H),
             ("shared_scale_storage_ptr", rows * H // B), ("intermediate_ptr", padded * I * 2), ("intermediate_codes_ptr", padded * I),
             ("intermediate_scales_ptr", padded * I // B), ("task_expert_ptr", tiles * 4), ("task_valid_rows_ptr", tiles * 4),
             ("expert_tile_base", (g["experts"] + 1) * 4), ("token_map_ptr", padded * 4), ("token_weights_ptr", padded * 4),
             ("scatter_ptr", pairs * H * 2), ("plan_scratch_ptr", ((pairs + 63) // 64 * g["experts"] + pairs) * 4), ("sync_ptr", 4096 + 8 * 512 * 4)]
    at, offsets = 0, {}
    for name, size in sizes:
        offsets[name] = at
        at += align256(size)
    return offsets, at, tile_m, tiles


def sha256(path):
    return hashlib.sha256(open(path, "rb").read()).hexdigest() if path and os.path.exists(path) else None


def bindings(library):
    return {"abi": 1, "architecture": "gfx950", "physical_cus": 256, "source": "this repository", "source_commit": None,
            "library_sha256": sha256(library),
            "entries": [{"index": i, "name": n, "kernel_id": k, "pointers": p, "i32_scalars": s} for i, (n, k, p, s) in enumerate(ENTRIES)]}


def runtime_contract(g, rows, library):
    offsets, scratch_bytes, tile_m, tiles = scratch_layout(g, rows)
    pointers = {}
    for name in DYN_POINTERS:
        pointers[name] = {"role": ROLE[name], "offset": 0} if name in ROLE else {"role": "scratch", "offset": offsets[name]}
    scalars = {"num_tokens": rows, "max_rows": rows, "rows_padded": tiles * tile_m, "max_phys_tiles": tiles, "tile_m": tile_m, "groups": 1}
    return {"abi": 1, "rows": rows, "experts": g["experts"], "hidden": g["hidden"], "intermediate": g["intermediate"], "topk": g["topk"],
            "deterministic": True, "swiglu_limit": g["swiglu_limit"], "scratch_bytes": scratch_bytes, "scratch_initializer": "zero",
            "kernel_library_sha256": sha256(library), "input_format": "bf16_rows", "precision":
            "Canonical MXFP4 E8M0 K32;W4A8;FP32 FC1 through SwiGLU;BF16 activation boundary and output;deterministic topk sum",
            "nodes": [{"entry": 0, "kernel_id": "integration.tp_moe.dynamic", "pointers": pointers, "scalars": scalars},
                      {"entry": 2, "kernel_id": "moe.w4a16.topk_sum",
                       "pointers": {"fc2_ptr": {"role": "scratch", "offset": offsets["scatter_ptr"]}, "output_ptr": {"role": "output", "offset": 0},
                                    "num_token_non_padded_ptr": {"role": "output", "offset": 0}},
                       "scalars": {"active_m": rows, "weight_num_experts": 0, "route_num_experts": 0}}]}


def micro_contract(g, rows, library):
    """The micro sequence for a few rows (the reference's runtime/kernels/moe-runtime-m6-micro-fp32-v1/runtime-contract.json):
    quantize the rows, both projections with the FP32 projections of FC1 kept, ordered route sum."""
    pairs = rows * g["topk"]
    tiles = max_phys_tiles(pairs, 16, g["experts"])
    H, I, B = g["hidden"], g["intermediate"], g["act_block"]
    sizes = [("values_ptr", rows * H), ("scale_rows_ptr", rows * H // B), ("scale_mma_ptr", rows * H // B), ("projections_ptr", pairs * 2 * I * 4),
             ("intermediate_ptr", tiles * 16 * I * 2), ("route_output_ptr", pairs * H * 2), ("task_expert_ptr", tiles * 4),
             ("task_valid_rows_ptr", tiles * 4), ("expert_tile_base", (g["experts"] + 1) * 4), ("token_map_ptr", tiles * 16 * 4),
             ("tile_weights_ptr", tiles * 16 * 4)]
    at, off = 0, {}
    for name, size in sizes:
        off[name] = at
        at += align256(size)
    scratch = lambda name: {"role": "scratch", "offset": off[name]}
    ones = {"role": "ones", "offset": 0}
    micro = {"packed_a_ptr": scratch("values_ptr"), "a_scales_ptr": scratch("scale_rows_ptr"), "w13_ptr": {"role": "w13", "offset": 0},
             "w13_scales_ptr": {"role": "s13", "offset": 0}, "intermediate_ptr": scratch("intermediate_ptr"),
             "projections_ptr": scratch("projections_ptr"), "token_weights_ptr": {"role": "routing_weights", "offset": 0},
             "topk_ids_ptr": {"role": "ids", "offset": 0}, "alpha1_ptr": ones, "input_scale_ptr": ones, "w2_ptr": {"role": "w2", "offset": 0},
             "w2_scales_ptr": {"role": "s2", "offset": 0}, "route_output_ptr": scratch("route_output_ptr"), "alpha2_ptr": ones,
             "down_scale_ptr": ones}
    for name in ["task_expert_ptr", "task_valid_rows_ptr", "expert_tile_base", "token_map_ptr", "tile_weights_ptr"]:
        micro[name] = scratch(name)
    return {"abi": 1, "rows": rows, "experts": g["experts"], "hidden": H, "intermediate": I, "topk": g["topk"], "deterministic": True,
            "swiglu_limit": g["swiglu_limit"], "scratch_bytes": at, "scratch_initializer": "zero", "kernel_library_sha256": sha256(library),
            "projection_dtype": "float32", "input_format": "bf16_rows",
            "nodes": [{"entry": 12, "kernel_id": "gemm.mxfp8_quant_cute",
                       "pointers": {"source_ptr": {"role": "input", "offset": 0}, "values_ptr": scratch("values_ptr"),
                                    "scale_rows_ptr": scratch("scale_rows_ptr"), "scale_mma_ptr": scratch("scale_mma_ptr")},
                       "scalars": {"m": rows, "source_k": H, "grid_x": rows * 10}},
                      {"entry": 11, "kernel_id": "moe.w4a8.compact_micro", "pointers": micro,
                       "scalars": {"num_pairs": pairs, "max_active_clusters": 48}},
                      {"entry": 2, "kernel_id": "moe.w4a16.topk_sum",
                       "pointers": {"fc2_ptr": scratch("route_output_ptr"), "output_ptr": {"role": "output", "offset": 0},
                                    "num_token_non_padded_ptr": {"role": "output", "offset": 0}},
                       "scalars": {"active_m": rows, "weight_num_experts": 0, "route_num_experts": 0}}]}


def native_contract(g, library):
    return {"abi": 1, "architecture": "gfx950", "physical_cus": 256, "hidden": g["hidden"], "experts": g["experts"], "router_max_rows": 16,
            "router_n_split": 1, "shared_intermediate": g["shared_intermediate"], "swiglu_limit": g["swiglu_limit"],
            "library_sha256": sha256(library), "pdl": False}


BENCHMARK_GEOMETRY = dict(hidden=4096, experts=256, topk=6, intermediate=2048, shared_intermediate=2048, act_block=128, swiglu_limit=10.0)


def main(out=OUT, library=None):
    """Writes the contracts to `out`; `library`: the built kernel library whose SHA-256 they pin (None: the hash fields stay
    null, as in the committed copies, since no library is committed)."""
    os.makedirs(out, exist_ok=True)
    lib = library
    json.dump(bindings(lib), open(os.path.join(out, "bindings.json"), "w"), indent=1)
    json.dump(native_contract(BENCHMARK_GEOMETRY, lib), open(os.path.join(out, "native.json"), "w"), indent=1)
    for rows in (4, 32, 4096):
        json.dump(runtime_contract(BENCHMARK_GEOMETRY, rows, lib), open(os.path.join(out, "runtime-contract-m%d.json" % rows), "w"), indent=1)
    json.dump(micro_contract(BENCHMARK_GEOMETRY, 4, lib), open(os.path.join(out, "runtime-contract-micro-m4.json"), "w"), indent=1)


if __name__ == "__main__":
    main()
