"""CPU-side checks of the drop-in boundary: the shared libraries load without a GPU and export every symbol the header
declares, the operator contracts agree with the library's entry table, and argument validation answers with the
reference's error conventions before anything would touch a device."""
import ctypes
import importlib
import json
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pkg = importlib.import_module("titanic-flash-41_amd")
native = pkg.native
contracts = importlib.import_module("titanic-flash-41_amd.contracts")


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "titanic_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ca_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = native.load()
    names = declared_symbols()
    assert len(names) >= 18
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(native.EXPORTS) == names


def test_abi_versions_and_kernel_table():
    lib = native.load()
    assert lib.ca_ffn_abi() == 1 and lib.ca_primitives_abi() == 1
    names = native.kernel_names()
    for required in ["ca_route_padding_rows", "ca_ffn_sum_shared", "ca_moe_group_sum_rows", "ca_moe_frontend", "ca_moe_route_frontend",
                     "ca_route_topk", "ca_route_census", "ca_expert_compact_words", "ca_expert_compact_scales", "ca_expert_scale_codes4",
                     "ca_expert_scale_code1", "ca_expert_scale_code1_check", "ca_expert_scale_code1_census", "ca_shared_swiglu_quant"]:
        assert required in names, required        # the names the reference resolves from its code modules (src/ffn.rs, src/expert_packing.rs)
    assert lib.ca_kernel_name(len(names)) is None


def test_contracts_match_the_entry_table():
    lib = native.load()
    b = contracts.bindings(native.KERNEL_LIB)
    assert len(b["entries"]) == lib.ca_primitives_entries()
    assert [e["index"] for e in b["entries"]] == list(range(len(b["entries"])))
    # the node sequence the reference's workspace admits (src/moe.rs:378-383)
    c = contracts.runtime_contract(contracts.BENCHMARK_GEOMETRY, 4, native.KERNEL_LIB)
    assert [n["kernel_id"] for n in c["nodes"]] == ["integration.tp_moe.dynamic", "moe.w4a16.topk_sum"]
    assert c["scratch_initializer"] == "zero" and c["deterministic"] and c["swiglu_limit"] == 10.0
    node = c["nodes"][0]
    assert sorted(node["pointers"]) == sorted(b["entries"][0]["pointers"]) and sorted(node["scalars"]) == sorted(b["entries"][0]["i32_scalars"])
    for p in node["pointers"].values():
        assert p["role"] in {"input", "ids", "routing_weights", "scratch", "w13", "s13", "w2", "s2"}
        assert p["role"] != "scratch" or p["offset"] < c["scratch_bytes"]
    assert node["scalars"]["rows_padded"] == node["scalars"]["max_phys_tiles"] * node["scalars"]["tile_m"]
    committed = os.path.join(ROOT, "titanic-flash-41_amd", "contracts", "bindings.json")
    if os.path.exists(committed):
        on_disk = json.load(open(committed))
        assert [(e["kernel_id"], e["pointers"], e["i32_scalars"]) for e in on_disk["entries"]] == \
               [(e["kernel_id"], e["pointers"], e["i32_scalars"]) for e in b["entries"]]


def test_argument_validation_needs_no_device():
    lib = native.load()
    bad = native.Geometry(1000, 16, 2, 512, 512, 0, 1.0, 128, 128, 128, -1, 10.0)
    assert lib.ca_ffn_configure(ctypes.byref(bad)) == -4
    assert lib.ca_ffn_configure(None) == -1
    good = native.Geometry(1024, 16, 2, 512, 512, 0, 1.0, 128, 128, 128, -1, 10.0)
    assert lib.ca_ffn_configure(ctypes.byref(good)) == 0
    # accepted widths: token rows of a multiple of 512 up to 4,096 or of 1,024 up to 8,192; expert widths multiples of 512 up to 4,096
    # (the reference's 5,120 token width is one; its expert width 576 / 2,304 goes in padded: 1,024 / 2,560)
    for hidden, inter, shared, want in [(5120, 2560, 2560, 0), (5120, 1024, 1024, 0), (8192, 4096, 512, 0), (3584, 1536, 3072, 0),
                                        (5120, 576, 576, -4), (5120, 2304, 2304, -4), (4608, 512, 512, -4), (9216, 512, 512, -4),
                                        (4096, 4608, 512, -4), (4096, 512, 8192, -4)]:
        trial = native.Geometry(hidden, 384, 6, inter, shared, 1, 1.5, 32, 32, 32, 129264, 10.0)
        assert lib.ca_ffn_configure(ctypes.byref(trial)) == want, (hidden, inter, shared)
    assert lib.ca_ffn_configure(ctypes.byref(good)) == 0
    back = native.Geometry()
    assert lib.ca_ffn_geometry(ctypes.byref(back)) == 0 and (back.hidden, back.experts, back.act_block) == (1024, 16, 128)
    assert lib.ca_router_logits(0, None, None, None, None) == -1 and lib.ca_router_logits(17, None, None, None, None) == -1
    assert lib.ca_shared_swiglu(0, None, None, None) == -1 and lib.ca_ffn_add(70000, None, None, None, None) == -1
    assert lib.ca_moe_nibble_permute(None, 16, 0, None) == -1
    assert lib.ca_primitives_launch(None, 0, None, 0, None, 0, None) == -1
    # the profiling marks take none, five (between the launches) or seven events (+ the FC1 kernel's own start / completion)
    assert lib.ca_primitives_marks(None, None, 0) == -1
    grid = (ctypes.c_uint32 * 3)(1, 1, 1)
    assert lib.ca_kernel_launch(b"no_such_kernel", grid, grid, 0, (ctypes.c_void_p * 1)(), None) == -3


def test_contexts_carry_their_geometry_and_the_library_is_pinned(tmp_path):
    import shutil
    lib = native.load()
    st = ctypes.c_int32(7)
    assert not lib.ca_primitives_open_geometry(None, ctypes.byref(st)) and st.value == -1
    bad = native.Geometry(1000, 16, 2, 512, 512, 0, 1.0, 128, 128, 128, -1, 10.0)
    assert not lib.ca_primitives_open_geometry(ctypes.byref(bad), ctypes.byref(st)) and st.value == -4
    assert lib.ca_router_logits_in(None, 1, None, None, None, None) == -1 and lib.ca_ffn_add_in(None, 1, None, None, None, None) == -1
    assert lib.ca_shared_swiglu_in(None, 1, None, None, None) == -1 and lib.ca_primitives_spin_limit(None, 1) == -1 and lib.ca_primitives_shared_reserve(None, 8) == -1
    assert lib.ca_primitives_geometry(None, None) == -1
    # the host mirror refuses a kernel library whose SHA-256 differs from the manifest beside it (src/ffn.rs:70-74), before loading it
    shutil.copy(native.KERNEL_LIB, tmp_path / "libtitanic_moe_hip.so")
    (tmp_path / "manifest.json").write_text(json.dumps({"library_sha256": "0" * 64}))
    host_lib = pkg.host.load()
    err = ctypes.create_string_buffer(256)
    g = native.Geometry(1024, 16, 2, 512, 512, 0, 1.0, 128, 128, 128, -1, 10.0)
    handle = host_lib.tfh_layer_create(str(tmp_path / "libtitanic_moe_hip.so").encode(), ctypes.byref(g), 4, (ctypes.c_void_p * 11)(), 0, 1, 1, 1, 0, 1, 1, err, 256)
    assert not handle and b"hash mismatch" in err.value
    # the manifest the build wrote pins the library that is loaded
    manifest = json.load(open(os.path.join(os.path.dirname(native.KERNEL_LIB), "manifest.json")))
    import hashlib
    assert manifest["library_sha256"] == hashlib.sha256(open(native.KERNEL_LIB, "rb").read()).hexdigest()


def test_host_library_loads_and_reports_a_missing_kernel_library():
    host = pkg.host
    lib = host.load()
    err = ctypes.create_string_buffer(256)
    g = native.Geometry(1024, 16, 2, 512, 512, 0, 1.0, 128, 128, 128, -1, 10.0)
    ptrs = (ctypes.c_void_p * 11)()
    handle = lib.tfh_layer_create(b"/nonexistent/libtitanic_moe_hip.so", ctypes.byref(g), 4, ptrs, 0, 1, 1, 1, 0, 1, 1, err, 256)
    assert not handle and b"load kernel library" in err.value
