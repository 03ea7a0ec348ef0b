"""GPU test of ca_moe_dynamic_static, the entry point that allocates nothing: the routed experts of entry 0 with every scratch
region in the library's static device array.  Its route outputs must equal entry 0's bit for bit, on two calls in a row, the
second with a smaller input (the array keeps the first call's contents)."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import GpuLayer, geometry, native, np_of, synth

pytestmark = pytest.mark.gpu


def routed_by_entry0(g, ops, x, rows):
    layer = GpuLayer(g, ops, rows)
    layer.run(x[:rows], fuse_route=False)
    out = dict(ids=layer.ids.clone(), weights=layer.weights.clone(), route_out=np_of(layer.route_out).view(np.uint16).copy(),
               w13=layer.w13, s13=layer.s13, w2=layer.w2, s2=layer.s2)
    return layer, out


def test_static_scratch_entry_equals_entry0_twice():
    lib = native.load()
    g = geometry(1024, 16, 2, 512, 512, "reference")
    ops = synth.LayerOperands(g, "static", device="cuda")
    x = synth.activations("static", 8, 1024).cuda().contiguous()
    assert lib.ca_moe_dynamic_static_capacity() == 16 << 20
    for rows in (8, 3):                      # the second call is smaller: stale contents of the first stay behind it in the array
        layer, want = routed_by_entry0(g, ops, x, rows)
        got = torch.full((rows, g.topk, g.hidden), 0x7fc0, dtype=torch.int16, device="cuda")
        xr = x[:rows].contiguous()
        torch.cuda.synchronize()
        st = lib.ca_moe_dynamic_static(ctypes.c_void_p(layer.ctx), native.ptr(xr), native.ptr(want["ids"]), native.ptr(want["weights"]),
                                       native.ptr(want["w13"]), native.ptr(want["s13"]), native.ptr(want["w2"]), native.ptr(want["s2"]),
                                       native.ptr(got), rows, None)
        torch.cuda.synchronize()
        assert st == 0, st
        live = np_of(want["ids"]) >= 0
        assert np.array_equal(np_of(got).view(np.uint16)[live], want["route_out"][live]), rows
        # argument checks: nulls, row counts the static array does not take
        assert lib.ca_moe_dynamic_static(ctypes.c_void_p(layer.ctx), None, None, None, None, None, None, None, None, rows, None) == -1
        assert lib.ca_moe_dynamic_static(ctypes.c_void_p(layer.ctx), native.ptr(xr), native.ptr(want["ids"]), native.ptr(want["weights"]),
                                         native.ptr(want["w13"]), native.ptr(want["s13"]), native.ptr(want["w2"]), native.ptr(want["s2"]),
                                         native.ptr(got), 65, None) == -5
        layer.close()
