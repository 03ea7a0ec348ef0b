"""ctypes binding of the C ABI in include/titanic_moe.h (libtitanic_moe_hip.so).

The product path has no fallback: if the library is missing the import fails with the build command to run.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_LIB = os.path.join(HERE, "libtitanic_moe_hip.so")
CODE_OBJECT = os.path.join(HERE, "titanic_moe_gfx950.hsaco")
REFERENCE_LAYER_OBJECT = os.path.join(HERE, "titanic_moe_gfx950_reference_layer.hsaco")

EXPORTS = ["ca_ffn_abi", "ca_ffn_configure", "ca_ffn_geometry", "ca_router_logits", "ca_shared_swiglu", "ca_ffn_add",
           "ca_router_logits_wide", "ca_kernel_launch", "ca_kernel_count", "ca_kernel_name", "ca_moe_nibble_permute",
           "ca_primitives_abi", "ca_primitives_open", "ca_primitives_close", "ca_primitives_launch", "ca_primitives_launch2",
           "ca_primitives_entries", "ca_primitives_scratch_bytes", "ca_primitives_marks", "ca_encode", "ca_decode", "ca_local_live",
           "ca_pack_bf16", "ca_primitives_spin_limit", "ca_primitives_shared_reserve", "ca_primitives_open_geometry", "ca_primitives_geometry", "ca_router_logits_in",
           "ca_router_logits_wide_in", "ca_shared_swiglu_in", "ca_ffn_add_in", "ca_moe_dynamic_static", "ca_moe_dynamic_static_capacity",
           "ca_ffn_norm_quant", "ca_ffn_sum_residual", "ca_hc_combine_norm_quant", "ca_hc_post", "ca_ffn_sum_hc_post"]


class Geometry(ctypes.Structure):
    _fields_ = [("hidden", ctypes.c_int32), ("experts", ctypes.c_int32), ("topk", ctypes.c_int32),
                ("intermediate", ctypes.c_int32), ("shared_intermediate", ctypes.c_int32), ("scoring", ctypes.c_int32),
                ("route_scale", ctypes.c_float), ("act_block", ctypes.c_int32), ("shared_bn", ctypes.c_int32),
                ("shared_bk", ctypes.c_int32), ("alt_token", ctypes.c_int64), ("swiglu_limit", ctypes.c_float)]


_lib = None


def library_sha256():
    """SHA-256 of the kernel library file as it lies beside this module (what a counter file is stamped with)."""
    import hashlib
    with open(KERNEL_LIB, "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(KERNEL_LIB):
        raise ImportError("%s is not built: run `python -c \"import __graft_entry__ as g; g.build()\"` at the repository root"
                          % KERNEL_LIB)
    lib = ctypes.CDLL(KERNEL_LIB)
    vp, i32, u64p, i32p = ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_int32)
    lib.ca_ffn_abi.restype = ctypes.c_int
    lib.ca_ffn_configure.argtypes = [ctypes.POINTER(Geometry)]
    lib.ca_ffn_geometry.argtypes = [ctypes.POINTER(Geometry)]
    lib.ca_router_logits.argtypes = [ctypes.c_int, vp, vp, vp, vp]
    lib.ca_router_logits_wide.argtypes = [ctypes.c_int, vp, vp, vp, vp]
    lib.ca_shared_swiglu.argtypes = [ctypes.c_int, vp, vp, vp]
    lib.ca_ffn_add.argtypes = [ctypes.c_int, vp, vp, vp, vp]
    lib.ca_kernel_launch.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32),
                                     ctypes.c_uint32, ctypes.POINTER(ctypes.c_void_p), vp]
    lib.ca_kernel_name.restype = ctypes.c_char_p
    lib.ca_kernel_name.argtypes = [ctypes.c_int]
    lib.ca_moe_nibble_permute.argtypes = [vp, ctypes.c_uint64, ctypes.c_int, vp]
    lib.ca_primitives_abi.restype = i32
    lib.ca_primitives_open.restype = vp
    lib.ca_primitives_open.argtypes = [i32p]
    lib.ca_primitives_close.argtypes = [vp]
    lib.ca_primitives_close.restype = None
    lib.ca_primitives_launch.restype = i32
    lib.ca_primitives_launch.argtypes = [vp, i32, u64p, ctypes.c_size_t, i32p, ctypes.c_size_t, vp]
    lib.ca_primitives_launch2.restype = i32
    lib.ca_primitives_launch2.argtypes = [vp, i32, u64p, ctypes.c_size_t, vp]
    lib.ca_primitives_entries.restype = i32
    lib.ca_primitives_scratch_bytes.restype = ctypes.c_int64
    lib.ca_primitives_scratch_bytes.argtypes = [vp, i32, i32]
    lib.ca_encode.argtypes = [vp, vp, vp, vp, ctypes.c_int, ctypes.c_int, vp]
    lib.ca_decode.argtypes = [vp, vp, vp, vp, ctypes.c_int, ctypes.c_int, vp]
    lib.ca_local_live.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, vp]
    lib.ca_pack_bf16.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, vp]
    lib.ca_primitives_marks.restype = i32
    lib.ca_primitives_marks.argtypes = [vp, ctypes.POINTER(vp), ctypes.c_size_t]
    lib.ca_primitives_spin_limit.restype = i32
    lib.ca_primitives_spin_limit.argtypes = [vp, i32]
    lib.ca_primitives_shared_reserve.restype = i32
    lib.ca_primitives_shared_reserve.argtypes = [vp, i32]
    lib.ca_primitives_open_geometry.restype = vp
    lib.ca_primitives_open_geometry.argtypes = [ctypes.POINTER(Geometry), i32p]
    lib.ca_primitives_geometry.restype = i32
    lib.ca_primitives_geometry.argtypes = [vp, ctypes.POINTER(Geometry)]
    lib.ca_moe_dynamic_static.restype = i32
    lib.ca_moe_dynamic_static.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, vp]
    lib.ca_moe_dynamic_static_capacity.restype = ctypes.c_int64
    lib.ca_router_logits_in.argtypes = [vp, ctypes.c_int, vp, vp, vp, vp]
    lib.ca_router_logits_wide_in.argtypes = [vp, ctypes.c_int, vp, vp, vp, vp]
    lib.ca_shared_swiglu_in.argtypes = [vp, ctypes.c_int, vp, vp, vp]
    lib.ca_ffn_add_in.argtypes = [vp, ctypes.c_int, vp, vp, vp, vp]
    lib.ca_ffn_norm_quant.argtypes = [vp, ctypes.c_int, vp, vp, ctypes.c_float, vp, vp, vp, vp, vp, vp]
    lib.ca_ffn_sum_residual.argtypes = [vp, ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, vp, vp]
    lib.ca_hc_combine_norm_quant.argtypes = [vp, ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.ca_hc_post.argtypes = [vp, ctypes.c_int, vp, vp, vp, vp, vp, vp]
    lib.ca_ffn_sum_hc_post.argtypes = [vp, ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    _lib = lib
    return lib


def kernel_names():
    lib = load()
    return [lib.ca_kernel_name(i).decode() for i in range(lib.ca_kernel_count())]


class _Arg:
    """One kernel argument kept alive for the duration of a launch."""

    def __init__(self, value):
        if isinstance(value, ctypes._SimpleCData):
            self.c = value
        elif isinstance(value, float):
            self.c = ctypes.c_float(value)
        elif isinstance(value, int):
            self.c = ctypes.c_int32(value)
        elif value is None:
            self.c = ctypes.c_void_p(0)
        else:  # torch tensor
            self.c = ctypes.c_void_p(value.data_ptr())


def open_context(geometry):
    """A context of the library with this geometry (ca_primitives_open_geometry); close it with ca_primitives_close."""
    lib = load()
    status = ctypes.c_int32(0)
    ctx = lib.ca_primitives_open_geometry(ctypes.byref(geometry), ctypes.byref(status))
    if not ctx or status.value != 0:
        raise RuntimeError("ca_primitives_open_geometry failed: %d" % status.value)
    return ctx


def ptr(t):
    """Device pointer argument (None -> null)."""
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def launch(name, grid, block, args, stream=0, shared=0):
    """ca_kernel_launch with python values: tensors and ptr() are pointers, ints are int32, floats float32; use ctypes
    values (c_int64 ...) for anything else."""
    lib = load()
    if isinstance(grid, int):
        grid = (grid, 1, 1)
    if isinstance(block, int):
        block = (block, 1, 1)
    keep = [_Arg(a) for a in args]
    argv = (ctypes.c_void_p * len(keep))(*[ctypes.cast(ctypes.pointer(k.c), ctypes.c_void_p) for k in keep])
    status = lib.ca_kernel_launch(name.encode(), (ctypes.c_uint32 * 3)(*grid), (ctypes.c_uint32 * 3)(*block), shared, argv,
                                  ctypes.c_void_p(stream))
    if status != 0:
        raise RuntimeError("ca_kernel_launch(%s) failed: %d" % (name, status))


def primitives_launch(ctx, index, pointers, scalars, stream=0):
    lib = load()
    p = (ctypes.c_uint64 * len(pointers))(*[0 if t is None else (t if isinstance(t, int) else t.data_ptr()) for t in pointers])
    s = (ctypes.c_int32 * len(scalars))(*scalars)
    return lib.ca_primitives_launch(ctypes.c_void_p(ctx), index, p, len(pointers), s, len(scalars), ctypes.c_void_p(stream))
