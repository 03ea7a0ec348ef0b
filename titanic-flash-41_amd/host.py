"""ctypes binding of libtitanic_ffn_host.so, the C++ host mirror of the reference's Rust FFN operators
(LayerFfn / Router / Workspace / prepare_layer).  Inputs are torch tensors (device memory only); results are numpy."""
import ctypes
import os

import numpy as np

from . import native

HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB = os.path.join(HERE, "libtitanic_ffn_host.so")
_lib = None

EXTRA_TAPS = {"sync": np.uint32}       # the front-end's hand-off region (not a layer tap: not in taps())
TAPS = {"logits": np.float32, "ids": np.int32, "weights": np.float32, "xq": np.uint8, "xs": np.uint8, "xq_min": np.uint8,
        "xs_min": np.uint8, "h": np.uint16, "hq": np.uint8, "hs": np.uint8, "task_expert": np.int32, "task_valid": np.int32,
        "tile_base": np.int32, "token_map": np.int32, "token_weights": np.float32, "route_out": np.uint16, "routed": np.uint16,
        "shared_up": np.uint16, "shared_act": np.uint16, "shared_aq": np.uint8, "shared_as": np.uint8, "shared_down": np.uint16,
        "out": np.uint16}


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(HOST_LIB):
            raise ImportError("%s is not built: run __graft_entry__.build()" % HOST_LIB)
        lib = ctypes.CDLL(HOST_LIB)
        vp, cp, sz = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t
        lib.tfh_layer_create.restype = vp
        lib.tfh_layer_create.argtypes = [cp, ctypes.POINTER(native.Geometry), ctypes.c_int, ctypes.POINTER(vp), ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, cp, sz]
        lib.tfh_layer_destroy.argtypes = [vp]
        lib.tfh_layer_destroy.restype = None
        lib.tfh_layer_set_tokens.argtypes = [vp, vp, ctypes.c_int, vp, cp, sz]
        lib.tfh_layer_run.argtypes = [vp, ctypes.c_uint64, cp, sz]
        lib.tfh_layer_capture.argtypes = [vp, ctypes.POINTER(ctypes.c_uint64), ctypes.c_int, cp, sz]
        lib.tfh_layer_time.argtypes = [vp, ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float), cp, sz]
        lib.tfh_layer_time_phase.argtypes = [vp, ctypes.c_int, ctypes.c_uint64, ctypes.c_int, ctypes.POINTER(ctypes.c_float), cp, sz]
        lib.tfh_layer_profile_step.argtypes = [vp, ctypes.c_uint64, ctypes.POINTER(ctypes.c_float), cp, sz]
        lib.tfh_layer_profile_marks.argtypes = [vp, ctypes.POINTER(ctypes.c_uint64), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float), cp, sz]
        lib.tfh_layer_pair_run.argtypes = [vp, ctypes.c_uint64, ctypes.POINTER(ctypes.c_int64), ctypes.c_int, ctypes.c_uint64, ctypes.POINTER(ctypes.c_int64),
                                           ctypes.c_int, ctypes.c_int, vp, vp, cp, sz]
        lib.tfh_layer_tap.restype = ctypes.c_longlong
        lib.tfh_layer_tap.argtypes = [vp, cp, vp, sz, cp, sz]
        lib.tfh_layer_census.argtypes = [vp, vp, cp, sz]
        lib.tfh_layer_info.argtypes = [vp, ctypes.POINTER(ctypes.c_longlong)]
        lib.tfh_layer_info.restype = None
        _lib = lib
    return _lib


class HostError(RuntimeError):
    pass


class Layer:
    """One LayerFfn + Workspace + TokenRows on cuda:0 for `rows` token rows."""

    def __init__(self, geometry, operands, rows, overlap=True, sum_shared=True, route_front=True, code_scales=False, fold_shared=True, gate_front=True):
        self.lib = load()
        native.load()
        self.g, self.rows = geometry, rows
        self._err = ctypes.create_string_buffer(512)
        names = ["gate_w", "bias", "bias_alt", "w13", "s13", "w2", "s2", "sh_w13", "sh_s13", "sh_w2", "sh_s2"]
        tensors = [getattr(operands, n).contiguous() for n in names]
        on_device = tensors[0].is_cuda
        assert all(t.is_cuda == on_device for t in tensors)
        ptrs = (ctypes.c_void_p * 11)(*[t.data_ptr() for t in tensors])
        if on_device:
            import torch
            torch.cuda.synchronize()
        self.h = self.lib.tfh_layer_create(native.KERNEL_LIB.encode(), ctypes.byref(geometry), rows, ptrs, int(on_device), int(overlap),
                                           int(sum_shared), int(route_front), int(code_scales), int(fold_shared), int(gate_front), self._err, 512)
        if not self.h:
            raise HostError(self._err.value.decode())
        self.h = ctypes.c_void_p(self.h)

    @classmethod
    def from_checkpoint(cls, geometry, root, prefix, rows, overlap=True, sum_shared=True, route_front=True, code_scales=False, fold_shared=True,
                        gate_front=True):
        """The layer with its operands read from a safetensors checkpoint directory by the host mirror's own scanner."""
        self = cls.__new__(cls)
        self.lib = load()
        native.load()
        self.g, self.rows = geometry, rows
        self._err = ctypes.create_string_buffer(512)
        self.lib.tfh_layer_create_from_checkpoint.restype = ctypes.c_void_p
        self.lib.tfh_layer_create_from_checkpoint.argtypes = [ctypes.c_char_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_char_p] + \
            [ctypes.c_int] * 6 + [ctypes.c_char_p, ctypes.c_size_t]
        self.h = self.lib.tfh_layer_create_from_checkpoint(native.KERNEL_LIB.encode(), ctypes.byref(geometry), rows, root.encode(), prefix.encode(),
                                                           int(overlap), int(sum_shared), int(route_front), int(code_scales), int(fold_shared),
                                                           int(gate_front), self._err, 512)
        if not self.h:
            raise HostError(self._err.value.decode())
        self.h = ctypes.c_void_p(self.h)
        return self

    def _check(self, status):
        if status < 0:
            raise HostError(self._err.value.decode())
        return status

    def close(self):
        if self.h:
            self.lib.tfh_layer_destroy(self.h)
            self.h = None

    def set_tokens(self, ids=None, live=None, padding=None):
        ids = np.zeros(self.rows, np.int64) if ids is None else np.ascontiguousarray(ids, np.int64)
        pad = None if padding is None else np.ascontiguousarray(padding, np.int32)
        self._check(self.lib.tfh_layer_set_tokens(self.h, ids.ctypes.data, self.rows if live is None else live,
                                                  None if pad is None else pad.ctypes.data, self._err, 512))

    def keep_intermediate(self, on):
        """Many rows: whether FC1 also stores the BF16 intermediate (a tap; FC2 reads the FP8 codes)."""
        self.lib.tfh_layer_keep_intermediate.argtypes = [ctypes.c_void_p, ctypes.c_int]
        self.lib.tfh_layer_keep_intermediate.restype = None
        self.lib.tfh_layer_keep_intermediate(self.h, int(on))

    def run(self, x):
        assert x.is_cuda and x.is_contiguous() and x.numel() == self.rows * self.g.hidden
        self._check(self.lib.tfh_layer_run(self.h, x.data_ptr(), self._err, 512))

    def run_quantized(self, x, codes, scales):
        """One pass with the shared expert fed from the caller's pre-quantized rows (E4M3 codes, UE8M0 scales; device tensors)."""
        self.lib.tfh_layer_run_quantized.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_char_p, ctypes.c_size_t]
        self._check(self.lib.tfh_layer_run_quantized(self.h, x.data_ptr(), codes.data_ptr(), scales.data_ptr(), self._err, 512))

    def run_row_transport(self, x, packed_out=None):
        """One pass through the one-rank row transport: pack to wire rows, routed experts from the packed rows, shared expert from
        the decoded codes.  `packed_out`: optional uint8 device tensor [rows, hidden * 37 // 32] that receives the packed rows."""
        self.lib.tfh_layer_run_row_transport.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_char_p, ctypes.c_size_t]
        assert x.is_cuda and x.is_contiguous() and x.numel() == self.rows * self.g.hidden
        self._check(self.lib.tfh_layer_run_row_transport(self.h, x.data_ptr(), packed_out.data_ptr() if packed_out is not None else 0, self._err, 512))

    def capture(self, xs):
        """Captures one pass over each tensor of `xs` (or the single tensor `xs`), in order, into one graph."""
        xs = [xs] if not isinstance(xs, (list, tuple)) else list(xs)
        assert all(x.is_cuda and x.is_contiguous() for x in xs)
        ptrs = (ctypes.c_uint64 * len(xs))(*[x.data_ptr() for x in xs])
        return self._check(self.lib.tfh_layer_capture(self.h, ptrs, len(xs), self._err, 512))

    def time(self, order, warmup, steps):
        ms = ctypes.c_float(0)
        arr = (ctypes.c_int * len(order))(*order)
        self._check(self.lib.tfh_layer_time(self.h, arr, len(order), warmup, steps, ctypes.byref(ms), self._err, 512))
        return ms.value

    def time_phase(self, entry, x, iterations):
        ms = ctypes.c_float(0)
        self._check(self.lib.tfh_layer_time_phase(self.h, entry, x.data_ptr(), iterations, ctypes.byref(ms), self._err, 512))
        return ms.value

    def profile_step(self, x):
        """Milliseconds of (router, front-end, FC1, FC2, shared expert, sum, whole pass) of one eager pass."""
        ms = (ctypes.c_float * 7)()
        self._check(self.lib.tfh_layer_profile_step(self.h, x.data_ptr(), ms, self._err, 512))
        return list(ms)

    def profile_marks(self, xs, passes, exact=False):
        """Mean milliseconds of (front-end, FC1 + SwiGLU, FC2, sum, first mark to last, the FC1 + SwiGLU kernel alone) over `passes`
        eager passes of the layer's own schedule cycling through the inputs `xs`.  The first five are intervals between events
        recorded between the launches on the launch stream (a launch plus the gap to its neighbour); the last is between two
        events that take the kernel's own start and completion (`exact` runs only, whose other intervals carry that launch path's
        overhead; few rows only; 0 otherwise)."""
        ptrs = (ctypes.c_uint64 * len(xs))(*[x.data_ptr() for x in xs])
        ms = (ctypes.c_float * 6)()
        self._check(self.lib.tfh_layer_profile_marks(self.h, ptrs, len(xs), passes, int(exact), ms, self._err, 512))
        return list(ms)

    def pair_run(self, xa, tokens_a, live_a, xb, tokens_b, live_b, pool_shared=False):
        """Two owners of this layer through the pooled launch (Paired::run): returns both owners' outputs [rows][hidden] (BF16 bits).
        `pool_shared`: the shared expert runs once over the pooled rows instead of once per owner."""
        ia = (ctypes.c_int64 * self.rows)(*[int(t) for t in tokens_a])
        ib = (ctypes.c_int64 * self.rows)(*[int(t) for t in tokens_b])
        oa = np.empty((self.rows, self.g.hidden), np.uint16)
        ob = np.empty((self.rows, self.g.hidden), np.uint16)
        self._check(self.lib.tfh_layer_pair_run(self.h, xa.data_ptr(), ia, live_a, xb.data_ptr(), ib, live_b, int(pool_shared),
                                                oa.ctypes.data_as(ctypes.c_void_p), ob.ctypes.data_as(ctypes.c_void_p), self._err, 512))
        return oa, ob

    def spin_limit(self, limit):
        """Polls a wait inside the front-end launch may take before the waiter does the work itself (0: gives up at once)."""
        self.lib.tfh_layer_spin_limit.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
        self._check(self.lib.tfh_layer_spin_limit(self.h, limit, self._err, 512))

    def zero_sync(self):
        """The host's reset of the front-end's hand-off region (after a wait has expired)."""
        self.lib.tfh_layer_zero_sync.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]
        self._check(self.lib.tfh_layer_zero_sync(self.h, self._err, 512))

    def tap(self, name):
        dtype = TAPS.get(name) or EXTRA_TAPS[name]
        size = self._check(self.lib.tfh_layer_tap(self.h, name.encode(), None, 0, self._err, 512))
        out = np.empty(size // np.dtype(dtype).itemsize, dtype)
        self._check(self.lib.tfh_layer_tap(self.h, name.encode(), out.ctypes.data, size, self._err, 512))
        return out

    def run_geometry(self):
        """The geometry the layer runs with: the given one with the expert widths padded to multiples of 512 (zero weights)."""
        out = type(self.g)()
        self.lib.tfh_layer_geometry.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.lib.tfh_layer_geometry.restype = None
        self.lib.tfh_layer_geometry(self.h, ctypes.byref(out))
        return out

    def taps(self):
        g, rows = self.run_geometry(), self.rows
        K, H, I, S, B = g.topk, g.hidden, g.intermediate, g.shared_intermediate, g.act_block
        t = {n: self.tap(n) for n in TAPS}
        shape = {"logits": (rows, g.experts), "ids": (rows, K), "weights": (rows, K), "xq": (rows, H), "xs": (rows, H // B),
                 "xq_min": (rows, H), "xs_min": (rows, H // B), "h": (-1, I), "hq": (-1, I), "hs": (-1, I // B),
                 "route_out": (rows, K, H), "routed": (rows, H), "shared_up": (rows, 2 * S), "shared_act": (rows, S),
                 "shared_aq": (rows, S), "shared_as": (rows, S // B), "shared_down": (rows, H), "out": (rows, H)}
        for n, s in shape.items():
            t[n] = t[n].reshape(s)
        return t

    def census(self):
        counts = np.zeros(self.g.experts, np.uint32)
        self._check(self.lib.tfh_layer_census(self.h, counts.ctypes.data, self._err, 512))
        return counts

    def info(self):
        v = (ctypes.c_longlong * 8)()
        self.lib.tfh_layer_info(self.h, v)
        return dict(zip(["tile_m", "max_tiles", "scratch_bytes", "atlas_bytes", "expert_bytes", "scale_code_bytes", "raw_rows", "coded_rows"], v))


def checkpoint_contract(geometry, prefix):
    """What the loader requires of a checkpoint for one layer: a list of (tensor name, dtype string, shape tuple)."""
    lib = load()
    lib.tfh_checkpoint_contract.restype = ctypes.c_longlong
    lib.tfh_checkpoint_contract.argtypes = [ctypes.c_char_p, ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]
    need = lib.tfh_checkpoint_contract(prefix.encode(), ctypes.byref(geometry), None, 0)
    text = ctypes.create_string_buffer(need)
    lib.tfh_checkpoint_contract(prefix.encode(), ctypes.byref(geometry), text, need)
    rows = []
    for line in text.value.decode().splitlines():
        name, dtype, shape = line.split(" ")
        rows.append((name, dtype, tuple(int(d) for d in shape.split(","))))
    return rows


def checkpoint_layer(geometry, root, prefix):
    """Scans a safetensors checkpoint directory and assembles one layer's operands on the host (no device involved).
    Returns (dict of numpy arrays in the canonical layout, tensors in the checkpoint, shards)."""
    lib = load()
    g = geometry
    H, E, I, S = g.hidden, g.experts, g.intermediate, g.shared_intermediate
    shapes = [("gate_w", np.uint16, (E, H)), ("bias", np.float32, (E,)), ("bias_alt", np.float32, (E,)),
              ("w13", np.uint8, (E, 2 * I, H // 2)), ("s13", np.uint8, (E, 2 * I, H // 32)), ("w2", np.uint8, (E, H, I // 2)),
              ("s2", np.uint8, (E, H, I // 32)), ("sh_w13", np.uint8, (2 * S, H)), ("sh_s13", np.uint8, (2 * S // g.shared_bn, H // g.shared_bk)),
              ("sh_w2", np.uint8, (H, S)), ("sh_s2", np.uint8, (H // g.shared_bn, S // g.shared_bk))]
    arrays = {n: np.empty(shape, dtype) for n, dtype, shape in shapes}
    outs = (ctypes.c_void_p * 11)(*[arrays[n].ctypes.data for n, _, _ in shapes])
    sizes = (ctypes.c_size_t * 11)(*[arrays[n].nbytes for n, _, _ in shapes])
    counts = (ctypes.c_size_t * 2)()
    err = ctypes.create_string_buffer(512)
    lib.tfh_checkpoint_layer.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_char_p, ctypes.c_size_t]
    if lib.tfh_checkpoint_layer(root.encode(), prefix.encode(), ctypes.byref(geometry), outs, sizes, counts, err, 512) != 0:
        raise HostError(err.value.decode())
    return arrays, counts[0], counts[1]
