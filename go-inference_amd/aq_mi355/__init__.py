"""ctypes binding of libaq_mi355.so -- plumbing for tests, the smoke check and the benchmark.

The product is the shared library; this module only loads it and marshals numpy
arrays and device pointers into its C ABI (include/aq_mi355.h, include/aq_mi355_host.h).
It raises if the library has not been built: there is no fallback path.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libaq_mi355.so")

AQ_OK = 0
AQ_ERR_ARG = -1
AQ_ERR_SHAPE = -2
AQ_ERR_UNSUPPORTED = -3
AQ_ERR_INDEX = -4
AQ_ERR_NOMEM = -5
AQ_ERR_NODEVICE = -6
AQ_ERR_SIZE = -7
AQ_OUT_F32 = 0x1

AQ_IN_F32 = 2
AQ_LOGITS_BF16 = 4
AQ_BF16_STEPS = 8
AQ_W_TILED = 0x10
AQ_ACT_GELU_TANH = 1
AQ_ACT_SILU = 2
OP_QMV = 0
OP_QMM = 1

_c = ctypes
_vp, _i, _u, _sz, _f = _c.c_void_p, _c.c_int, _c.c_uint, _c.c_size_t, _c.c_float
_cp = _c.c_char_p

class HostLinear(ctypes.Structure):
    """aqh_linear (include/aq_mi355_host.h)."""
    _fields_ = [("weight", _vp), ("scales", _vp), ("biases", _vp), ("bias", _vp),
                ("weight_len", _sz), ("scales_len", _sz), ("biases_len", _sz), ("bias_len", _sz),
                ("out_dim", _i), ("in_dim", _i), ("group_size", _i), ("bits", _i), ("quantised", _i),
                ("experts", _i), ("expert_rows", _i)]

    def view(self, which):
        """numpy uint8 view of weight / scales / biases / bias (valid while the file stays open)."""
        ptr, n = getattr(self, which), getattr(self, which + "_len")
        if not ptr:
            return None
        return np.ctypeslib.as_array(ctypes.cast(ptr, ctypes.POINTER(ctypes.c_uint8)), shape=(n,))


class DeviceLinear(ctypes.Structure):
    """aq_device_linear (include/aq_mi355.h)."""
    _fields_ = [("weight", _vp), ("scales", _vp), ("biases", _vp), ("rows", _i), ("in_dim", _i), ("group_size", _i),
                ("bits", _i), ("experts", _i)]


class GgufAffineLayout(ctypes.Structure):
    """aq_gguf_affine_layout (include/aq_mi355.h)."""
    _fields_ = [("bits", _i), ("group_size", _i), ("packed_cols", _c.c_int64), ("groups", _c.c_int64),
                ("src_bytes", _c.c_uint64), ("packed_bytes", _c.c_uint64), ("scales_bytes", _c.c_uint64)]


GGUF_F32, GGUF_Q4_0, GGUF_Q4_1, GGUF_Q8_0, GGUF_Q4_K, GGUF_Q5_K, GGUF_Q6_K = 0, 2, 3, 8, 12, 13, 14


# name -> (restype, argtypes); every symbol include/*.h declares
PROTOTYPES = {
    "aq_version": (_cp, []),
    "aq_last_error": (_cp, []),
    "aq_create": (_i, [_i, _c.POINTER(_vp)]),
    "aq_destroy": (None, [_vp]),
    "aq_use_stream": (_i, [_vp, _vp]),
    "aq_use_own_stream": (_i, [_vp]),
    "aq_device_name": (_i, [_vp, _cp, _sz]),
    "aq_malloc": (_i, [_vp, _sz, _c.POINTER(_vp)]),
    "aq_free": (_i, [_vp, _vp]),
    "aq_h2d": (_i, [_vp, _vp, _vp, _sz]),
    "aq_d2h": (_i, [_vp, _vp, _vp, _sz]),
    "aq_d2d": (_i, [_vp, _vp, _vp, _sz]),
    "aq_fill_zero": (_i, [_vp, _vp, _sz]),
    "aq_sync": (_i, [_vp]),
    "aq_timer_start": (_i, [_vp]),
    "aq_timer_stop": (_i, [_vp, _c.POINTER(_f)]),
    "aq_capture_begin": (_i, [_vp]),
    "aq_capture_end": (_i, [_vp, _c.POINTER(_vp)]),
    "aq_graph_launch": (_i, [_vp, _vp]),
    "aq_graph_destroy": (None, [_vp]),
    "aq_qmv": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _u]),
    "aq_qmm": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _u]),
    "aq_qmv_multi": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _u]),
    "aq_qmm_multi": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _u]),
    "aq_reserve_workspace": (_i, [_vp, _i, _i]),
    "aq_reserve_workspace_bytes": (_i, [_vp, _sz]),
    "aq_workspace_bytes": (_sz, [_vp]),
    "aq_gather_qmv": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _u]),
    "aq_qmv_gate_up": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _u]),
    "aq_gather_qmv_gate_up": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i,
                                   _u]),
    "aq_qmv_act": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _u]),
    "aq_gather_qmv_act": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i,
                               _u]),
    "aq_act_mul": (_i, [_vp, _vp, _vp, _vp, _c.c_int64, _i]),
    "aq_moe_route": (_i, [_vp, _vp, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _u]),
    "aq_moe_combine": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _u]),
    "aq_qmv_greedy": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i]),
    "aq_probe_read": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "aq_qmv_greedy_selected": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i]),
    "aq_qmv_greedy_static": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i]),
    "aq_qmv_scores": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i, _i, _i, _i]),
    "aq_packed_topk": (_i, [_vp, _vp, _c.c_int64, _i, _vp]),
    "aq_pack_best": (_c.c_uint64, [_f, _i]),
    "aq_unpack_best": (_i, [_c.c_uint64, _f, _i, _c.POINTER(_i), _c.POINTER(_f)]),
    "aq_upload_linear": (_i, [_vp, _c.POINTER(HostLinear), _c.POINTER(DeviceLinear)]),
    "aq_tile_device_linear": (_i, [_vp, _c.POINTER(DeviceLinear)]),
    "aq_upload_fused_gate_up": (_i, [_vp, _c.POINTER(HostLinear), _c.POINTER(HostLinear), _c.POINTER(DeviceLinear)]),
    "aq_free_device_linear": (_i, [_vp, _c.POINTER(DeviceLinear)]),
    "aq_dequant_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _c.c_int64, _i, _i, _i]),
    "aq_tiled_bytes": (_c.c_int64, [_c.c_int64, _i, _i, _i]),
    "aq_tile_weights": (_i, [_vp, _vp, _vp, _vp, _c.c_int64, _i, _i, _i, _vp]),
    "aq_untile_weights": (_i, [_vp, _vp, _c.c_int64, _i, _i, _i, _vp, _vp, _vp]),
    "aq_packed_topk_sample": (_i, [_vp, _vp, _i, _c.c_float, _c.c_float, _c.c_float, _c.c_double, _vp]),
    "aq_gguf_affine_layout_of": (_i, [_i, _c.c_int64, _c.c_int64, _c.POINTER(GgufAffineLayout)]),
    "aq_gguf_to_affine": (_i, [_vp, _i, _vp, _c.c_uint64, _c.c_int64, _c.c_int64, _vp, _vp, _vp]),
    "aq_matvec_host": (_i, [_vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _i, _i, _i, _i, _vp, _sz]),
    "aq_proj_quant_matmul_host": (_i, [_vp, _vp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _i, _i, _i, _i, _i]),
    "aq_variant_count": (_i, [_i]),
    "aq_variant_name": (_cp, [_i, _i]),
    "aq_force_variant": (_i, [_vp, _i, _i]),
    "aq_last_variant": (_cp, [_vp, _i]),
    "aqh_last_error": (_cp, []),
    "aqh_register_rocm_backend": (None, []),
    "aqh_backend_quant_registered": (_i, [_cp, _cp]),
    "aqh_backend_quant_bits": (_i, [_cp, _cp]),
    "aqh_backend_quant_matvec": (_i, [_cp, _cp, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _i, _i, _i, _i, _vp, _sz,
                                      _c.POINTER(_sz)]),
    "aqh_proj_quant_matmul_into": (_i, [_vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _i, _i, _i, _i, _i]),
    "aqh_concat_quant_rows": (_i, [_vp, _sz, _vp, _sz, _vp, _i, _vp, _sz, _vp, _sz, _vp, _i, _i, _i, _i, _i, _i, _i,
                                   _vp, _vp, _vp, _c.POINTER(_i)]),
    "aqh_safetensors_open": (_i, [_cp, _c.POINTER(_vp)]),
    "aqh_safetensors_close": (None, [_vp]),
    "aqh_safetensors_count": (_i, [_vp]),
    "aqh_safetensors_name": (_i, [_vp, _i, _cp, _sz]),
    "aqh_safetensors_tensor": (_i, [_vp, _cp, _cp, _c.POINTER(_c.c_int64), _c.POINTER(_i), _c.POINTER(_vp),
                                    _c.POINTER(_sz)]),
    "aqh_load_linear": (_i, [_vp, _cp, _i, _c.POINTER(HostLinear)]),
    "aqh_repack_b1_to_b2": (_i, [_vp, _sz, _sz, _sz, _i, _i, _i, _vp, _sz]),
    "aqh_affine_geometry": (None, [_i, _i, _i, _c.POINTER(_i), _c.POINTER(_i)]),
}


def tiled_bytes(N, K, group_size=64, bits=4):
    return load().aq_tiled_bytes(N, K, group_size, bits)


class AqError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("aq_mi355 error %d: %s" % (code, msg))
        self.code = code
        self.msg = msg


_lib = None


def load():
    """dlopen the in-tree library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("libaq_mi355.so is not built (run: python go-inference_amd/build.py); "
                           "there is no non-HIP path")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _ptr(obj):
    """Device pointer (int / DeviceBuffer) or host numpy array -> void*."""
    if obj is None:
        return None
    if isinstance(obj, DeviceBuffer):
        return obj.ptr
    if isinstance(obj, np.ndarray):
        return obj.ctypes.data
    return int(obj)


class DeviceBuffer:
    """A hipMalloc'd span owned through aq_malloc / aq_free."""

    def __init__(self, ctx, nbytes):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = _vp()
        ctx._check(ctx.lib.aq_malloc(ctx.handle, self.nbytes, ctypes.byref(p)))
        self.ptr = p.value or 0

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        self.ctx._check(self.ctx.lib.aq_h2d(self.ctx.handle, self.ptr, arr.ctypes.data, arr.nbytes))
        return self

    def download(self, dtype, count=None):
        dtype = np.dtype(dtype)
        if count is None:
            count = self.nbytes // dtype.itemsize
        out = np.empty(count, dtype=dtype)
        self.ctx._check(self.ctx.lib.aq_d2h(self.ctx.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            self.ctx.lib.aq_free(self.ctx.handle, self.ptr)
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Context:
    def __init__(self, device=0):
        self.lib = load()
        h = _vp()
        rc = self.lib.aq_create(device, ctypes.byref(h))
        if rc != AQ_OK:
            raise AqError(rc, self.lib.aq_last_error().decode())
        self.handle = h

    def close(self):
        if self.handle:
            self.lib.aq_destroy(self.handle)
            self.handle = None

    def _check(self, rc):
        if rc != AQ_OK:
            raise AqError(rc, self.lib.aq_last_error().decode())

    def device_name(self):
        buf = ctypes.create_string_buffer(256)
        self._check(self.lib.aq_device_name(self.handle, buf, 256))
        return buf.value.decode()

    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def to_device(self, arr):
        arr = np.ascontiguousarray(arr)
        return DeviceBuffer(self, max(arr.nbytes, 16)).upload(arr)

    def sync(self):
        self._check(self.lib.aq_sync(self.handle))

    def fill_zero(self, buf, nbytes=None):
        self._check(self.lib.aq_fill_zero(self.handle, _ptr(buf), buf.nbytes if nbytes is None else nbytes))

    def timer_start(self):
        self._check(self.lib.aq_timer_start(self.handle))

    def timer_stop(self):
        ms = _f()
        self._check(self.lib.aq_timer_stop(self.handle, ctypes.byref(ms)))
        return ms.value

    def capture_begin(self):
        self._check(self.lib.aq_capture_begin(self.handle))

    def capture_end(self):
        g = _vp()
        self._check(self.lib.aq_capture_end(self.handle, ctypes.byref(g)))
        return g

    def graph_launch(self, graph):
        self._check(self.lib.aq_graph_launch(self.handle, graph))

    def graph_destroy(self, graph):
        self.lib.aq_graph_destroy(graph)

    def qmv(self, x, w, s, b, y, M, K, N, group_size=64, bits=4, flags=0):
        self._check(self.lib.aq_qmv(self.handle, _ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(y), M, K, N, group_size,
                                    bits, flags))

    def qmm(self, x, w, s, b, y, M, K, N, group_size=64, bits=4, flags=0):
        self._check(self.lib.aq_qmm(self.handle, _ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(y), M, K, N, group_size,
                                    bits, flags))

    def qmv_multi(self, x, ws, ss, bs, ys, Ns, M, K, group_size=64, bits=4, flags=0):
        """ws, ss, bs, ys: sequences of device buffers (one per weight matrix); Ns: their row counts."""
        n = len(ws)
        arr = lambda seq: (_c.c_void_p * n)(*[_ptr(t) for t in seq])
        self._check(self.lib.aq_qmv_multi(self.handle, _ptr(x), n, arr(ws), arr(ss), arr(bs), arr(ys),
                                          (_c.c_int * n)(*Ns), M, K, group_size, bits, flags))

    def qmm_multi(self, x, ws, ss, bs, ys, Ns, M, K, group_size=64, bits=4, flags=0):
        """aq_qmm over several weight matrices that share x: one pass over x for the members that need the same form."""
        n = len(ws)
        arr = lambda seq: (_c.c_void_p * n)(*[_ptr(t) for t in seq])
        self._check(self.lib.aq_qmm_multi(self.handle, _ptr(x), n, arr(ws), arr(ss), arr(bs), arr(ys),
                                          (_c.c_int * n)(*Ns), M, K, group_size, bits, flags))

    def prepared_qmv(self, x, w, s, b, y, M, K, N, group_size=64, bits=4, flags=0):
        """The same call as qmv with every argument converted once: returns a function of no arguments.  For loops
        whose per-call host work would otherwise be this wrapper's argument handling."""
        fn, check, h = self.lib.aq_qmv, self._check, self.handle
        args = (_ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(y), M, K, N, group_size, bits, flags)
        return lambda: check(fn(h, *args))

    def prepared_qmv_multi(self, x, ws, ss, bs, ys, Ns, M, K, group_size=64, bits=4, flags=0):
        """qmv_multi with its pointer arrays built once: returns a function of no arguments."""
        n = len(ws)
        arr = lambda seq: (_c.c_void_p * n)(*[_ptr(t) for t in seq])
        fn, check, h = self.lib.aq_qmv_multi, self._check, self.handle
        args = (_ptr(x), n, arr(ws), arr(ss), arr(bs), arr(ys), (_c.c_int * n)(*Ns), M, K, group_size, bits, flags)
        return lambda: check(fn(h, *args))

    def tile_weights(self, w, s, b, N, K, group_size=64, bits=4):
        """The tile-major tensor (a new device buffer) of the MLX arrays w, s, b."""
        n = tiled_bytes(N, K, group_size, bits)
        if n < 0:
            raise AqError(AQ_ERR_UNSUPPORTED, "no tile-major layout for this geometry")
        out = self.alloc(n)
        self._check(self.lib.aq_tile_weights(self.handle, _ptr(w), _ptr(s), _ptr(b), N, K, group_size, bits, out.ptr))
        return out

    def untile_weights(self, tiled, N, K, w, s, b, group_size=64, bits=4):
        self._check(self.lib.aq_untile_weights(self.handle, _ptr(tiled), N, K, group_size, bits, _ptr(w), _ptr(s), _ptr(b)))

    def reserve_workspace(self, M, K):
        self._check(self.lib.aq_reserve_workspace(self.handle, M, K))

    def reserve_workspace_bytes(self, nbytes):
        self._check(self.lib.aq_reserve_workspace_bytes(self.handle, nbytes))

    def workspace_bytes(self):
        return int(self.lib.aq_workspace_bytes(self.handle))

    def gather_qmv(self, x, w, s, b, lhs, rhs, y, routes, x_rows, K, N, num_experts, expert_rows, row_base=0,
                   group_size=64, bits=4, flags=0):
        self._check(self.lib.aq_gather_qmv(self.handle, _ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(lhs), _ptr(rhs),
                                           _ptr(y), routes, x_rows, K, N, num_experts, expert_rows, row_base,
                                           group_size, bits, flags))

    def qmv_gate_up(self, x, gate, up, y, M, K, N, group_size=64, bits=4, act=AQ_ACT_GELU_TANH, flags=0):
        """gate, up: (packed, scales, biases) device buffers of the two projections."""
        self._check(self.lib.aq_qmv_gate_up(self.handle, _ptr(x), _ptr(gate[0]), _ptr(gate[1]), _ptr(gate[2]),
                                            _ptr(up[0]), _ptr(up[1]), _ptr(up[2]), _ptr(y), M, K, N, group_size, bits,
                                            act, flags))

    def gather_qmv_gate_up(self, x, w, s, b, lhs, rhs, y, routes, x_rows, K, N, num_experts, expert_rows,
                           gate_row_base, up_row_base, group_size=64, bits=4, act=AQ_ACT_GELU_TANH, flags=0):
        self._check(self.lib.aq_gather_qmv_gate_up(self.handle, _ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(lhs),
                                                   _ptr(rhs), _ptr(y), routes, x_rows, K, N, num_experts, expert_rows,
                                                   gate_row_base, up_row_base, group_size, bits, act, flags))

    def qmv_act(self, gate_x, up_x, w, s, b, y, M, K, N, group_size=64, bits=4, act=AQ_ACT_GELU_TANH, flags=0):
        self._check(self.lib.aq_qmv_act(self.handle, _ptr(gate_x), _ptr(up_x), _ptr(w), _ptr(s), _ptr(b), _ptr(y), M,
                                        K, N, group_size, bits, act, flags))

    def gather_qmv_act(self, gate_x, up_x, w, s, b, lhs, rhs, y, routes, x_rows, K, N, num_experts, expert_rows,
                       row_base=0, group_size=64, bits=4, act=AQ_ACT_GELU_TANH, flags=0):
        self._check(self.lib.aq_gather_qmv_act(self.handle, _ptr(gate_x), _ptr(up_x), _ptr(w), _ptr(s), _ptr(b),
                                               _ptr(lhs), _ptr(rhs), _ptr(y), routes, x_rows, K, N, num_experts,
                                               expert_rows, row_base, group_size, bits, act, flags))

    def act_mul(self, gate, up, y, n, act=AQ_ACT_GELU_TANH):
        self._check(self.lib.aq_act_mul(self.handle, _ptr(gate), _ptr(up), _ptr(y), n, act))

    def moe_route(self, logits, rows, num_experts, top_k, ids, weights, token_of_route=None, expert_scales=None,
                  normalise=True, flags=0):
        self._check(self.lib.aq_moe_route(self.handle, _ptr(logits), rows, num_experts, top_k, _ptr(expert_scales),
                                          1 if normalise else 0, _ptr(ids), _ptr(weights), _ptr(token_of_route), flags))

    def moe_combine(self, route_rows, weights, out, rows, top_k, n, flags=0):
        self._check(self.lib.aq_moe_combine(self.handle, _ptr(route_rows), _ptr(weights), _ptr(out), rows, top_k, n,
                                            flags))

    def qmv_greedy(self, x, w, s, b, best, M, K, N, group_size=64, bits=4, suppress=None, suppress_count=0):
        self._check(self.lib.aq_qmv_greedy(self.handle, _ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(suppress), suppress_count,
                                           _ptr(best), M, K, N, group_size, bits))

    def probe_read(self, w, s, b, K, N, mode=0):
        self._check(self.lib.aq_probe_read(self.handle, _ptr(w), _ptr(s), _ptr(b), K, N, mode))

    def qmv_greedy_selected(self, x, w, s, b, rows, count, best, K, N, group_size=64, bits=4):
        self._check(self.lib.aq_qmv_greedy_selected(self.handle, _ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(rows), count,
                                                    _ptr(best), K, N, group_size, bits))

    def qmv_greedy_static(self, x, w, s, b, best, K, N, group_size=64, bits=4, suppress=None, suppress_count=0):
        self._check(self.lib.aq_qmv_greedy_static(self.handle, _ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(suppress),
                                                  suppress_count, _ptr(best), K, N, group_size, bits))

    def qmv_scores(self, x, w, s, b, scores, M, K, N, group_size=64, bits=4, suppress=None, suppress_count=0):
        self._check(self.lib.aq_qmv_scores(self.handle, _ptr(x), _ptr(w), _ptr(s), _ptr(b), _ptr(suppress), suppress_count,
                                           _ptr(scores), M, K, N, group_size, bits))

    def packed_topk(self, scores, count, top_k, out):
        self._check(self.lib.aq_packed_topk(self.handle, _ptr(scores), count, top_k, _ptr(out)))

    def upload_linear(self, host_linear):
        out = DeviceLinear()
        self._check(self.lib.aq_upload_linear(self.handle, ctypes.byref(host_linear), ctypes.byref(out)))
        return out

    def upload_fused_gate_up(self, gate, up):
        out = DeviceLinear()
        self._check(self.lib.aq_upload_fused_gate_up(self.handle, ctypes.byref(gate), ctypes.byref(up), ctypes.byref(out)))
        return out

    def tile_device_linear(self, dev_linear):
        self._check(self.lib.aq_tile_device_linear(self.handle, ctypes.byref(dev_linear)))

    def free_device_linear(self, dev_linear):
        self._check(self.lib.aq_free_device_linear(self.handle, ctypes.byref(dev_linear)))

    def dequant_f32(self, w, s, b, out, N, K, group_size=64, bits=4):
        self._check(self.lib.aq_dequant_f32(self.handle, _ptr(w), _ptr(s), _ptr(b), _ptr(out), N, K, group_size,
                                            bits))

    def packed_topk_sample(self, top, top_k, temperature, top_p, softcap, draw, out):
        self._check(self.lib.aq_packed_topk_sample(self.handle, _ptr(top), top_k, temperature, top_p, softcap, draw, _ptr(out)))

    def gguf_to_affine(self, gguf_type, src, src_bytes, rows, cols, packed, scales, biases):
        """GGUF blocks at `src` (device) -> packed / scales / biases (device), sized by gguf_affine_layout()."""
        self._check(self.lib.aq_gguf_to_affine(self.handle, gguf_type, _ptr(src), src_bytes, rows, cols, _ptr(packed),
                                               _ptr(scales), _ptr(biases)))

    def force_variant(self, op, variant):
        self._check(self.lib.aq_force_variant(self.handle, op, variant))

    def last_variant(self, op):
        return self.lib.aq_last_variant(self.handle, op).decode()

    # host-slice entry points -------------------------------------------------
    def matvec_host(self, x, packed, scales, biases, out_dim, in_dim, group_size, bits):
        """model.QuantMatVec.MatVec over host bytes; returns out_dim*2 bytes (uint8 array)."""
        x, packed, scales, biases = (np.ascontiguousarray(a).view(np.uint8).reshape(-1)
                                     for a in (x, packed, scales, biases))
        out = np.zeros(max(out_dim, 0) * 2, dtype=np.uint8)
        self._check(self.lib.aq_matvec_host(self.handle, x.ctypes.data, x.size, packed.ctypes.data, packed.size,
                                            scales.ctypes.data, scales.size, biases.ctypes.data, biases.size,
                                            out_dim, in_dim, group_size, bits, out.ctypes.data, out.size))
        return out

    def proj_quant_matmul_host(self, x_f32, packed, scales, biases, M, K, N, group_size, bits):
        x_f32 = np.ascontiguousarray(x_f32, dtype=np.float32).reshape(-1)
        packed, scales, biases = (np.ascontiguousarray(a).view(np.uint8).reshape(-1) for a in (packed, scales, biases))
        out = np.zeros(max(M * N, 0), dtype=np.float32)
        self._check(self.lib.aq_proj_quant_matmul_host(self.handle, out.ctypes.data, x_f32.ctypes.data, x_f32.size,
                                                       packed.ctypes.data, packed.size, scales.ctypes.data,
                                                       scales.size, biases.ctypes.data, biases.size, M, K, N,
                                                       group_size, bits))
        return out.reshape(M, N)


class SafetensorsFile:
    """aqh_safetensors_* : a memory-mapped safetensors file read by the library's own loader."""

    def __init__(self, path):
        self.lib = load()
        h = _vp()
        rc = self.lib.aqh_safetensors_open(os.fsencode(path), ctypes.byref(h))
        if rc != AQ_OK:
            raise AqError(rc, self.lib.aqh_last_error().decode())
        self.handle = h

    def close(self):
        if self.handle:
            self.lib.aqh_safetensors_close(self.handle)
            self.handle = None

    def names(self):
        out = []
        buf = ctypes.create_string_buffer(1024)
        for i in range(self.lib.aqh_safetensors_count(self.handle)):
            if self.lib.aqh_safetensors_name(self.handle, i, buf, 1024) != AQ_OK:
                raise AqError(AQ_ERR_SIZE, self.lib.aqh_last_error().decode())
            out.append(buf.value.decode())
        return out

    def tensor(self, name):
        """(dtype, shape, uint8 view)"""
        dtype = ctypes.create_string_buffer(16)
        shape = (_c.c_int64 * 8)()
        rank, data, n = _i(0), _vp(), _sz(0)
        rc = self.lib.aqh_safetensors_tensor(self.handle, name if isinstance(name, bytes) else name.encode(), dtype, shape, ctypes.byref(rank), ctypes.byref(data),
                                             ctypes.byref(n))
        if rc != AQ_OK:
            raise AqError(rc, self.lib.aqh_last_error().decode())
        view = (np.ctypeslib.as_array(ctypes.cast(data, ctypes.POINTER(ctypes.c_uint8)), shape=(n.value,))
                if n.value else np.zeros(0, np.uint8))
        return dtype.value.decode(), [int(shape[i]) for i in range(rank.value)], view

    def load_linear(self, prefix, in_dim):
        """model.LoadLinear; None when prefix.weight is absent."""
        out = HostLinear()
        rc = self.lib.aqh_load_linear(self.handle, prefix.encode(), in_dim, ctypes.byref(out))
        if rc == AQ_ERR_INDEX:
            return None
        if rc != AQ_OK:
            raise AqError(rc, self.lib.aqh_last_error().decode())
        return out


def gguf_affine_layout(gguf_type, rows, cols):
    """What a GGUF tensor of this type and shape repacks to (no device needed); raises AqError as the Go
    repack returns errors."""
    lib = load()
    lay = GgufAffineLayout()
    rc = lib.aq_gguf_affine_layout_of(gguf_type, rows, cols, ctypes.byref(lay))
    if rc != AQ_OK:
        raise AqError(rc, lib.aq_last_error().decode())
    return lay


def pack_best(score, token):
    return int(load().aq_pack_best(score, token))


def unpack_best(packed, softcap=0.0, vocab_size=2 ** 31 - 1):
    """(token, score) of a packed greedy / top-k value; raises AqError as the Go helper returns errors."""
    lib = load()
    tok, sc = _c.c_int(0), _c.c_float(0)
    rc = lib.aq_unpack_best(packed, softcap, vocab_size, ctypes.byref(tok), ctypes.byref(sc))
    if rc != AQ_OK:
        raise AqError(rc, lib.aq_last_error().decode())
    return tok.value, sc.value


def variant_names(op):
    lib = load()
    return [lib.aq_variant_name(op, i).decode() for i in range(lib.aq_variant_count(op))]
