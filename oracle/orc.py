"""ctypes binding of oracle/liborc.so -- TEST INFRASTRUCTURE.

Only tests/, the smoke check and the benchmark's cpu_baseline leg import this module;
the product (go-inference_amd/) never does.  `build()` runs `make -C oracle`.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liborc.so")

ORC_OK = 0
ORC_ERR_BITS = -1
ORC_ERR_DIMS = -2
ORC_ERR_SIZE = -3
ORC_ERR_INDEX = -4

_lib = None


def build(force=False):
    if force or not os.path.exists(LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.orc_f32_to_bf16.restype = ctypes.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.orc_bf16_to_f32.restype = ctypes.c_float
        _lib.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.orc_extract_code.restype = ctypes.c_uint32
        _lib.orc_extract_code.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int]
        _lib.orc_set_code.restype = None
        _lib.orc_set_code.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_uint32]
        _lib.orc_max_threads.restype = ctypes.c_int
    return _lib


def _u8(a):
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1)


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else None


class OracleError(ValueError):
    def __init__(self, code):
        super().__init__("oracle rejected the arguments (code %d)" % code)
        self.code = code


def _check(rc):
    if rc != ORC_OK:
        raise OracleError(rc)


def f32_to_bf16(v):
    return int(lib().orc_f32_to_bf16(ctypes.c_float(v)))


def bf16_to_f32(h):
    return float(lib().orc_bf16_to_f32(ctypes.c_uint16(h)))


def extract_code(row_bytes, bit_off, bits):
    row_bytes = _u8(row_bytes)
    return int(lib().orc_extract_code(_p(row_bytes), bit_off, bits))


def set_code(row_bytes, bit_off, bits, code):
    assert row_bytes.dtype == np.uint8 and row_bytes.flags.c_contiguous
    lib().orc_set_code(_p(row_bytes), bit_off, bits, code)


def dequantize(packed, scales, biases, out_dim, in_dim, bits, group_size):
    packed, scales, biases = _u8(packed), _u8(scales), _u8(biases)
    out = np.empty(max(out_dim, 0) * max(in_dim, 0), dtype=np.float32)
    rc = lib().orc_dequantize(_p(packed), ctypes.c_size_t(packed.size), _p(scales), ctypes.c_size_t(scales.size),
                              _p(biases), ctypes.c_size_t(biases.size), out_dim, in_dim, bits, group_size, _p(out))
    _check(rc)
    return out.reshape(out_dim, in_dim)


def quantize(values, out_dim, in_dim, bits, group_size):
    values = np.ascontiguousarray(values, dtype=np.float32).reshape(-1)
    packed = np.zeros(max(out_dim * in_dim * bits // 8, 1), dtype=np.uint8)
    sb = max(out_dim * (in_dim // max(group_size, 1)) * 2, 1)
    scales = np.zeros(sb, dtype=np.uint8)
    biases = np.zeros(sb, dtype=np.uint8)
    rc = lib().orc_quantize(_p(values), ctypes.c_size_t(values.size), out_dim, in_dim, bits, group_size, _p(packed),
                            _p(scales), _p(biases))
    _check(rc)
    return packed, scales, biases


def repack_b1_to_b2(packed, out_dim, in_dim):
    packed = _u8(packed)
    out = np.zeros(max(out_dim * in_dim // 4, 1), dtype=np.uint8)
    _check(lib().orc_repack_b1_to_b2(_p(packed), ctypes.c_size_t(packed.size), out_dim, in_dim, _p(out)))
    return out


def matnt_quant_host(x_f32, packed, scales, biases, M, K, N, group_size, bits, threads=1):
    x = np.ascontiguousarray(x_f32, dtype=np.float32).reshape(-1)
    packed, scales, biases = _u8(packed), _u8(scales), _u8(biases)
    out = np.zeros(M * N, dtype=np.float32)
    _check(lib().orc_matnt_quant_host(_p(out), _p(x), _p(packed), _p(scales), _p(biases), M, K, N, group_size, bits,
                                      threads))
    return out.reshape(M, N)


def reference_affine_matvec(x, packed, scales, biases, out_dim, in_dim, group_size, bits):
    """bf16 bytes in, bf16 bytes (uint8 array, out_dim*2) out."""
    x, packed, scales, biases = _u8(x), _u8(packed), _u8(scales), _u8(biases)
    out = np.zeros(max(out_dim, 0) * 2, dtype=np.uint8)
    rc = lib().orc_reference_affine_matvec(_p(x), ctypes.c_size_t(x.size), _p(packed), ctypes.c_size_t(packed.size),
                                           _p(scales), ctypes.c_size_t(scales.size), _p(biases),
                                           ctypes.c_size_t(biases.size), out_dim, in_dim, group_size, bits, _p(out))
    _check(rc)
    return out


def hip_reference_projection(x_f32, weights_u32, scales_u16, biases_u16, rows, cols, group_size, bits):
    x = np.ascontiguousarray(x_f32, dtype=np.float32).reshape(-1)
    w = np.ascontiguousarray(weights_u32, dtype=np.uint32).reshape(-1)
    s = np.ascontiguousarray(scales_u16, dtype=np.uint16).reshape(-1)
    b = np.ascontiguousarray(biases_u16, dtype=np.uint16).reshape(-1)
    out = np.zeros(max(rows, 0), dtype=np.float32)
    rc = lib().orc_hip_reference_projection(_p(x), ctypes.c_size_t(x.size), _p(w), ctypes.c_size_t(w.size), _p(s),
                                            ctypes.c_size_t(s.size), _p(b), ctypes.c_size_t(b.size), rows, cols,
                                            group_size, bits, _p(out))
    _check(rc)
    return out


def hip_reference_projection_batch(x_f32, tokens, weights_u32, scales_u16, biases_u16, rows, cols, group_size, bits):
    x = np.ascontiguousarray(x_f32, dtype=np.float32).reshape(-1)
    w = np.ascontiguousarray(weights_u32, dtype=np.uint32).reshape(-1)
    s = np.ascontiguousarray(scales_u16, dtype=np.uint16).reshape(-1)
    b = np.ascontiguousarray(biases_u16, dtype=np.uint16).reshape(-1)
    out = np.zeros(tokens * rows, dtype=np.float32)
    _check(lib().orc_hip_reference_projection_batch(_p(x), tokens, _p(w), _p(s), _p(b), rows, cols, group_size, bits,
                                                    _p(out)))
    return out.reshape(tokens, rows)


def gather_qmv(x_u16, x_rows, packed_u32, scales_u16, biases_u16, lhs, rhs, routes, num_experts, expert_rows,
               row_base, N, K, group_size, bits):
    """Returns (float64 sums [routes,N], bf16 bits [routes,N])."""
    x = np.ascontiguousarray(x_u16, dtype=np.uint16).reshape(-1)
    w = np.ascontiguousarray(packed_u32, dtype=np.uint32).reshape(-1)
    s = np.ascontiguousarray(scales_u16, dtype=np.uint16).reshape(-1)
    b = np.ascontiguousarray(biases_u16, dtype=np.uint16).reshape(-1)
    lhs_a = None if lhs is None else np.ascontiguousarray(lhs, dtype=np.int32)
    rhs_a = np.ascontiguousarray(rhs, dtype=np.int32)
    o64 = np.zeros(max(routes * N, 1), dtype=np.float64)
    o16 = np.zeros(max(routes * N, 1), dtype=np.uint16)
    rc = lib().orc_gather_qmv(_p(x), x_rows, _p(w), _p(s), _p(b), _p(lhs_a), _p(rhs_a), routes, num_experts,
                              expert_rows, row_base, N, K, group_size, bits, _p(o64), _p(o16))
    _check(rc)
    return o64[:routes * N].reshape(routes, N), o16[:routes * N].reshape(routes, N)


ACT_GELU_TANH = 1
ACT_SILU = 2


def act_multiply(act, gate_f32, up_f32):
    g = np.ascontiguousarray(gate_f32, dtype=np.float32)
    u = np.ascontiguousarray(up_f32, dtype=np.float32)
    assert g.shape == u.shape
    out = np.zeros(g.shape, dtype=np.float32)
    _check(lib().orc_act_multiply(act, _p(g), _p(u), ctypes.c_int64(g.size), _p(out)))
    return out


def act_gate_mul_bf16(act, gate_u16, up_u16):
    g = np.ascontiguousarray(gate_u16, dtype=np.uint16)
    u = np.ascontiguousarray(up_u16, dtype=np.uint16)
    assert g.shape == u.shape
    out = np.zeros(g.shape, dtype=np.uint16)
    _check(lib().orc_act_gate_mul_bf16(act, _p(g), _p(u), ctypes.c_int64(g.size), _p(out)))
    return out


def moe_route(logits_f32, top_k, expert_scales=None, normalise=True):
    """logits [rows, experts] -> (ids int32 [rows, top_k], weights float32 [rows, top_k])."""
    lg = np.ascontiguousarray(logits_f32, dtype=np.float32)
    rows, experts = lg.shape
    sc = None if expert_scales is None else np.ascontiguousarray(expert_scales, dtype=np.float32)
    ids = np.zeros((rows, max(top_k, 1)), dtype=np.int32)
    w = np.zeros((rows, max(top_k, 1)), dtype=np.float32)
    _check(lib().orc_moe_route(_p(lg), rows, experts, top_k, _p(sc), 1 if normalise else 0, _p(ids), _p(w)))
    return ids, w


def moe_combine(route_rows_f32, weights_f32, rows, top_k, n, bf16_steps=False):
    y = np.ascontiguousarray(route_rows_f32, dtype=np.float32).reshape(rows * top_k, n)
    w = np.ascontiguousarray(weights_f32, dtype=np.float32).reshape(-1)
    out = np.zeros((rows, n), dtype=np.float32)
    _check(lib().orc_moe_combine(_p(y), _p(w), rows, top_k, n, 1 if bf16_steps else 0, _p(out)))
    return out


def pack_greedy_best(score, token):
    fn = lib().orc_pack_greedy_best
    fn.restype = ctypes.c_uint64
    fn.argtypes = [ctypes.c_float, ctypes.c_int]
    return int(fn(score, token))


def unpack_greedy_best(packed, softcap=0.0, vocab_size=2 ** 31 - 1):
    fn = lib().orc_unpack_greedy_best
    fn.argtypes = [ctypes.c_uint64, ctypes.c_float, ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_float)]
    tok, sc = ctypes.c_int(0), ctypes.c_float(0)
    _check(fn(packed, softcap, vocab_size, ctypes.byref(tok), ctypes.byref(sc)))
    return tok.value, sc.value


def greedy_sample_suppress(logits_f32, suppress=None):
    lg = np.ascontiguousarray(logits_f32, dtype=np.float32).reshape(-1)
    sup = None if suppress is None else np.ascontiguousarray(suppress, dtype=np.int32)
    idx, val = ctypes.c_int(0), ctypes.c_float(0)
    _check(lib().orc_greedy_sample_suppress(_p(lg), lg.size, _p(sup), 0 if sup is None else sup.size, ctypes.byref(idx),
                                            ctypes.byref(val)))
    return idx.value, val.value


GGUF_F32, GGUF_Q4_0, GGUF_Q4_1, GGUF_Q8_0, GGUF_Q4_K, GGUF_Q5_K, GGUF_Q6_K = 0, 2, 3, 8, 12, 13, 14


def gguf_affine_layout(gguf_type, rows, cols):
    """(bits, group_size, packed_cols, groups, src_bytes) of the affine tensors a GGUF tensor repacks to."""
    bits, gs = ctypes.c_int(), ctypes.c_int()
    pc, groups, src = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_uint64()
    fn = lib().orc_gguf_affine_layout
    fn.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                   ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_uint64)]
    _check(fn(gguf_type, rows, cols, bits, gs, pc, groups, src))
    return bits.value, gs.value, pc.value, groups.value, src.value


def gguf_to_affine(gguf_type, rows, cols, data):
    """GGUF block bytes -> (packed uint32 [rows, packed_cols], scales uint16 [rows, groups], biases uint16)."""
    data = _u8(data)
    bits, gs, pc, groups, _ = gguf_affine_layout(gguf_type, rows, cols)
    w = np.zeros((rows, pc), np.uint32)
    s = np.zeros((rows, groups), np.uint16)
    b = np.zeros((rows, groups), np.uint16)
    fn = lib().orc_gguf_to_affine
    fn.argtypes = [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p,
                   ctypes.c_void_p, ctypes.c_void_p]
    _check(fn(gguf_type, rows, cols, _p(data), data.size, _p(w), _p(s), _p(b)))
    return w, s, b


def gguf_f32_to_bf16(v):
    fn = lib().orc_gguf_f32_to_bf16
    fn.argtypes, fn.restype = [ctypes.c_float], ctypes.c_uint16
    return int(fn(v))


def gguf_f16_to_f32(h):
    fn = lib().orc_gguf_f16_to_f32
    fn.argtypes, fn.restype = [ctypes.c_uint16], ctypes.c_float
    return float(fn(h))


def packed_topk_sample(packed_u64, temperature, top_p, softcap, draw):
    """rocm_packed_topk_sample over a descending packed list; returns the chosen packed value (0 = none)."""
    packed = np.ascontiguousarray(packed_u64, dtype=np.uint64)
    out = ctypes.c_uint64(0)
    fn = lib().orc_packed_topk_sample
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_double,
                   ctypes.POINTER(ctypes.c_uint64)]
    _check(fn(_p(packed), packed.size, temperature, top_p, softcap, draw, ctypes.byref(out)))
    return int(out.value)


def softcap_logits(logits_f32, softcap):
    out = np.array(logits_f32, dtype=np.float32)
    fn = lib().orc_softcap_logits
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_float]
    _check(fn(_p(out), out.size, softcap))
    return out


def host_sample(logits_f32, temperature, top_k, top_p, draw):
    """hipGemma4Q4HostSampleResult over (already softcapped) logits -> (token, score)."""
    logits = np.ascontiguousarray(logits_f32, dtype=np.float32)
    tok, sc = ctypes.c_int(0), ctypes.c_float(0)
    fn = lib().orc_host_sample
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_double,
                   ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_float)]
    _check(fn(_p(logits), logits.size, temperature, top_k, top_p, draw, ctypes.byref(tok), ctypes.byref(sc)))
    return tok.value, float(sc.value)


def max_threads():
    return int(lib().orc_max_threads())
