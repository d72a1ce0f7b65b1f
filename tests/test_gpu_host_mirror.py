"""The plug-in surface a Go backend registers against, driven end to end on the device:
model.BackendQuant("rocm","affine").MatVec (QuantParity) and attn.ProjQuantMatMulInto."""
import ctypes

import numpy as np
import pytest

import fixtures as F
from gpu_util import say

pytestmark = pytest.mark.gpu


def _matvec(lib, x, p, s, b, out_dim, in_dim, gs, bits):
    x, p, s, b = (np.ascontiguousarray(a).view(np.uint8).reshape(-1) for a in (x, p, s, b))
    out = np.zeros(max(out_dim, 1) * 2, dtype=np.uint8)
    n = ctypes.c_size_t(0)
    rc = lib.aqh_backend_quant_matvec(b"rocm", b"affine", x.ctypes.data, x.size, p.ctypes.data, p.size, s.ctypes.data, s.size,
                                      b.ctypes.data, b.size, out_dim, in_dim, gs, bits, out.ctypes.data, out.size, ctypes.byref(n))
    return rc, out[:n.value]


def test_quant_parity(aqlib, ctx, orc):
    """enginetest.QuantParity (go/engine/enginetest/quant_parity.go:77-108): byte-identical or <= 0.05 per element."""
    say("QuantParity rocm/affine")
    aqlib.aqh_register_rocm_backend()
    assert aqlib.aqh_backend_quant_registered(b"rocm", b"affine") == 1
    assert aqlib.aqh_backend_quant_bits(b"rocm", b"affine") == 0
    fx = F.quant_affine_fixture()
    rc, got = _matvec(aqlib, fx["x"], fx["packed"], fx["scales"], fx["biases"], 8, 128, 64, 4)
    assert rc == 0, aqlib.aqh_last_error()
    want = orc.reference_affine_matvec(fx["x"], fx["packed"], fx["scales"], fx["biases"], 8, 128, 64, 4)
    assert got.size == want.size
    gv, wv = F.bf16_bits_to_f32(got.view(np.uint16)), F.bf16_bits_to_f32(want.view(np.uint16))
    assert np.array_equal(got, want) or np.abs(gv - wv).max() <= 0.05
    # our own bar is tighter: within one bf16 ulp
    from gpu_util import check_bf16_store
    check_bf16_store(got.view(np.uint16), wv.astype(np.float64), "QuantParity")


def test_matvec_contract_errors_and_zero_size(aqlib, ctx):
    """Malformed sizes give an error, never a crash; zero-sized dims give an empty result
    (go/engine/enginetest/quant_reference_test.go:42-74)."""
    say("MatVec contract")
    aqlib.aqh_register_rocm_backend()
    fx = F.quant_affine_fixture()
    x, p, s, b = fx["x"].view(np.uint8), fx["packed"].view(np.uint8).reshape(-1), fx["scales"].view(np.uint8).reshape(-1), fx["biases"].view(np.uint8).reshape(-1)
    assert _matvec(aqlib, x[:-1], p, s, b, 8, 128, 64, 4)[0] != 0
    assert _matvec(aqlib, x, p[:-1], s, b, 8, 128, 64, 4)[0] != 0
    assert _matvec(aqlib, x, p, s, b, 8, 128, 3, 4)[0] != 0
    assert _matvec(aqlib, x, p, s, b, 8, 128, 64, 0)[0] != 0
    assert _matvec(aqlib, x, p, s, b, 8, 128, 64, 9)[0] != 0
    e = np.zeros(0, dtype=np.uint8)
    rc, out = _matvec(aqlib, e, e, e, e, 0, 0, 64, 4)
    assert rc == 0 and out.size == 0


@pytest.mark.parametrize("name,M,K,N,bits,gs", [("decode-qmv-gs64-b4", 1, 512, 40, 4, 64), ("decode-qmv-gs128-b2", 1, 256, 24, 2, 128),
                                                ("prefill-qmm_t-alN-true", 3, 512, 64, 4, 64), ("prefill-qmm_t-alN-false", 5, 256, 40, 2, 128),
                                                ("prefill-qmm_t-b8-smallN", 2, 128, 8, 8, 64)])
def test_proj_quant_matmul_into(aqlib, ctx, orc, name, M, K, N, bits, gs):
    """TestMatMulQuantF32NTInto_ParityDecodeAndPrefill (go/engine/metal/quant_seam_backend_test.go:46-87):
    QuantizeTensor(cbqSynthW) -> device vs DequantizeTensor + f64 matNT at 1e-2*(1+|want|)."""
    say("ProjQuantMatMulInto", name)
    aqlib.aqh_register_rocm_backend()
    w = F.cbq_synth_w(N, K)
    p, s, b = orc.quantize(w, N, K, bits, gs)
    deq = orc.dequantize(p, s, b, N, K, bits, gs).astype(np.float64)
    x = np.array([np.float32((i % 9) - 4) * np.float32(0.05) for i in range(M * K)], dtype=np.float32)
    want = x.astype(np.float64).reshape(M, K) @ deq.T
    out = np.zeros(M * N, dtype=np.float32)
    rc = aqlib.aqh_proj_quant_matmul_into(out.ctypes.data, out.size, x.ctypes.data, x.size, p.ctypes.data, p.size, s.ctypes.data, s.size,
                                          b.ctypes.data, b.size, M, K, N, gs, bits)
    assert rc == 0, aqlib.aqh_last_error()
    assert (np.abs(out.reshape(M, N) - want) <= 1e-2 * (1 + np.abs(want))).all()
    # the seam equals matNTQuantHost on the bf16-rounded activations to well inside that bound
    xb = F.bf16_bits_to_f32(F.f32_to_bf16_bits(x))
    host = orc.matnt_quant_host(xb, p, s, b, M, K, N, gs, bits)
    assert np.abs(out.reshape(M, N) - host).max() <= 4e-3 * max(1.0, np.abs(host).max())


def test_proj_quant_matmul_into_errors(aqlib, ctx, orc):
    """go/engine/metal/quant_seam_backend_test.go:92-102"""
    aqlib.aqh_register_rocm_backend()
    p, s, b = orc.quantize(F.cbq_synth_w(16, 128), 16, 128, 4, 64)
    out = np.zeros(16, dtype=np.float32)
    x100, x128 = np.zeros(100, dtype=np.float32), np.zeros(128, dtype=np.float32)
    call = lambda x, gs: aqlib.aqh_proj_quant_matmul_into(out.ctypes.data, out.size, x.ctypes.data, x.size, p.ctypes.data, p.size,
                                                          s.ctypes.data, s.size, b.ctypes.data, b.size, 1, 128, 16, gs, 4)
    assert call(x100, 64) != 0
    assert call(x128, 60) != 0
    assert call(x128, 64) == 0
