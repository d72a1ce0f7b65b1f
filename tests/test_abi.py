"""No-GPU checks of the C ABI: the library loads, exports every symbol the headers declare,
and its host-side logic (registry, row concat, geometry, argument rejection) behaves like the
Go declarations it mirrors.  Nothing here launches a kernel."""
import ctypes
import os
import re

import numpy as np
import pytest

import fixtures as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(aqh?_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(aqlib):
    import aq_mi355
    names = _declared("aq_mi355.h") + _declared("aq_mi355_host.h")
    assert len(names) >= 30
    for n in names:
        assert hasattr(aqlib, n), "missing export " + n
        assert n in aq_mi355.PROTOTYPES, "binding lacks a prototype for " + n
    assert b"gfx950" in aqlib.aq_version()


def test_null_context_is_rejected(aqlib):
    import aq_mi355
    assert aqlib.aq_qmv(None, None, None, None, None, None, 1, 64, 8, 64, 4, 0) == aq_mi355.AQ_ERR_ARG
    assert b"ctx" in aqlib.aq_last_error()
    assert aqlib.aq_gather_qmv(None, None, None, None, None, None, None, None, 1, 1, 64, 8, 1, 8, 0, 64, 4, 0) == aq_mi355.AQ_ERR_ARG
    assert aqlib.aq_sync(None) == aq_mi355.AQ_ERR_ARG


def test_variant_tables(aqlib):
    import aq_mi355
    q = aq_mi355.variant_names(aq_mi355.OP_QMV)
    m = aq_mi355.variant_names(aq_mi355.OP_QMM)
    assert len(q) == len(set(q)) and len(m) == len(set(m)) and q and m
    assert any(n.startswith("qmv_b4_m1_") and "_g1_" in n for n in q)
    assert any(n.startswith("qmmt_b8_") for n in m) and any(n.startswith("qmmh_b4_") for n in m)


def test_backend_quant_registry(aqlib):
    """go/model/quant_test.go:92-109: registration is keyed backend/kind and overwrites."""
    assert aqlib.aqh_backend_quant_registered(b"nowhere", b"affine") == 0
    aqlib.aqh_register_rocm_backend()
    aqlib.aqh_register_rocm_backend()
    assert aqlib.aqh_backend_quant_registered(b"rocm", b"affine") == 1
    assert aqlib.aqh_backend_quant_registered(b"rocm", b"gptq") == 0
    assert aqlib.aqh_backend_quant_bits(b"rocm", b"affine") == 0  # "the model config declares it"


def test_concat_quant_rows_is_a_byte_append(aqlib):
    """go/model/quant_weight.go:45-63"""
    wa, sa, ba = F.synthetic_affine(3, 128, 4, 64, seed=1)
    wb, sb, bb = F.synthetic_affine(5, 128, 4, 64, seed=2)
    u8 = lambda a: np.ascontiguousarray(a).view(np.uint8).reshape(-1)
    po, so, bo = np.zeros(8 * 64, np.uint8), np.zeros(8 * 4, np.uint8), np.zeros(8 * 4, np.uint8)
    od = ctypes.c_int(0)
    args = lambda in_b, bits_b, gs_b: (u8(wa).ctypes.data, u8(wa).size, u8(sa).ctypes.data, u8(sa).size, u8(ba).ctypes.data, 3,
                                       u8(wb).ctypes.data, u8(wb).size, u8(sb).ctypes.data, u8(sb).size, u8(bb).ctypes.data, 5,
                                       128, in_b, 4, bits_b, 64, gs_b, po.ctypes.data, so.ctypes.data, bo.ctypes.data, ctypes.byref(od))
    assert aqlib.aqh_concat_quant_rows(*args(128, 4, 64)) == 0
    assert od.value == 8
    assert np.array_equal(po, np.concatenate([u8(wa), u8(wb)]))
    assert np.array_equal(so, np.concatenate([u8(sa), u8(sb)]))
    assert np.array_equal(bo, np.concatenate([u8(ba), u8(bb)]))
    assert aqlib.aqh_concat_quant_rows(*args(256, 4, 64)) != 0   # InDim mismatch -> nil
    assert aqlib.aqh_concat_quant_rows(*args(128, 8, 64)) != 0   # Bits mismatch
    assert aqlib.aqh_concat_quant_rows(*args(128, 4, 32)) != 0   # GroupSize mismatch


@pytest.mark.parametrize("in_dim,scales_last,packed_last,want", [(4096, 64, 512, (64, 4)), (4096, 128, 1024, (32, 8)),
                                                                 (3840, 60, 720, (64, 6)), (256, 2, 16, (128, 2)),
                                                                 (0, 4, 4, (0, 0)), (128, -1, -1, (0, 0))])
def test_affine_geometry(aqlib, in_dim, scales_last, packed_last, want):
    """go/model/linear.go:91-110"""
    gs, bits = ctypes.c_int(-1), ctypes.c_int(-1)
    aqlib.aqh_affine_geometry(in_dim, scales_last, packed_last, ctypes.byref(gs), ctypes.byref(bits))
    assert (gs.value, bits.value) == want


def test_pack_and_unpack_best_match_the_oracle(aqlib, orc):
    """aq_pack_best / aq_unpack_best are host code (hipPackGreedyBest / hipUnpackGreedyBest,
    go/engine/hip/hip_projection_launch.go:2393-2416)."""
    import aq_mi355
    for score, token in [(1.0, 2), (-3.5, 0), (0.0, 262143), (-0.0, 1), (1e-40, 5), (3.4e38, 77)]:
        p = aq_mi355.pack_best(score, token)
        assert p == orc.pack_greedy_best(score, token)
        assert aq_mi355.unpack_best(p, 0.0, 262144) == orc.unpack_greedy_best(p, 0.0, 262144)
    p = aq_mi355.pack_best(45.0, 9)
    assert aq_mi355.unpack_best(p, 30.0, 100) == orc.unpack_greedy_best(p, 30.0, 100)
    for args, code in [((0, 0.0, 10), aq_mi355.AQ_ERR_INDEX), ((aq_mi355.pack_best(1.0, 10), 0.0, 10), aq_mi355.AQ_ERR_INDEX),
                       ((aq_mi355.pack_best(1.0, 1), -1.0, 10), aq_mi355.AQ_ERR_ARG),
                       ((aq_mi355.pack_best(1.0, 1), float("inf"), 10), aq_mi355.AQ_ERR_ARG),
                       ((aq_mi355.pack_best(1.0, 1), 0.0, 0), aq_mi355.AQ_ERR_SHAPE)]:
        with pytest.raises(aq_mi355.AqError) as e:
            aq_mi355.unpack_best(*args)
        assert e.value.code == code


def test_tiled_bytes_needs_no_device(aqlib):
    """aq_tiled_bytes is pure arithmetic: it agrees with the numpy statement of the tile-major layout."""
    import aq_mi355
    for n, k in ((14336, 4096), (17, 4096), (33, 2816), (64, 3200), (5, 128), (100, 16384)):
        w, s, b = F.synthetic_affine(min(n, 40), k, 4, 64, seed=n + k)
        sets_ref = (min(n, 40) + 15) // 16
        per_set = F.tile_major(w, s, b, min(n, 40), k).size // sets_ref
        assert aq_mi355.tiled_bytes(n, k) == (n + 15) // 16 * per_set
    assert aq_mi355.tiled_bytes(14336, 4096) == 14336 * 4096 // 2 + 2 * 14336 * 64 * 2
    for n, k, gs, bits in ((16, 4096, 64, 8), (16, 4096, 32, 4), (16, 4096, 128, 4), (16, 192, 64, 4), (0, 4096, 64, 4)):
        assert aq_mi355.tiled_bytes(n, k, gs, bits) == -1
    assert aqlib.aq_tile_weights(None, None, None, None, 16, 4096, 64, 4, None) == aq_mi355.AQ_ERR_ARG
    assert aqlib.aq_untile_weights(None, None, 16, 4096, 64, 4, None, None, None) == aq_mi355.AQ_ERR_ARG
