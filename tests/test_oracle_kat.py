"""Pins the CPU oracle (oracle/aq_oracle.c) against the known-answer vectors and fixtures the
reference's own tests hold, and against what the mathematics fixes.  No GPU."""
import math

import numpy as np
import pytest

import fixtures as F


# ---- bf16 codecs ---------------------------------------------------------------------------

def test_bf16_round_trip_list(orc):
    # go/engine/enginetest/quant_reference_test.go:98-110
    for v in [0, 1, -1, 12.5, 0.25, -3.75, 100, -0.03125]:
        assert orc.bf16_to_f32(orc.f32_to_bf16(v)) == v


def test_bf16_constants(orc):
    # go/engine/hip/hip_projection_reference_test.go:201-210
    assert orc.bf16_to_f32(0x3F80) == 1.0
    assert orc.bf16_to_f32(0xC000) == -2.0
    assert orc.bf16_to_f32(0x7F80) == math.inf
    assert math.isnan(orc.bf16_to_f32(0x7FC0))
    assert orc.f32_to_bf16(12.5) == 0x4148


def test_bf16_widen_exhaustive(orc):
    for h in range(0, 65536, 1):
        want = np.array([h], dtype=np.uint32) << 16
        got = np.array([orc.bf16_to_f32(h)], dtype=np.float32).view(np.uint32)
        if not (math.isnan(orc.bf16_to_f32(h))):
            assert got[0] == want[0]


def test_bf16_rne_ties_and_nan(orc):
    # 1 + 2^-8 is exactly half way between bf16 1.0 (even) and 1.0078125 (odd): stays 1.0
    assert orc.f32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80
    # 1.0078125 + 2^-8 is half way between odd 0x3F81 and even 0x3F82: goes up
    assert orc.f32_to_bf16(1.0078125 + 2.0 ** -8) == 0x3F82
    assert orc.f32_to_bf16(1.0 + 2.0 ** -8 + 2.0 ** -20) == 0x3F81
    assert orc.f32_to_bf16(-(1.0 + 2.0 ** -8)) == 0xBF80
    assert orc.f32_to_bf16(3.4e38) == 0x7F80  # rounds up into +inf
    h = orc.f32_to_bf16(float("nan"))
    assert (h & 0x7F80) == 0x7F80 and (h & 0x007F) != 0


def test_bf16_rne_matches_torch(orc):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(7)
    vals = np.concatenate([rng.normal(0, 1, 4000), rng.normal(0, 1e-3, 2000), rng.normal(0, 1e4, 2000)]).astype(np.float32)
    want = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([orc.f32_to_bf16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(F.f32_to_bf16_bits(vals), want)  # the numpy helper the other tests lean on


# ---- code packing ---------------------------------------------------------------------------

def test_set_extract_packing_order(orc):
    # codes [3,5] at 4 bit pack to 0x53 (go/engine/enginetest/quant_reference_test.go:13-21)
    row = np.zeros(1, dtype=np.uint8)
    orc.set_code(row, 0, 4, 3)
    orc.set_code(row, 4, 4, 5)
    assert row[0] == 0x53
    # 0x76543210 holds codes 0..7 in column order (go/engine/hip/hip_projection_reference_test.go:71-85)
    word = np.array([0x76543210], dtype=np.uint32)
    assert [orc.extract_code(word, 4 * c, 4) for c in range(8)] == list(range(8))


@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8])
def test_set_extract_round_trip_all_widths(orc, bits):
    rng = np.random.default_rng(bits)
    k = 64
    codes = rng.integers(0, 1 << bits, size=k)
    row = np.zeros(k * bits // 8, dtype=np.uint8)
    for c, v in enumerate(codes):
        orc.set_code(row, c * bits, bits, int(v))
    assert [orc.extract_code(row, c * bits, bits) for c in range(k)] == [int(v) for v in codes]
    # the byte-walking packer and the word packer used by the fixtures describe the same layout
    assert np.array_equal(F.pack_codes(codes.reshape(1, -1), bits).view(np.uint8).reshape(-1), row)


def test_quant_affine_fixture_round_trips(orc):
    # go/engine/enginetest/quant_reference_test.go:80-92
    fx = F.quant_affine_fixture()
    rows = fx["packed"].view(np.uint8).reshape(fx["out_dim"], -1)
    for r in range(fx["out_dim"]):
        for c in range(fx["in_dim"]):
            assert orc.extract_code(rows[r], c * 4, 4) == (c * 5 + r * 3 + 1) % 16


# ---- ReferenceAffineMatVec -------------------------------------------------------------------

def test_reference_affine_matvec_good(orc):
    # 1x2, scale 2, bias 1, codes [3,5] -> w [7,11]; x [1, 0.5] -> 12.5 exactly (quant_reference_test.go:13-38)
    packed = np.array([0x53], dtype=np.uint8)
    s = np.array([orc.f32_to_bf16(2.0)], dtype=np.uint16)
    b = np.array([orc.f32_to_bf16(1.0)], dtype=np.uint16)
    x = np.array([orc.f32_to_bf16(1.0), orc.f32_to_bf16(0.5)], dtype=np.uint16)
    out = orc.reference_affine_matvec(x, packed, s, b, 1, 2, 2, 4)
    assert out.view(np.uint16)[0] == orc.f32_to_bf16(12.5)


def test_reference_affine_matvec_bad(orc):
    # quant_reference_test.go:42-61
    fx = F.quant_affine_fixture()
    x, p, s, b = fx["x"].view(np.uint8), fx["packed"].view(np.uint8), fx["scales"].view(np.uint8), fx["biases"].view(np.uint8)
    od, idim, gs, bits = fx["out_dim"], fx["in_dim"], fx["group_size"], fx["bits"]
    with pytest.raises(orc.OracleError):
        orc.reference_affine_matvec(x[:-1], p, s, b, od, idim, gs, bits)
    with pytest.raises(orc.OracleError):
        orc.reference_affine_matvec(x, p.reshape(-1)[:-1], s, b, od, idim, gs, bits)
    with pytest.raises(orc.OracleError):
        orc.reference_affine_matvec(x, p, s, b, od, idim, 3, bits)
    with pytest.raises(orc.OracleError):
        orc.reference_affine_matvec(x, p, s, b, od, idim, gs, 0)
    with pytest.raises(orc.OracleError):
        orc.reference_affine_matvec(x, p, s, b, od, idim, gs, 9)


def test_reference_affine_matvec_ugly_zero_sized(orc):
    # quant_reference_test.go:66-74
    e = np.zeros(0, dtype=np.uint8)
    assert orc.reference_affine_matvec(e, e, e, e, 0, 0, 64, 4).size == 0


# ---- hipReferenceMLXAffineProjection ---------------------------------------------------------

def test_hip_reference_q4_known_answer(orc):
    # go/engine/hip/hip_projection_reference_test.go:71-85 -> [28, 38]
    out = orc.hip_reference_projection(np.ones(8), [0x76543210, 0xFEDCBA98], [0x3F80, 0x3F00], [0x0000, 0xBF80], 2, 8, 8, 4)
    assert out.tolist() == [28.0, 38.0]


def test_hip_reference_q6_q8_known_answers(orc):
    # go/engine/hip/hip_projection_reference_test.go:87-106 -> [120, 136] and [10, 26]
    v6 = np.array([list(range(16)), [16, 15, 14, 13, 12, 11, 10, 9, 8, 7, 6, 5, 4, 3, 2, 1]])
    out6 = orc.hip_reference_projection(np.ones(16), F.pack_codes(v6, 6), [0x3F80, 0x3F80], [0, 0], 2, 16, 16, 6)
    assert out6.tolist() == [120.0, 136.0]
    v8 = np.array([[1, 2, 3, 4], [5, 6, 7, 8]])
    out8 = orc.hip_reference_projection(np.ones(4), F.pack_codes(v8, 8), [0x3F80, 0x3F80], [0, 0], 2, 4, 4, 8)
    assert out8.tolist() == [10.0, 26.0]


def test_hip_reference_batch_known_answer(orc):
    # go/engine/hip/hip_kernels_test.go:612-654 -> [28, 38, 56, 76], laid out [token][row]
    x = np.concatenate([np.ones(8), 2 * np.ones(8)])
    out = orc.hip_reference_projection_batch(x, 2, [0x76543210, 0xFEDCBA98], [0x3F80, 0x3F00], [0x0000, 0xBF80], 2, 8, 8, 4)
    assert out.reshape(-1).tolist() == [28.0, 38.0, 56.0, 76.0]


def test_hip_reference_bad_shapes(orc):
    # go/engine/hip/hip_projection_reference_test.go:139-145: cols*bits not a word multiple; group not dividing
    with pytest.raises(orc.OracleError):
        orc.hip_reference_projection([1.0], [0], [0x3F80], [0], 1, 7, 7, 4)
    with pytest.raises(orc.OracleError):
        orc.hip_reference_projection(np.ones(8), [0], [0x3F80], [0], 1, 8, 3, 4)
    with pytest.raises(orc.OracleError):
        orc.hip_reference_projection(np.ones(8), [0], [0x3F80], [0], 1, 8, 8, 5)


# ---- DequantizeTensor / QuantizeTensor -------------------------------------------------------

def test_example_quantize_tensor(orc):
    # go/model/quant/mlxaffine/mlxaffine_example_test.go:14-35
    w = np.array([np.float32(0.01) * np.float32(i - 32) for i in range(64)], dtype=np.float32)
    p, s, b = orc.quantize(w, 1, 64, 4, 64)
    assert (p.size, s.size, b.size) == (32, 2, 2)
    got = orc.dequantize(p, s, b, 1, 64, 4, 64)
    assert "%.3f" % w[0] == "-0.320" and "%.3f" % got[0, 0] == "-0.320"


@pytest.mark.parametrize("bits,gs,out_dim,in_dim", [(4, 64, 8, 3840), (4, 32, 4, 256), (8, 64, 6, 512), (8, 32, 3, 128),
                                                     (2, 64, 5, 640), (4, 64, 3, 64)])
def test_quantize_round_trip_within_group_bound(orc, bits, gs, out_dim, in_dim):
    # go/model/quant/mlxaffine/mlxaffine_test.go:32-78
    w = F.synth_weight(out_dim, in_dim)
    p, s, b = orc.quantize(w, out_dim, in_dim, bits, gs)
    got = orc.dequantize(p, s, b, out_dim, in_dim, bits, gs)
    assert np.isfinite(got).all()
    wg = w.reshape(out_dim, in_dim // gs, gs)
    step = (wg.max(axis=2) - wg.min(axis=2)) / np.float32((1 << bits) - 1)
    bound = 1.5 * step + 0.02 * np.abs(wg).max(axis=2) + 1e-6
    err = np.abs(got.reshape(wg.shape) - wg)
    assert (err <= bound[..., None]).all()


def test_quantize_codes_are_a_fixed_point(orc):
    # go/model/quant/mlxaffine/mlxaffine_test.go:87-112
    w = F.synth_weight(6, 512)
    p1, s1, b1 = orc.quantize(w, 6, 512, 4, 64)
    d1 = orc.dequantize(p1, s1, b1, 6, 512, 4, 64)
    p2, s2, b2 = orc.quantize(d1, 6, 512, 4, 64)
    assert np.array_equal(p1, p2)
    d2 = orc.dequantize(p2, s2, b2, 6, 512, 4, 64)
    assert np.abs(d2 - d1).max() <= 5e-3


def test_quantize_constant_group(orc):
    # go/model/quant/mlxaffine/mlxaffine_test.go:117-139
    w = np.full(2 * 64, 0.25, dtype=np.float32)
    p, s, b = orc.quantize(w, 2, 64, 4, 64)
    got = orc.dequantize(p, s, b, 2, 64, 4, 64)
    assert np.isfinite(got).all() and np.abs(got - 0.25).max() <= 0.01


@pytest.mark.parametrize("out_dim,in_dim,gs", [(4, 128, 128), (8, 256, 128), (3, 64, 64), (5, 96, 32)])
def test_repack_b1_to_b2_exact(orc, out_dim, in_dim, gs):
    # go/model/quant/mlxaffine/repack_test.go:26-65: exact float32 equality
    w = F.synth_weight(out_dim, in_dim)
    p, s, b = orc.quantize(w, out_dim, in_dim, 1, gs)
    ref = orc.dequantize(p, s, b, out_dim, in_dim, 1, gs)
    p2 = orc.repack_b1_to_b2(p, out_dim, in_dim)
    assert p2.size == out_dim * (in_dim // 16) * 4
    got = orc.dequantize(p2, s, b, out_dim, in_dim, 2, gs)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_dequantize_brute_force_all_codes(orc, bits):
    """Every code value against sampled bf16 (scale, bias) pairs: the C loop must equal a float32
    multiply-then-add done one scalar at a time in numpy, and also the fused form (the product is
    exact, so both must agree)."""
    rng = np.random.default_rng(100 + bits)
    ncodes = 1 << bits
    per = 32 // bits
    k = max(per, ncodes)  # one group holding every code at least once
    k = (k + per - 1) // per * per
    for _ in range(200):
        sb = rng.integers(0, 65536, size=2).astype(np.uint16)
        sf, bf = F.bf16_bits_to_f32(sb)
        if not (np.isfinite(sf) and np.isfinite(bf)):
            continue
        codes = (np.arange(k) % ncodes).astype(np.uint32).reshape(1, k)
        got = orc.dequantize(F.pack_codes_fast(codes, bits), sb[:1], sb[1:], 1, k, bits, k)
        with np.errstate(all="ignore"):
            want = (np.float32(sf) * codes.astype(np.float32)).astype(np.float32) + np.float32(bf)
            fused = (np.float64(sf) * codes.astype(np.float64) + np.float64(bf)).astype(np.float32)
        assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))
        ok = np.isfinite(fused)
        assert np.array_equal(got[ok].view(np.uint32), fused[ok].view(np.uint32))


def test_dequantize_matches_numpy_formula_and_rejects_bad_sizes(orc):
    """Same tensor through the broadcast-shift numpy formula of tools/mlxaffine_dequant.py:52-69."""
    words, s, b = F.synthetic_affine(24, 512, 4, 64, seed=11)
    got = orc.dequantize(words, s, b, 24, 512, 4, 64)
    assert np.array_equal(got.view(np.uint32), F.numpy_dequant(words, s, b, 4, 64, 512).view(np.uint32))
    words8, s8, b8 = F.synthetic_affine(7, 256, 8, 32, seed=12)
    got8 = orc.dequantize(words8, s8, b8, 7, 256, 8, 32)
    assert np.array_equal(got8.view(np.uint32), F.numpy_dequant(words8, s8, b8, 8, 32, 256).view(np.uint32))
    with pytest.raises(orc.OracleError):
        orc.dequantize(words.reshape(-1)[:-1], s, b, 24, 512, 4, 64)
    with pytest.raises(orc.OracleError):
        orc.dequantize(words, s.reshape(-1)[:-1], b, 24, 512, 4, 64)
    with pytest.raises(orc.OracleError):
        orc.dequantize(words, s, b, 24, 512, 3, 64)
    with pytest.raises(orc.OracleError):
        orc.dequantize(words, s, b, 24, 512, 4, 60)


# ---- matNTQuantHost and cross-agreement ------------------------------------------------------

def test_matnt_quant_host_is_sequential_f64(orc):
    """Tiny case recomputed with a python float (= float64) ascending-k loop over numpy's fp32 dequant."""
    words, s, b = F.synthetic_affine(5, 128, 4, 64, seed=21)
    x = F.bf16_bits_to_f32(F.synthetic_x(3, 128, seed=22)).reshape(3, 128)
    got = orc.matnt_quant_host(x, words, s, b, 3, 128, 5, 64, 4)
    w = F.numpy_dequant(words, s, b, 4, 64, 128)
    for m in range(3):
        for n in range(5):
            acc = 0.0
            for k in range(128):
                acc += float(x[m, k]) * float(w[n, k])
            assert got[m, n] == np.float32(acc)


def test_matnt_quant_host_threads_bit_identical(orc):
    words, s, b = F.synthetic_affine(64, 256, 4, 64, seed=23)
    x = F.bf16_bits_to_f32(F.synthetic_x(4, 256, seed=24)).reshape(4, 256)
    a = orc.matnt_quant_host(x, words, s, b, 4, 256, 64, 64, 4, threads=1)
    c = orc.matnt_quant_host(x, words, s, b, 4, 256, 64, 64, 4, threads=4)
    assert np.array_equal(a.view(np.uint32), c.view(np.uint32))


def test_all_ones_closed_form(orc):
    """x = 1: y[n] = sum_g (scale_g * sum(codes in g) + group * bias_g), exact in float64.
    A dropped bias term, a wrong group index or a transposed scale table fails here."""
    rng = np.random.default_rng(5)
    n, k, gs = 6, 256, 64
    codes = rng.integers(0, 16, size=(n, k)).astype(np.uint32)
    s = F.f32_to_bf16_bits(rng.uniform(0.01, 0.2, size=(n, k // gs)).astype(np.float32))
    b = F.f32_to_bf16_bits(rng.uniform(-1, 1, size=(n, k // gs)).astype(np.float32))
    sf, bf = F.bf16_bits_to_f32(s).astype(np.float64), F.bf16_bits_to_f32(b).astype(np.float64)
    want = (sf * codes.reshape(n, k // gs, gs).sum(axis=2) + gs * bf).sum(axis=1)
    ones = np.full(k, 0x3F80, dtype=np.uint16)
    words = F.pack_codes_fast(codes, 4)
    got_bf16 = F.bf16_bits_to_f32(orc.reference_affine_matvec(ones, words, s, b, n, k, gs, 4).view(np.uint16))
    assert np.array_equal(got_bf16, F.bf16_bits_to_f32(F.f32_to_bf16_bits(want.astype(np.float32))))
    got_host = orc.matnt_quant_host(np.ones(k, dtype=np.float32), words, s, b, 1, k, n, gs, 4)
    assert np.allclose(got_host.reshape(-1), want, rtol=1e-6, atol=1e-6)
    got_hip = orc.hip_reference_projection(np.ones(k), words, s, b, n, k, gs, 4)
    assert np.allclose(got_hip, want, rtol=1e-5, atol=1e-5)


def test_references_agree_on_the_parity_fixture(orc):
    """a3 (fp32 w, f64 acc), a4 (f64 w, f64 acc, bf16 out) and a5 (fp32 acc) on quantAffineFixture,
    against an independent numpy float64 matmul."""
    fx = F.quant_affine_fixture()
    xf = F.bf16_bits_to_f32(fx["x"])
    want = F.reference_f64(fx["x"], fx["packed"], fx["scales"], fx["biases"], 4, 64, 128).reshape(-1)
    a4 = F.bf16_bits_to_f32(orc.reference_affine_matvec(fx["x"], fx["packed"], fx["scales"], fx["biases"], 8, 128, 64, 4).view(np.uint16))
    assert np.array_equal(a4, F.bf16_bits_to_f32(F.f32_to_bf16_bits(want.astype(np.float32))))
    a3 = orc.matnt_quant_host(xf, fx["packed"], fx["scales"], fx["biases"], 1, 128, 8, 64, 4).reshape(-1)
    assert np.allclose(a3, want, rtol=0, atol=1e-5)
    a5 = orc.hip_reference_projection(xf, fx["packed"], fx["scales"], fx["biases"], 8, 128, 64, 4)
    assert np.allclose(a5, want, rtol=0, atol=1e-4)


@pytest.mark.parametrize("fixture", ["hw_fixture_q8_cols256", "hw_fixture_q8_cols3072"])
def test_hardware_fixtures_against_numpy(orc, fixture):
    fx = getattr(F, fixture)()
    want = F.numpy_dequant(fx["packed"], fx["scales"], fx["biases"], 8, fx["group_size"], fx["cols"]).astype(np.float64) @ fx["x"].astype(np.float64)
    got = orc.hip_reference_projection(fx["x"], fx["packed"], fx["scales"], fx["biases"], fx["rows"], fx["cols"], fx["group_size"], 8)
    assert np.abs(got - want).max() <= 1e-3


# ---- gather ---------------------------------------------------------------------------------

@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
@pytest.mark.parametrize("name,out_dim,in_dim,gs,expert_rows,row_base,batched", [
    ("fast shared-x", 32, 512, 64, 32, 0, False), ("fast batched-x", 32, 512, 64, 32, 0, True),
    ("plain shared-x", 24, 256, 32, 24, 0, False), ("fast gate_up rowBase", 32, 512, 64, 64, 32, False)])
def test_gather_equals_sliced_matvec(orc, bits, name, out_dim, in_dim, gs, expert_rows, row_base, batched):
    """Route z == the plain matvec on expert rhs[z]'s row slice with x row lhs[z]
    (the cases of go/engine/metal/qmv_gather_test.go:87-129; invariant of moe_quant_test.go:1143-1185)."""
    if in_dim * bits % 32:
        pytest.skip("packed-row alignment")
    E, routes = 4, 3
    fx = F.gather_fixture(out_dim, in_dim, gs, bits, E, expert_rows, batched, routes)
    _, got = orc.gather_qmv(fx["x"], fx["x_rows"], fx["packed"], fx["scales"], fx["biases"], fx["lhs"], fx["rhs"], routes, E,
                            expert_rows, row_base, out_dim, in_dim, gs, bits)
    wpr, gpr = in_dim * bits // 32, in_dim // gs
    W = fx["packed"].reshape(E, expert_rows, wpr)
    S = fx["scales"].reshape(E, expert_rows, gpr)
    B = fx["biases"].reshape(E, expert_rows, gpr)
    X = fx["x"].reshape(fx["x_rows"], in_dim)
    for z in range(routes):
        e = fx["rhs"][z]
        xr = X[fx["lhs"][z]] if batched else X[0]
        want = orc.reference_affine_matvec(xr, W[e, row_base:row_base + out_dim], S[e, row_base:row_base + out_dim],
                                           B[e, row_base:row_base + out_dim], out_dim, in_dim, gs, bits)
        assert np.array_equal(got[z], want.view(np.uint16))


def test_gather_rejects_bad_indices(orc):
    fx = F.gather_fixture(8, 64, 64, 4, 4, 8, False, 3)
    bad = fx["rhs"].copy()
    bad[1] = 4
    with pytest.raises(orc.OracleError):
        orc.gather_qmv(fx["x"], 1, fx["packed"], fx["scales"], fx["biases"], None, bad, 3, 4, 8, 0, 8, 64, 64, 4)
    bad[1] = -1
    with pytest.raises(orc.OracleError):
        orc.gather_qmv(fx["x"], 1, fx["packed"], fx["scales"], fx["biases"], None, bad, 3, 4, 8, 0, 8, 64, 64, 4)


# ---- activations of the fused MLP kernels ---------------------------------------------------------

def _torch_act(torch, act, v64):
    f = torch.nn.functional
    return f.gelu(v64, approximate="tanh") if act == 1 else f.silu(v64)


@pytest.mark.parametrize("act", [1, 2])
def test_act_multiply_matches_library_routine(orc, act):
    """expectedGELUTanhMultiply (go/engine/hip/hip_kernels_test.go:8127-8137) reduces to the library's
    tanh-approximated GELU (SiLU: gated_delta.go:228) taken in float64, rounded to float32, times up."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(11 + act)
    g = np.concatenate([rng.normal(0, 2, 6000), rng.normal(0, 0.01, 1000), np.linspace(-12, 12, 1001)]).astype(np.float32)
    u = rng.normal(0, 1.5, g.size).astype(np.float32)
    got = orc.act_multiply(act, g, u)
    a32 = _torch_act(torch, act, torch.from_numpy(g).double()).float().numpy()
    want = a32 * u
    # libm and the library may round tanh/exp differently in the last float64 place: at most one fp32 ulp,
    # except deep in the negative tail, where 1 + tanh cancels and only the absolute size (< 1e-12) matters
    ok = (np.abs(got - want) <= np.spacing(np.abs(want).astype(np.float32))) | (np.abs(got - want) <= 1e-12 * np.abs(g * u))
    assert ok.all()
    assert np.mean(got == want) > 0.99


@pytest.mark.parametrize("act", [1, 2])
def test_act_closed_forms(orc, act):
    one = np.ones(1, np.float32)
    f = lambda v: float(orc.act_multiply(act, np.array([v], np.float32), one)[0])
    assert f(0.0) == 0.0
    # both activations are x * s(x) with s(x) + s(-x) = 1, so f(x) - f(-x) = x
    for v in [0.125, 0.5, 1.0, 2.5, 7.0]:
        assert abs((f(v) - f(-v)) - v) <= 2e-7 * max(1.0, v)
    assert abs(f(30.0) - 30.0) < 1e-5 and abs(f(-30.0)) < 1e-5
    if act == 1:
        # 0.5 * (1 + tanh(sqrt(2/pi) * 1.044715))
        assert abs(f(1.0) - 0.5 * (1 + math.tanh(0.7978845608028654 * 1.044715))) < 1e-7
    else:
        assert abs(f(1.0) - 1 / (1 + math.exp(-1))) < 1e-7
    # the multiplier is applied after the activation, in float32
    g = np.array([1.5, -0.75], np.float32)
    assert np.array_equal(orc.act_multiply(act, g, np.array([2.0, -4.0], np.float32)),
                          orc.act_multiply(act, g, np.ones(2, np.float32)) * np.array([2.0, -4.0], np.float32))


@pytest.mark.parametrize("act", [1, 2])
def test_act_gate_mul_bf16_matches_library_routine(orc, act):
    """hostGeluMul (go/engine/metal/ffn_megakernel_test.go:17-31): bf16 in, fp32 inside, one bf16 rounding."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(21 + act)
    g = F.f32_to_bf16_bits(rng.normal(0, 2, 20000).astype(np.float32))
    u = F.f32_to_bf16_bits(rng.normal(0, 1.5, 20000).astype(np.float32))
    got = orc.act_gate_mul_bf16(act, g, u)
    tg = torch.from_numpy(F.bf16_bits_to_f32(g)).double()
    tu = torch.from_numpy(F.bf16_bits_to_f32(u)).double()
    exact = (_torch_act(torch, act, tg) * tu).numpy()
    want = F.f32_to_bf16_bits(exact.astype(np.float32))
    key = lambda b: np.where(b.astype(np.int32) & 0x8000, -(b.astype(np.int32) & 0x7FFF), b.astype(np.int32) & 0x7FFF)
    d = np.abs(key(got) - key(want))
    absd = np.abs(F.bf16_bits_to_f32(got).astype(np.float64) - exact)
    # fp32 internals vs an exact product: a rounding boundary may flip; in the negative GELU tail the fp32
    # form 1 + tanh cancels, which is the function the reference defines, so only absolute size counts there
    assert ((d <= 1) | (absd <= 1e-6)).all()
    assert np.mean(d == 0) > 0.98
    # exact special values
    z = orc.act_gate_mul_bf16(act, np.array([0x0000, 0x3F80], np.uint16), np.array([0x3F80, 0x0000], np.uint16))
    assert z[0] == 0 and z[1] == 0


@pytest.mark.parametrize("gs", [32, 64])
def test_gelu_hardware_fixture_oracle_vs_independent_float64(orc, gs):
    """The fused gate|up expectation of go/engine/hip/hip_hardware_test.go:2318-2407, built from the oracle's
    projection + activation, against numpy dequant -> float64 matmul -> the library GELU."""
    torch = pytest.importorskip("torch")
    fx = F.hw_fixture_q4_gelu_cols2560(gs)
    proj = lambda m: orc.hip_reference_projection(fx["x"], m["packed"], m["scales"], m["biases"], fx["rows"], fx["cols"], gs, 4)
    want = orc.act_multiply(orc.ACT_GELU_TANH, proj(fx["gate"]), proj(fx["up"]))
    deq = lambda m: F.numpy_dequant(m["packed"], m["scales"], m["biases"], 4, gs, fx["cols"]).astype(np.float64)
    x64 = fx["x"].astype(np.float64)
    g64, u64 = deq(fx["gate"]) @ x64, deq(fx["up"]) @ x64
    ref = torch.nn.functional.gelu(torch.from_numpy(g64), approximate="tanh").numpy() * u64
    assert np.abs(want - ref).max() <= 1e-5     # far inside the reference's own 0.03
    assert np.abs(ref).max() > 1e-3             # the fixture's outputs are small but not trivial


# ---- MoE router and combine ---------------------------------------------------------------------------

def _independent_route(logits, top_k, scales=None, normalise=True):
    """numpy restatement by another route: lexsort for the order, scipy for the softmax."""
    from scipy.special import softmax
    lg = np.asarray(logits, dtype=np.float32)
    ids = np.stack([np.lexsort((np.arange(lg.shape[1]), -r.astype(np.float64)))[:top_k] for r in lg]).astype(np.int32)
    sel = np.take_along_axis(lg.astype(np.float64), ids, axis=1)
    w = softmax(sel, axis=1) if normalise else np.take_along_axis(softmax(lg.astype(np.float64), axis=1), ids, axis=1)
    if scales is not None:
        w = w * np.asarray(scales, dtype=np.float64)[ids]
    return ids, w


def test_moe_route_reference_known_answers(orc):
    # go/engine/hip/hip_qwen3_moe_router_test.go:19-58: a two-way softmax is a sigmoid
    ids, w = orc.moe_route(np.array([[1, 3, 2, 0]], np.float32), 2, normalise=True)
    assert ids.tolist() == [[1, 2]]
    s1 = 1 / (1 + math.exp(-1))
    assert abs(w[0, 0] - s1) < 1e-7 and abs(w[0, 1] - (1 - s1)) < 1e-7
    assert abs(w.sum() - 1) < 1e-6
    ids, w = orc.moe_route(np.array([[1, 3, 2, 0]], np.float32), 2, normalise=False)
    total = math.exp(1) + math.exp(3) + math.exp(2) + math.exp(0)
    assert ids.tolist() == [[1, 2]]
    assert abs(w[0, 0] - math.exp(3) / total) < 1e-7 and abs(w[0, 1] - math.exp(2) / total) < 1e-7
    assert w.sum() < 1.0
    # :64-73 both orders select the same experts
    lg = np.array([[-2, 5, 0.5, 3, -1, 1.2]], np.float32)
    assert orc.moe_route(lg, 3, normalise=True)[0].tolist() == orc.moe_route(lg, 3, normalise=False)[0].tolist() == [[1, 3, 5]]
    # go/engine/hip/hip_moe_launch_test.go:1861-1882
    assert orc.moe_route(np.array([[0.1, 2, 1, -1]], np.float32), 2)[0].tolist() == [[1, 2]]


def test_moe_route_gemma_batch_fixture_with_expert_scales(orc):
    """TestHIPGemma4MoEBatchRouteGroups_Good_MatchesReference (go/engine/hip/hip_moe_launch_test.go:1369-1400):
    weight = prob * expert scale; row 1 holds a tie (5, 5) that the lower expert id wins."""
    scores = np.array([[1, 4, 2, 3], [5, 5, -1, 0], [-2, 1, 7, 3]], np.float32)
    scales = np.array([1, 0.5, 2, 1.5], np.float32)
    ids, w = orc.moe_route(scores, 2, expert_scales=scales)
    assert ids.tolist() == [[1, 3], [0, 1], [2, 3]]
    wi, ww = _independent_route(scores, 2, scales)
    assert np.array_equal(ids, wi) and np.abs(w - ww).max() < 1e-7
    assert abs(w[1, 0] - 0.5 * 1.0) < 1e-7 and abs(w[1, 1] - 0.5 * 0.5) < 1e-7   # equal scores: 1/2 each, scaled


def test_moe_route_hardware_fixture_128_experts_with_ties(orc):
    """TestHIPHardwareMoERouterParallel_Good (go/engine/hip/hip_hardware_test.go:1197-1220): logits
    (e*37 % 23)/8 over 128 experts, top 8 -- every score value repeats five or six times."""
    lg = np.array([[np.float32((e * 37) % 23) / np.float32(8) for e in range(128)]], np.float32)
    for norm in (True, False):
        ids, w = orc.moe_route(lg, 8, normalise=norm)
        wi, ww = _independent_route(lg, 8, normalise=norm)
        assert np.array_equal(ids, wi)
        assert np.abs(w - ww).max() < 1e-7
    ids, _ = orc.moe_route(lg, 8)
    sel = lg[0, ids[0]]
    assert np.all(np.diff(sel) <= 0)
    for a, b in zip(range(7), range(1, 8)):
        if sel[a] == sel[b]:
            assert ids[0, a] < ids[0, b]


def test_moe_route_random_rows_and_rejections(orc):
    rng = np.random.default_rng(5)
    lg = rng.normal(0, 2, (37, 200)).astype(np.float32)
    lg[:, 7] = lg[:, 150]  # ties across lanes
    sc = rng.uniform(0.5, 2, 200).astype(np.float32)
    for norm in (True, False):
        ids, w = orc.moe_route(lg, 6, sc, norm)
        wi, ww = _independent_route(lg, 6, sc, norm)
        assert np.array_equal(ids, wi) and np.abs(w - ww).max() < 2e-7
    for bad in (np.nan, np.inf, -np.inf):
        x = lg.copy()
        x[3, 5] = bad
        with pytest.raises(orc.OracleError):
            orc.moe_route(x, 6)
    with pytest.raises(orc.OracleError):
        orc.moe_route(lg, 0)
    with pytest.raises(orc.OracleError):
        orc.moe_route(lg, 201)


def test_moe_combine_fp32_and_bf16_steps(orc):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(6)
    rows, top_k, n = 5, 8, 33
    y = rng.normal(0, 1, (rows * top_k, n)).astype(np.float32)
    w = rng.uniform(0, 1, rows * top_k).astype(np.float32)
    got = orc.moe_combine(y, w, rows, top_k, n)
    # float32 products summed in rank order: the library's float32 arithmetic, rank by rank
    ty, tw = torch.from_numpy(y).reshape(rows, top_k, n), torch.from_numpy(w).reshape(rows, top_k, 1)
    acc = torch.zeros(rows, n)
    for r in range(top_k):
        acc = acc + ty[:, r] * tw[:, r]
    assert np.array_equal(got, acc.numpy())
    assert np.abs(got - (y.reshape(rows, top_k, n).astype(np.float64) * w.reshape(rows, top_k, 1)).sum(1)).max() < 1e-5
    # bf16 steps: torch.bfloat16 rounds after every multiply and add
    yb = torch.from_numpy(y).bfloat16().reshape(rows, top_k, n)
    wb = torch.from_numpy(w).bfloat16().reshape(rows, top_k, 1)
    accb = yb[:, 0] * wb[:, 0]
    for r in range(1, top_k):
        accb = accb + yb[:, r] * wb[:, r]
    gotb = orc.moe_combine(yb.float().numpy().reshape(rows * top_k, n), w, rows, top_k, n, bf16_steps=True)
    assert np.array_equal(F.f32_to_bf16_bits(gotb), accb.view(torch.int16).numpy().view(np.uint16))
    # one route with weight one is the identity
    assert np.array_equal(orc.moe_combine(y[:3], np.ones(3, np.float32), 3, 1, n), y[:3])


# ---- packed (score, token) values and the greedy reference --------------------------------------------

def test_greedy_sample_reference_known_answer(orc):
    # go/engine/hip/hip_transformer_reference_test.go:182-188
    assert orc.greedy_sample_suppress([-1, 0.25, 0.2]) == (1, 0.25)
    assert orc.greedy_sample_suppress([3, 7, 7, 1])[0] == 1                  # first maximum wins
    assert orc.greedy_sample_suppress([3, 7, 7, 1], [1])[0] == 2             # suppressed tokens are skipped
    assert orc.greedy_sample_suppress([-5, -2, -9], [1]) == (0, -5.0)
    with pytest.raises(orc.OracleError):
        orc.greedy_sample_suppress([1, 2], [0, 1])
    with pytest.raises(orc.OracleError):
        orc.greedy_sample_suppress([])


def test_packed_best_orders_like_the_greedy_reference(orc):
    """max over pack(score, token) == (first) argmax: brute force over value sets that include negatives,
    signed zeros, denormals, equal scores and the float32 extremes."""
    vals = np.array([0.0, -0.0, 1e-45, -1e-45, 1.0, -1.0, 0.25, 0.2, 3.4e38, -3.4e38, 1e-30, -1e-30, 65504.0, 2.5, 2.5],
                    dtype=np.float32)
    for i, a in enumerate(vals):
        for j, b in enumerate(vals):
            pa, pb = orc.pack_greedy_best(float(a), 7), orc.pack_greedy_best(float(b), 7)
            if a < b:
                assert pa < pb, (a, b)
            elif a > b:
                assert pa > pb, (a, b)
    # equal scores: the lower token id packs higher
    assert orc.pack_greedy_best(2.5, 3) > orc.pack_greedy_best(2.5, 4)
    rng = np.random.default_rng(9)
    for _ in range(50):
        lg = rng.normal(0, 3, 40).astype(np.float32)
        lg[rng.integers(0, 40, 6)] = lg.max()        # ties for the maximum
        best = max(orc.pack_greedy_best(float(v), t) for t, v in enumerate(lg))
        tok, sc = orc.unpack_greedy_best(best)
        assert (tok, np.float32(sc)) == orc.greedy_sample_suppress(lg)
    # explicit layout: hipPackGreedyBest(1, 2) = key(1.0) << 32 | ^2
    assert orc.pack_greedy_best(1.0, 2) == ((0x3F800000 ^ 0x80000000) << 32) | 0xFFFFFFFD
    assert orc.pack_greedy_best(-1.0, 0) == ((~0xBF800000 & 0xFFFFFFFF) << 32) | 0xFFFFFFFF


def test_unpack_best_round_trip_softcap_and_errors(orc):
    for score, token in [(1.0, 2), (-3.5, 0), (0.0, 262143), (1e-40, 5)]:
        tok, sc = orc.unpack_greedy_best(orc.pack_greedy_best(score, token), 0.0, 262144)
        assert tok == token and np.float32(sc) == np.float32(score)
    tok, sc = orc.unpack_greedy_best(orc.pack_greedy_best(45.0, 9), 30.0, 100)
    assert tok == 9 and abs(sc - math.tanh(45.0 / 30.0) * 30.0) < 1e-5
    for args in [(0, 0.0, 10), (orc.pack_greedy_best(1.0, 10), 0.0, 10), (orc.pack_greedy_best(1.0, 1), -1.0, 10),
                 (orc.pack_greedy_best(1.0, 1), float("nan"), 10), (orc.pack_greedy_best(1.0, 1), 0.0, 0)]:
        with pytest.raises(orc.OracleError):
            orc.unpack_greedy_best(*args)
