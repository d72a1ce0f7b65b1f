"""The token-tile MFMA matvec kernels (5..32 rows of x as the rows of 16x16x32 MFMAs, one launch, no scratch):
the M-row contract of go/engine/metal/qmv_rows.go:14-60 and rocm_mlx_q4_projection_batch*
(go/engine/hip/kernels/quant/affine_projection_tuned.hipinc:292-472) beyond eight rows."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, check_accumulators, check_bf16_store, run_qmv, say

pytestmark = pytest.mark.gpu


def _tok_variants():
    import aq_mi355
    return [(i, n) for i, n in enumerate(aq_mi355.variant_names(0)) if n.startswith("qmvt_")]


def test_tok_every_variant(ctx, orc):
    """Each variant forced: 1..32 rows (16 for the one-set forms), K of one run of four groups up to several per
    wavefront (an idle wavefront, a ragged split), N that ends inside a set of 16 rows; fp32 accumulators and bf16
    stores; token t of an M-row call is bit-identical to token t of any other row count; 33 rows, a K that is no multiple
    of 256, a K beyond 16384, 8-bit codes are refused."""
    import aq_mi355
    N = 150
    try:
        for K, bits in [(K, bits) for bits in (4, 8) for K in (256, 768, 2048, 2816, 4096, 14336)]:
            words, s, b = F.synthetic_affine(N, K, bits, 64, seed=1500 + K // 256 + bits)
            x = F.synthetic_x(32, K, seed=1600 + K // 256)
            ref = F.reference_f64(x, words, s, b, bits, 64, K)
            dw = DeviceAffine(ctx, words, s, b)
            for idx, name in _tok_variants():
                if "_b%d_" % bits not in name:
                    continue
                ctx.force_variant(0, idx)
                full = None
                most = int(name.split("_m")[1].split("_")[0])  # rows of x the variant takes: 16, or 32 for the two-set forms
                for rows in [r for r in (most, 1, 5, 9, 16, 17, 31) if r <= most]:
                    say("tok variant", name, "K", K, "rows", rows)
                    acc = run_qmv(ctx, x[:rows], dw, rows, K, N, 64, bits, True)
                    assert ctx.last_variant(0) == name
                    check_accumulators(acc, ref[:rows], "%s K=%d rows=%d" % (name, K, rows))
                    if full is None:
                        full = acc
                    assert np.array_equal(acc.view(np.uint32), full[:rows].view(np.uint32)), (name, K, rows)
                some = min(17, most)
                out = run_qmv(ctx, x[:some], dw, some, K, N, 64, bits, False)
                check_bf16_store(out, ref[:some], name)
                assert np.array_equal(out, F.f32_to_bf16_bits(full[:some]).reshape(some, N))
            dw.free()
        idx, name = [v for v in _tok_variants() if "_b4_m32_" in v[1]][0]
        ctx.force_variant(0, idx)
        words, s, b = F.synthetic_affine(40, 16640, 4, 64, seed=1700)
        dw = DeviceAffine(ctx, words, s, b)
        for rows, K, bits in ((33, 1024, 4), (4, 1152, 4), (4, 1024, 8), (4, 16640, 4)):
            with pytest.raises(aq_mi355.AqError) as ei:
                run_qmv(ctx, np.zeros((rows, K), np.uint16), dw, rows, K, 40, 64, bits, True)
            assert ei.value.code == aq_mi355.AQ_ERR_ARG, (rows, K, bits)
        dw.free()
    finally:
        ctx.force_variant(0, -1)


@pytest.mark.parametrize("M", [2, 4, 5, 8, 16, 17, 32])
def test_tok_config2_full_shape_8bit(ctx, orc, M):
    """cfg 2's 8-bit variant at its full shape (K = 4096, N = 14336): the default path; accumulators against the
    float64 reference and, on sampled rows of x, the oracle's fp32-accumulated reference; bf16 store = RNE of the
    accumulator; two runs give the same bytes."""
    say("tok cfg2 8 bit", M)
    K, N = 4096, 14336
    words, s, b = F.synthetic_affine(N, K, 8, 64, seed=F.BASE_SEED + 2)
    x = F.synthetic_x(M, K, seed=F.BASE_SEED + 3)
    ref = F.reference_f64(x, words, s, b, 8, 64, K)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, 64, 8, True)
    assert ctx.last_variant(0).startswith("qmvt_b8_m16_" if M <= 16 else "qmvt_b8_m32_"), ctx.last_variant(0)
    check_accumulators(acc, ref, "tok cfg2 8 bit M=%d" % M)
    rows = sorted({0, M - 1})
    xf = F.bf16_bits_to_f32(x).reshape(M, K)
    o32 = orc.hip_reference_projection_batch(xf[rows].reshape(-1), len(rows), words, s, b, N, K, 64, 8)
    check_accumulators(acc[rows], o32, "tok cfg2 8 bit vs oracle M=%d" % M)
    out = run_qmv(ctx, x, dw, M, K, N, 64, 8, False)
    check_bf16_store(out, ref, "tok cfg2 8 bit bf16")
    assert np.array_equal(out, F.f32_to_bf16_bits(acc).reshape(M, N))
    again = run_qmv(ctx, x, dw, M, K, N, 64, 8, True)
    assert np.array_equal(again.view(np.uint32), acc.view(np.uint32))
    dw.free()


@pytest.mark.parametrize("M", [9, 16, 17, 32])
def test_tok_config2_full_shape(ctx, orc, M):
    """cfg 2 at its full shape (K = 4096, N = 14336) for the row counts above eight: the default path is the token-tile
    kernel (one launch); accumulators against the float64 reference and, on sampled rows of x, against the
    oracle's fp32-accumulated batch reference; bf16 store = RNE of the accumulator; two runs give the same bytes."""
    say("tok cfg2", M)
    K, N = 4096, 14336
    words, s, b = F.synthetic_affine(N, K, 4, 64, seed=F.BASE_SEED + 2)
    x = F.synthetic_x(M, K, seed=F.BASE_SEED + 3)
    ref = F.reference_f64(x, words, s, b, 4, 64, K)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, 64, 4, True)
    assert ctx.last_variant(0).startswith("qmvt_"), ctx.last_variant(0)
    check_accumulators(acc, ref, "tok cfg2 M=%d" % M)
    rows = sorted({0, M // 2, M - 1})
    xf = F.bf16_bits_to_f32(x).reshape(M, K)
    o32 = orc.hip_reference_projection_batch(xf[rows].reshape(-1), len(rows), words, s, b, N, K, 64, 4)
    check_accumulators(acc[rows], o32, "tok cfg2 vs oracle M=%d" % M)
    out = run_qmv(ctx, x, dw, M, K, N, 64, 4, False)
    check_bf16_store(out, ref, "tok cfg2 bf16")
    assert np.array_equal(out, F.f32_to_bf16_bits(acc).reshape(M, N))
    again = run_qmv(ctx, x, dw, M, K, N, 64, 4, True)
    assert np.array_equal(again.view(np.uint32), acc.view(np.uint32))
    dw.free()


def test_tok_call_in_a_graph_on_a_fresh_context(orc):
    """The token-tile path uses no workspace: a 32-row call can be captured on a context that has never run anything,
    and every replay equals the eager result."""
    import aq_mi355
    M, K, N = 32, 2048, 1000
    say("tok in a graph", M, K, N)
    words, s, b = F.synthetic_affine(N, K, 4, 64, seed=1931)
    x = F.synthetic_x(M, K, seed=1932)
    ref = F.reference_f64(x, words, s, b, 4, 64, K)
    fresh = aq_mi355.Context(0)
    try:
        dw = DeviceAffine(fresh, words, s, b)
        dx, dy = fresh.to_device(x), fresh.alloc(M * N * 4)
        fresh.capture_begin()
        fresh.qmv(dx, dw.w, dw.s, dw.b, dy, M, K, N, 64, 4, aq_mi355.AQ_OUT_F32)
        graph = fresh.capture_end()
        first = None
        for i in range(3):
            fresh.fill_zero(dy)
            fresh.graph_launch(graph)
            fresh.sync()
            got = dy.download(np.float32, M * N).copy()
            check_accumulators(got, ref, "replay %d" % i)
            if first is None:
                first = got
            assert np.array_equal(got.view(np.uint32), first.view(np.uint32)), i
        fresh.graph_destroy(graph)
        dw.free()
        dx.free()
        dy.free()
    finally:
        fresh.close()
