"""8-bit codes on the diagonal-MFMA kernels (the reference's q8 decode kernels,
go/engine/hip/kernels/quant/affine_projection.hipinc:105-149): parity with the float64 reference of the same bytes,
rows of a call against single-row calls, which shapes the selection gives them, and forced variants at the shapes
the selection leaves to other kernels."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, check_accumulators, check_bf16_store, run_qmv, say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("K,N,want", [(4096, 1000, "qmvd_b8_m4_r1_w8_d1_g0"), (2048, 777, "qmvd_b8_m4_"), (8192, 300, "qmvd_b8_m4_r1_w16_d1_g0"),
                                      (4096, 4096, "qmvd_b8_m4_r1_w8_d1_g0")])
def test_selected_shapes_match_the_reference_and_rows_match_single_rows(ctx, K, N, want):
    words, s, b = F.synthetic_affine(N, K, 8, 64, seed=F.BASE_SEED + 700 + K)
    dw = DeviceAffine(ctx, words, s, b)
    x = F.synthetic_x(4, K, seed=F.BASE_SEED + 701 + K)
    ref = F.reference_f64(x, words, s, b, 8, 64, K)
    rows = 2 if K == 2048 else 4  # (four steps: up to two rows here, more on the token-tile kernel)
    single = [run_qmv(ctx, x[r:r + 1], dw, 1, K, N, 64, 8, False)[0] for r in range(rows)]
    assert ctx.last_variant(0).startswith(want), ctx.last_variant(0)
    for M in range(1, rows + 1):
        say("diag b8", K, N, M)
        got = run_qmv(ctx, x[:M], dw, M, K, N, 64, 8, True)
        assert ctx.last_variant(0).startswith("qmvd_b8_m4_"), ctx.last_variant(0)
        check_accumulators(got, ref[:M], "diag b8 f32 %d %d %d" % (K, N, M))
        gb = run_qmv(ctx, x[:M], dw, M, K, N, 64, 8, False)
        check_bf16_store(gb, ref[:M], "diag b8 bf16 %d %d %d" % (K, N, M))
        for r in range(M):
            assert (gb[r] == single[r]).all(), (K, N, M, r)
    dw.free()


@pytest.mark.parametrize("K,N", [(640, 100), (1152, 333), (3072, 700), (1536, 64), (768, 48), (5120, 40), (7168, 96)])
def test_forced_variants_at_other_k(ctx, K, N):
    """K that is no whole number of steps, three chunks a step, odd numbers of steps: the kernels the selection would use
    if the rule were wider, forced by name."""
    import aq_mi355
    words, s, b = F.synthetic_affine(N, K, 8, 64, seed=F.BASE_SEED + 710 + K)
    dw = DeviceAffine(ctx, words, s, b)
    x = F.synthetic_x(4, K, seed=F.BASE_SEED + 711 + K)
    ref = F.reference_f64(x, words, s, b, 8, 64, K)
    names = aq_mi355.variant_names(0)
    ran = 0
    try:
        for i, nm in enumerate(names):
            if not nm.startswith("qmvd_b8_"):
                continue
            ctx.force_variant(0, i)
            for M in (1, 3, 4):
                try:
                    got = run_qmv(ctx, x[:M], dw, M, K, N, 64, 8, True)
                except aq_mi355.AqError:
                    continue  # this variant's split of K does not cover the row
                if ctx.last_variant(0) != nm:
                    continue  # (a forced variant that does not fit is passed over)
                say("diag b8 forced", nm, K, N, M)
                check_accumulators(got, ref[:M], "%s %d %d %d" % (nm, K, N, M))
                ran += 1
    finally:
        ctx.force_variant(0, -1)
    assert ran > 0, (K, N)
    dw.free()


def test_large_and_odd_shapes_stay_on_the_other_kernels(ctx):
    for K, N, M, want in ((4096, 14336, 1, "qmv_b8_m1_r1_w4_d4_g0_x0"), (3072, 512, 1, "qmv_b8_m1_"), (2048, 512, 4, "qmvt_b8_"),
                          (4096, 14336, 4, "qmvt_b8_")):
        words, s, b = F.synthetic_affine(N, K, 8, 64, seed=F.BASE_SEED + 720)
        dw = DeviceAffine(ctx, words, s, b)
        x = F.synthetic_x(M, K, seed=F.BASE_SEED + 721)
        say("b8 selection", K, N, M)
        got = run_qmv(ctx, x, dw, M, K, N, 64, 8, True)
        assert ctx.last_variant(0).startswith(want), (K, N, M, ctx.last_variant(0))
        check_accumulators(got, F.reference_f64(x, words, s, b, 8, 64, K), "b8 %d %d %d" % (K, N, M))
        dw.free()
