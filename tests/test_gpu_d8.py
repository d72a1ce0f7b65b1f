"""The MFMA matvec kernels for 8-bit codes (up to 16 rows of x as the rows of a 16x16x32 MFMA): the q8 forms of
rocm_mlx_q4_projection* (go/engine/hip/kernels/quant/affine_projection.hipinc:105-149,
affine_projection_tuned.hipinc:561-1051) and the M-row contract of go/engine/metal/qmv_rows.go:14-60."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, check_accumulators, check_bf16_store, run_qmv, say

pytestmark = pytest.mark.gpu


def _d8_variants():
    import aq_mi355
    return [(i, n) for i, n in enumerate(aq_mi355.variant_names(0)) if n.startswith("qmvd8_")]


def test_d8_every_variant(ctx, orc):
    """Each variant forced: 1..16 rows of x (the wavefront-staged and the workgroup-staged form), K of all the steps of
    1024 codes its wavefronts take, a last step of one run of four groups, an idle wavefront; N that ends inside a set of
    16 rows; fp32 accumulators and bf16 stores; token t of an M-row call is bit-identical to token t of any other row
    count; 17 rows, more steps than wavefronts, a K that is no multiple of 256 and 4-bit codes are refused."""
    import aq_mi355
    N = 150
    data = {}
    try:
        for idx, name in _d8_variants():
            nw = int(name.split("_w")[1])
            for K in sorted({1024 * nw, 1024 * nw - 256, 1024 * (nw - 1) + 256, 1024 * max(1, nw - 1)}):
                if K < 256:
                    continue
                if K not in data:
                    words, s, b = F.synthetic_affine(N, K, 8, 64, seed=2500 + K // 256)
                    x = F.synthetic_x(16, K, seed=2600 + K // 256)
                    data[K] = (DeviceAffine(ctx, words, s, b), x, F.reference_f64(x, words, s, b, 8, 64, K))
                dw, x, ref = data[K]
                ctx.force_variant(0, idx)
                full = None
                fits = [r for r in (16, 15, 8, 5, 4, 3, 2, 1) if r * (2 * K + 16) + r * (K // 128 + 1) * 16 <= 130 * 1024]
                for rows in fits:            # the largest first: the others are compared with its tokens
                    say("d8 variant", name, "K", K, "rows", rows)
                    acc = run_qmv(ctx, x[:rows], dw, rows, K, N, 64, 8, True)
                    assert ctx.last_variant(0) == name
                    # 8-bit weights reach ~5 and outputs ~100: the bounds are relative to that scale
                    scale = max(1.0, np.abs(ref[:rows]).max() / 8)
                    check_accumulators(acc / scale, ref[:rows] / scale, "%s K=%d rows=%d" % (name, K, rows))
                    if full is None:
                        full = acc
                    assert np.array_equal(acc.view(np.uint32), full[:rows].view(np.uint32)), (name, K, rows)
                if full is not None and full.shape[0] >= 3:
                    out = run_qmv(ctx, x[:3], dw, 3, K, N, 64, 8, False)
                    assert np.array_equal(out, F.f32_to_bf16_bits(full[:3]).reshape(3, N))
            dw, x, ref = data[1024 * nw]
            for rows, K, bits in ((17, 1024 * nw, 8), (1, 1024 * nw + 256, 8), (1, 1024 * nw - 64, 8), (1, 1024 * nw, 4)):
                with pytest.raises(aq_mi355.AqError) as ei:
                    run_qmv(ctx, np.zeros((rows, K), np.uint16), dw, rows, K, N, 64, bits, True)
                assert ei.value.code == aq_mi355.AQ_ERR_ARG, (name, rows, K, bits)
    finally:
        ctx.force_variant(0, -1)
    for dw, _, _ in data.values():
        dw.free()


@pytest.mark.parametrize("M", [5, 8, 16])
def test_d8_config2_full_shape(ctx, orc, M):
    """cfg 2's 8-bit variant at its full shape (K = 4096, N = 14336): the default path; accumulators against the
    float64 reference and, on sampled rows of x, the oracle's fp32-accumulated reference; bf16 store = RNE of the
    accumulator; two runs give the same bytes."""
    say("d8 cfg2", M)
    K, N = 4096, 14336
    words, s, b = F.synthetic_affine(N, K, 8, 64, seed=F.BASE_SEED + 2)
    x = F.synthetic_x(M, K, seed=F.BASE_SEED + 3)
    ref = F.reference_f64(x, words, s, b, 8, 64, K)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, 64, 8, True)
    assert ctx.last_variant(0).startswith("qmvd8_"), ctx.last_variant(0)
    check_accumulators(acc, ref, "d8 cfg2 M=%d" % M)
    rows = sorted({0, M - 1})
    xf = F.bf16_bits_to_f32(x).reshape(M, K)
    o32 = orc.hip_reference_projection_batch(xf[rows].reshape(-1), len(rows), words, s, b, N, K, 64, 8)
    check_accumulators(acc[rows], o32, "d8 cfg2 vs oracle M=%d" % M)
    out = run_qmv(ctx, x, dw, M, K, N, 64, 8, False)
    check_bf16_store(out, ref, "d8 cfg2 bf16")
    assert np.array_equal(out, F.f32_to_bf16_bits(acc).reshape(M, N))
    again = run_qmv(ctx, x, dw, M, K, N, 64, 8, True)
    assert np.array_equal(again.view(np.uint32), acc.view(np.uint32))
    dw.free()
