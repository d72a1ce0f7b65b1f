"""The kernel the library picks for a call, per (bits, group size, rows of x, K): one case per rule of the selection
table in csrc/aq_api.hip, each also checked against the float64 reference, so that a rule that sends a shape to a
family that cannot take it shows up as a wrong result and not only as a wrong name."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, check_accumulators, run_qmv, say

pytestmark = pytest.mark.gpu

N = 520  # ragged against every family's rows per workgroup (16, 32, 64, 128, 256)

# bits, group, rows, K, the kernel-name prefixes the rule may answer with
CASES = [
    (4, 64, 1, 4096, ("qmvd_",)),                    # diagonal MFMA: one row, K up to 16 steps of 1024
    (4, 64, 1, 14336, ("qmvd_",)),
    (4, 64, 8, 4096, ("qmvd_",)),                    # ... up to 8 rows at 2..4 steps
    (4, 64, 8, 4096 - 128, ("qmvd_",)),
    (4, 64, 16, 14336, ("qmvt_b4_m16_",)),           # token tile, 16-token form: 9..16 rows, K a multiple of 256
    (4, 32, 2, 1536, ("qmvd_",)),                    # groups of 32
    (8, 64, 8, 4096, ("qmvt_b8_m16_",)),             # token tile, 8 bit: 5..16 rows
    (8, 64, 16, 4096, ("qmvt_b8_m16_",)),
    (4, 64, 9, 4096, ("qmvt_b4_m16_",)),
    (4, 64, 17, 4096, ("qmvt_b4_m32_",)),            # token tile, 32-token form: 17..32 rows
    (4, 64, 32, 4096, ("qmvt_b4_m32_",)),
    (8, 64, 1, 4096, ("qmvd_b8_",)),                 # diagonal MFMA, 8 bit: up to four rows, K of 2048, 4096, 8192
    (8, 64, 4, 4096, ("qmvd_b8_",)),
    (8, 64, 1, 3072, ("qmv_b8_",)),                  # dot2: one row of 8-bit codes at other K
    (8, 128, 1, 4096, ("qmv_b8_",)),
    (8, 64, 4, 3072, ("qmvt_b8_m16_",)),             # token tile, 8 bit: 2..16 rows, K a multiple of 256
    (8, 64, 4, 4096 + 64, ("qmvb_", "qmv_b8_")),     # ... block MFMA or dot2 for other K
    (4, 64, 8, 14336, ("qmvd_b4_m4_",)),             # 5..8 rows at a K of more than four steps: two launches of four rows
    (4, 64, 3, 14336 + 128, ("qmvd_b4_m4_",)),       # ... up to four rows in one (15 steps, the last one short)
    (4, 64, 8, 16384 + 128, ("qmv_b4_",)),           # K beyond the diagonal kernels: the dot2 kernels, four rows a launch
    (4, 64, 12, 16384 + 128, ("qmvb_", "qmmf_", "qmmt_")),
    (4, 128, 1, 4096, ("qmv_b4_",)),                 # dot2: groups of 128
    (4, 64, 1, 2880, ("qmv_b4_",)),                  # dot2: K = 45 groups
    (4, 64, 3, 2880, ("qmvb_", "qmv_b4_")),
    (3, 64, 2, 512, ("qmv_generic",)),               # any width
    (6, 32, 1, 512, ("qmv_six",)),
    (6, 64, 1, 512, ("qmv_six",)),
    (6, 64, 4, 4096, ("qmv_six",)),
    (4, 64, 48, 4096, ("qmmf_",)),                   # 33..64 rows, K a multiple of 256: K shared out over workgroups
    (8, 64, 24, 4096, ("qmvt_b8_m32_",)),            # token tile, 8 bit, 32-token form
    (8, 64, 40, 4096, ("qmmf_",)),                   # 8 bit beyond 32 rows
    (4, 64, 20, 320, ("qmmt_b4_mb1_nb2_wm1_wn4",)),  # fewer than 64 rows, K no multiple of 256: 32 x 256 tiles
    (4, 64, 40, 320, ("qmmt_b4_mb2_nb2_wm1_wn4",)),  # ... 64 x 256 tiles
    (8, 64, 70, 320, ("qmmt_b8_mb2_nb2_wm2_wn2",)),  # 64 rows and more: 128 x 128 tiles
    (4, 64, 20, 4096 + 64, ("qmvb_", "qmmt_")),
]


@pytest.mark.parametrize("bits,gs,M,K,prefixes", CASES)
def test_selected_family(ctx, bits, gs, M, K, prefixes):
    say("selection", bits, gs, M, K)
    words, s, b = F.synthetic_affine(N, K, bits, gs, seed=900 + bits + M)
    x = F.synthetic_x(M, K, seed=950 + M)
    ref = F.reference_f64(x, words, s, b, bits, gs, K)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, gs, bits, True)
    name = ctx.last_variant(0)
    assert name.startswith(prefixes), (name, prefixes)
    check_accumulators(acc, ref, name)
    dw.free()


@pytest.mark.parametrize("M", [1, 3, 4])
def test_matmul_of_few_rows_runs_as_matvec(ctx, M):
    """aq_qmm with up to four rows of x takes the matvec selection: same kernel, same bytes as aq_qmv."""
    K = 4096
    words, s, b = F.synthetic_affine(N, K, 4, 64, seed=990)
    x = F.synthetic_x(M, K, seed=991)
    dw = DeviceAffine(ctx, words, s, b)
    via_qmv = run_qmv(ctx, x, dw, M, K, N, 64, 4, True)
    name = ctx.last_variant(0)
    via_qmm = run_qmv(ctx, x, dw, M, K, N, 64, 4, True, fn="qmm")
    assert ctx.last_variant(1) == name and name.startswith("qmvd_")
    assert np.array_equal(via_qmv.view(np.uint32), via_qmm.view(np.uint32))
    dw.free()


@pytest.mark.parametrize("off,bits,M,K,prefixes", [
    ("diag", 4, 1, 4096, ("qmv_b4_",)),                 # one row falls through to the dot2 kernels
    ("diag,dot2", 4, 1, 4096, ("qmv_generic",)),        # ... and past them to the any-width kernel
    ("tok", 4, 16, 4096, ("qmmf_", "qmvb_")),           # 16 rows without the token-tile kernels
    ("tok,tiles,blk", 4, 16, 4096, ("qmv_generic",)),
    ("blk", 8, 1, 3072, ("qmv_b8_",)),
    ("diag", 8, 1, 4096, ("qmv_b8_",)),                 # 8-bit codes without the diagonal kernels: dot2 again
    ("nothing-by-that-name", 4, 1, 4096, ("qmvd_",)),   # unknown names switch nothing off
])
def test_route_switches_from_the_environment(monkeypatch, off, bits, M, K, prefixes):
    """AQ_MI355_DISABLE, read when a context is created, takes kernel families out of the selection; the call then
    runs on the next family that takes the shape, with a result inside the same tolerance."""
    import aq_mi355
    say("route switches", off, bits, M, K)
    monkeypatch.setenv("AQ_MI355_DISABLE", off)
    c = aq_mi355.Context(0)
    try:
        words, s, b = F.synthetic_affine(N, K, bits, 64, seed=1200 + bits + M)
        x = F.synthetic_x(M, K, seed=1250 + M)
        ref = F.reference_f64(x, words, s, b, bits, 64, K)
        dw = DeviceAffine(c, words, s, b)
        acc = run_qmv(c, x, dw, M, K, N, 64, bits, True)
        name = c.last_variant(0)
        assert name.startswith(prefixes), (name, prefixes)
        check_accumulators(acc, ref, name)
        dw.free()
    finally:
        c.close()


@pytest.mark.parametrize("M,K,Nq,prefix", [
    (1024, 2048, 14336, "qmmh_b4_mb4_nb2_wm2_wn4"),        # 224 tiles of 256 x 256: 7/8 of a tile per CU
    (768, 2048, 14336, "qmmh_b4_mb3_nb2_wm2_wn4"),         # 168 such tiles or 224 of 192 x 256: one round either way
    (768, 2048, 10240, "qmmh_b4_mb4_nb2_wm2_wn2_s2c"),     # 120 such tiles, 240 of 256 x 128
    (256, 2048, 14336, "qmmt_b4_mb2_nb2_wm2_wn2"),         # 112 tiles of 256 x 128: the 128 x 128 tiles
])
def test_selected_prefill_tiles(ctx, M, K, Nq, prefix):
    """aq_qmm picks its tile kernel by how much of the chip the tiles cover; sampled output columns against float64."""
    say("prefill selection", M, K, Nq)
    words, s, b = F.synthetic_affine(Nq, K, 4, 64, seed=1300 + M)
    x = F.synthetic_x(M, K, seed=1350 + M)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, Nq, 64, 4, True, fn="qmm")
    assert ctx.last_variant(1) == prefix, ctx.last_variant(1)
    cols = np.random.default_rng(5).choice(Nq, 96, replace=False)
    ref = F.reference_f64(x, words[cols], s[cols], b[cols], 4, 64, K)
    check_accumulators(acc[:, cols], ref, prefix)
    dw.free()
