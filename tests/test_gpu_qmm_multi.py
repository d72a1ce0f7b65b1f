"""aq_qmm_multi: several weight matrices against one x at prefill sizes (the reference runs q|k|v and gate|up as one
matmul over model.ConcatQuantRows, go/model/quant_weight.go:32-62)."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, say

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits,M,K,Ns", [(4, 300, 1024, (520, 256, 130)), (4, 2048, 512, (4096, 1024)), (8, 130, 512, (257, 200)),
                                         (4, 40, 1024, (300, 520)), (4, 3, 2048, (64, 130, 48, 200, 96))])
def test_qmm_multi_equals_separate_calls(ctx, bits, M, K, Ns):
    """aq_qmm_multi (one pass over x for the members that need the same form of it) against one aq_qmm per member:
    the same bytes, whatever tile family each member's width selects."""
    say("qmm multi", bits, M, K, Ns)
    x = ctx.to_device(F.synthetic_x(M, K, seed=F.BASE_SEED + 600))
    mats, outs, refs = [], [], []
    for i, N in enumerate(Ns):
        w, s, b = F.synthetic_affine(N, K, bits, 64, seed=F.BASE_SEED + 610 + i)
        mats.append(DeviceAffine(ctx, w, s, b))
        y = ctx.alloc(M * N * 2)
        ctx.fill_zero(y)
        ctx.qmm(x, mats[-1].w, mats[-1].s, mats[-1].b, y, M, K, N, 64, bits, 0)
        ctx.sync()
        refs.append(y.download(np.uint16, M * N).copy())
        ctx.fill_zero(y)
        outs.append(y)
    for run in range(2):
        ctx.qmm_multi(x, [m.w for m in mats], [m.s for m in mats], [m.b for m in mats], outs, list(Ns), M, K, 64, bits, 0)
        ctx.sync()
        for i, N in enumerate(Ns):
            got = outs[i].download(np.uint16, M * N)
            assert (got == refs[i]).all(), (run, i, N, int((got != refs[i]).sum()))
            ctx.fill_zero(outs[i])
    # a single call afterwards must not believe the workspace still holds its x
    x2 = ctx.to_device(F.synthetic_x(M, K, seed=F.BASE_SEED + 601))
    y2 = ctx.alloc(M * Ns[0] * 2)
    ctx.qmm(x2, mats[0].w, mats[0].s, mats[0].b, y2, M, K, Ns[0], 64, bits, 0)
    ctx.sync()
    assert not (y2.download(np.uint16, M * Ns[0]) == refs[0]).all()
    for t in [x, x2, y2] + outs:
        t.free()
    for m in mats:
        m.free()
