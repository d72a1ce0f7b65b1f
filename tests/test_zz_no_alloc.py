"""aq_qmv_greedy_static, the entry point that allocates nothing, against aq_qmv_greedy (bit-identical packed best),
twice in a row on the same GPU, the second call with a smaller input: the scratch array keeps the first call's
contents."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, say

pytestmark = pytest.mark.gpu


def _best(buf):
    return int(buf.download(np.uint64, 1)[0])


@pytest.mark.parametrize("bits,gs,K,shapes", [(4, 32, 1536, (40000, 4112)), (4, 64, 2048, (9000, 520)), (8, 64, 1024, (3000, 257)),
                                               (4, 64, 512, (5000, 33))])
def test_static_greedy_matches_greedy(ctx, orc, bits, gs, K, shapes):
    import aq_mi355
    for call, N in enumerate(shapes):            # the second call is the smaller one
        say("greedy static", bits, gs, K, N)
        words, s, b = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 130 + call)
        dw = DeviceAffine(ctx, words, s, b)
        dx = ctx.to_device(F.synthetic_x(1, K, seed=F.BASE_SEED + 132 + call))
        sup = np.array([1, 5, N - 1], dtype=np.int32)
        dsup = ctx.to_device(sup)
        want, got = ctx.alloc(8), ctx.alloc(8)
        for suppress, count in ((None, 0), (dsup, 3)):
            ctx.qmv_greedy(dx, dw.w, dw.s, dw.b, want, 1, K, N, gs, bits, suppress, count)
            ctx.fill_zero(got)
            ctx.qmv_greedy_static(dx, dw.w, dw.s, dw.b, got, K, N, gs, bits, suppress, count)
            ctx.sync()
            assert _best(got) == _best(want) != 0, (N, count)
        token, _ = aq_mi355.unpack_best(_best(want), 0.0, N)
        assert token not in (1, 5, N - 1)
        for t in (dx, dsup, want, got):
            t.free()
        dw.free()


def test_static_greedy_limits(ctx):
    import aq_mi355
    buf = ctx.alloc(1 << 16)
    ctx.qmv_greedy_static(None, None, None, None, buf, 64, 0, 64, 4)          # no rows: "no result", like aq_qmv_greedy
    ctx.sync()
    with pytest.raises(aq_mi355.AqError) as e:                                  # 6-bit codes: not a fused shape
        ctx.qmv_greedy_static(buf, buf, buf, buf, buf, 64, 8, 32, 6)
    assert e.value.code == aq_mi355.AQ_ERR_UNSUPPORTED
    with pytest.raises(aq_mi355.AqError) as e:                                  # more partial maxima than the array holds
        ctx.qmv_greedy_static(buf, buf, buf, buf, buf, 64, 1 << 21, 64, 4)
    assert e.value.code == aq_mi355.AQ_ERR_SIZE
    buf.free()
