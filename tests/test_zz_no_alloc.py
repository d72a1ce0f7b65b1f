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


def _free_device_bytes():
    """hipMemGetInfo's free bytes, asked of the HIP runtime the library has loaded."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


@pytest.mark.parametrize("bits,gs,K,N", [(4, 64, 2048, 9000), (8, 64, 1024, 3000), (4, 64, 512, 5000)])
def test_static_greedy_allocates_nothing_and_replays_in_a_graph(ctx, bits, gs, K, N):
    """On a context that has run nothing else: the call leaves the free device memory and the context's scratch sizes
    as they were; captured into a graph it gives aq_qmv_greedy's packed best on every replay, also after the
    activations have changed between replays."""
    import aq_mi355
    say("greedy static, fresh context", bits, gs, K, N)
    fresh = aq_mi355.Context(0)
    try:
        words, s, b = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 140)
        dw = DeviceAffine(fresh, words, s, b)
        x0, x1 = F.synthetic_x(1, K, seed=F.BASE_SEED + 141), F.synthetic_x(1, K, seed=F.BASE_SEED + 142)
        dx = fresh.to_device(x0)
        dsup = fresh.to_device(np.array([2, N - 2], dtype=np.int32))
        got = fresh.alloc(8)
        fresh.fill_zero(got)
        fresh.sync()
        free0, scratch0 = _free_device_bytes(), fresh.workspace_bytes()
        fresh.qmv_greedy_static(dx, dw.w, dw.s, dw.b, got, K, N, gs, bits, dsup, 2)
        fresh.sync()
        first = _best(got)
        assert (_free_device_bytes(), fresh.workspace_bytes()) == (free0, scratch0)
        fresh.force_variant(0, 0)                # a forced matvec variant is not consulted: same kernels, same answer
        fresh.fill_zero(got)
        fresh.qmv_greedy_static(dx, dw.w, dw.s, dw.b, got, K, N, gs, bits, dsup, 2)
        fresh.force_variant(0, -1)
        fresh.sync()
        assert _best(got) == first
        assert (_free_device_bytes(), fresh.workspace_bytes()) == (free0, scratch0)
        # the same call under capture: nothing runs until the replays
        fresh.fill_zero(got)
        fresh.capture_begin()
        fresh.qmv_greedy_static(dx, dw.w, dw.s, dw.b, got, K, N, gs, bits, dsup, 2)
        graph = fresh.capture_end()
        assert fresh.workspace_bytes() == scratch0
        want = ctx.alloc(8)
        for replay, xv in enumerate((x0, x1, x0)):
            dx.upload(xv)
            ctx.qmv_greedy(dx, dw.w, dw.s, dw.b, want, 1, K, N, gs, bits, dsup, 2)
            ctx.sync()
            fresh.fill_zero(got)
            fresh.graph_launch(graph)
            fresh.sync()
            assert _best(got) == _best(want) != 0, replay
            if replay == 0:
                assert _best(got) == first
        fresh.graph_destroy(graph)
        for t in (dx, dsup, got, want):
            t.free()
        dw.free()
    finally:
        fresh.close()


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
