"""GPU parity of the lm_head entry points (projection with fused argmax, packed scores, packed top-k)
through the C ABI against the CPU oracle.  The winning token must be the oracle's greedy token for the
device's own fp32 scores (exact), and the device scores must sit within the matvec tolerance of the
float64 reference; where two float64 reference scores are closer than that tolerance either may win."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import MAX_ABS, DeviceAffine, check_accumulators, run_qmv, say

pytestmark = pytest.mark.gpu


def _u64(buf, n):
    return buf.download(np.uint64, n)


def _unpack(packed):
    import aq_mi355
    return aq_mi355.unpack_best(int(packed))


def _unpack_all(packed):
    """numpy form of the unpack, for whole score vectors (spot-checked against aq_unpack_best below)."""
    key = (packed >> np.uint64(32)).astype(np.uint32)
    bits = np.where(key & np.uint32(0x80000000), key ^ np.uint32(0x80000000), ~key)
    toks = (~packed.astype(np.uint32)).astype(np.int64)      # low word
    return toks, bits.view(np.float32).copy()


def _scores(ctx, x, dw, M, K, N, gs, bits, suppress=None):
    dx = ctx.to_device(np.ascontiguousarray(x, np.uint16))
    ds = None if suppress is None else ctx.to_device(np.asarray(suppress, np.int32))
    out = ctx.alloc(M * N * 8)
    ctx.qmv_scores(dx, dw.w, dw.s, dw.b, out, M, K, N, gs, bits, ds, 0 if suppress is None else len(suppress))
    ctx.sync()
    got = _u64(out, M * N).reshape(M, N)
    for t in (dx, ds, out):
        if t is not None:
            t.free()
    return got


def _greedy(ctx, x, dw, M, K, N, gs, bits, suppress=None):
    dx = ctx.to_device(np.ascontiguousarray(x, np.uint16))
    ds = None if suppress is None else ctx.to_device(np.asarray(suppress, np.int32))
    best = ctx.to_device(np.full(M, 0xDEADBEEF, np.uint64))   # the call clears it itself
    ctx.qmv_greedy(dx, dw.w, dw.s, dw.b, best, M, K, N, gs, bits, ds, 0 if suppress is None else len(suppress))
    ctx.sync()
    got = _u64(best, M)
    for t in (dx, ds, best):
        if t is not None:
            t.free()
    return got


@pytest.mark.parametrize("bits,gs,M,K,N,fused", [(4, 32, 1, 1536, 32768, True), (4, 64, 1, 4096, 20011, True),
                                                 (8, 64, 1, 1024, 4096, True), (4, 64, 1, 512, 37, True),
                                                 (6, 32, 1, 192, 301, False), (4, 64, 3, 512, 1000, False),
                                                 (4, 64, 20, 1024, 515, False), (4, 32, 1, 2048, 1000, True),
                                                 (4, 64, 1, 2816, 777, True), (4, 32, 1, 4096, 50, True)])
def test_greedy_and_scores_against_oracle(ctx, orc, bits, gs, M, K, N, fused):
    say("head", bits, gs, M, K, N)
    if 32 % bits == 0:
        words, s, b = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 100)
    else:
        rng = np.random.default_rng(3)
        words = F.pack_codes(rng.integers(0, 1 << bits, size=(N, K)), bits)
        s = F.f32_to_bf16_bits((np.abs(rng.normal(0, 0.02, (N, K // gs))) + 1e-3).astype(np.float32))
        b = F.f32_to_bf16_bits(rng.normal(0, 0.05, (N, K // gs)).astype(np.float32))
    x = F.synthetic_x(M, K, seed=F.BASE_SEED + 101)
    dw = DeviceAffine(ctx, words, s, b)
    ref = F.reference_f64(x, words, s, b, bits, gs, K)
    suppress = [int(np.argmax(ref[0])), 5, N - 1]
    for sup in (None, suppress):
        packed = _scores(ctx, x, dw, M, K, N, gs, bits, sup)
        # 4-bit codes in groups of 32 or 64 with more than 1024 columns: the diagonal-MFMA kernels
        diag = bits == 4 and K > 1024 and (K % 256 == 0 if gs == 32 else K % 128 == 0)
        if fused:
            assert ctx.last_variant(0) == ("qmv_scores_diag" if diag else "qmv_scores_dot2")
        toks, dev = _unpack_all(packed)
        live = packed != 0
        if sup is not None:
            assert not live[:, sup].any()
            live[:, sup] = True
            dev[:, sup] = ref[:, sup]
            toks[:, sup] = np.asarray(sup)
        assert live.all() and np.array_equal(toks, np.broadcast_to(np.arange(N), (M, N)))
        for n in np.random.default_rng(1).integers(0, N, 40):      # the vectorised unpack against the library's
            if packed[0, n]:
                assert _unpack(packed[0, n]) == (int(toks[0, n]), float(dev[0, n]))
        check_accumulators(dev, ref, "packed scores")
        best = _greedy(ctx, x, dw, M, K, N, gs, bits, sup)
        if fused:
            assert ctx.last_variant(0) == ("qmv_greedy_diag" if diag else "qmv_greedy_dot2")
        for m in range(M):
            tok, sc = _unpack(best[m])
            want_tok, want_sc = orc.greedy_sample_suppress(dev[m], sup)
            assert (tok, np.float32(sc)) == (want_tok, np.float32(want_sc)), (m, sup)
            assert best[m] == packed[m].max()
            # against the float64 reference: the winner's reference score is within tolerance of the best one
            r = ref[m].copy()
            if sup is not None:
                r[sup] = -np.inf
            assert r[tok] >= r.max() - 2 * MAX_ABS
    dw.free()


def test_greedy_ties_and_nonfinite_rows(ctx, orc):
    """Equal rows give equal scores: the lowest token id wins.  A row whose sum overflows is skipped."""
    say("head ties")
    K, N, gs, bits = 512, 64, 64, 4
    words, s, b = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 102)
    x = F.synthetic_x(1, K, seed=F.BASE_SEED + 103)
    ref = F.reference_f64(x, words, s, b, bits, gs, K)[0]
    top = int(np.argmax(ref))
    for dup in (3, 40, 63):            # copies of the winning row at other ids
        words[dup], s[dup], b[dup] = words[top], s[top], b[top]
    # a row of +inf scales times positive x sums would need signs; use a NaN bias instead: never a candidate
    b[10, 0] = 0x7FC0
    dw = DeviceAffine(ctx, words, s, b)
    best = _greedy(ctx, x, dw, 1, K, N, gs, bits)
    tok, _ = _unpack(best[0])
    assert tok == min(top, 3)
    packed = _scores(ctx, x, dw, 1, K, N, gs, bits)
    assert packed[0, 10] == 0
    best = _greedy(ctx, x, dw, 1, K, N, gs, bits, [min(top, 3)])
    assert _unpack(best[0])[0] == sorted({top, 3, 40, 63})[1]
    # everything suppressed: no result
    best = _greedy(ctx, x, dw, 1, K, N, gs, bits, list(range(N)))
    assert best[0] == 0
    dw.free()


@pytest.mark.parametrize("count,top_k", [(1, 1), (100, 8), (2048, 64), (2049, 5), (262144, 40), (70000, 64), (5, 8), (32000, 40), (4097, 64),
                                         (151936, 40), (1100000, 16)])
def test_packed_topk_sorted_descending(ctx, count, top_k):
    import aq_mi355
    say("packed topk", count, top_k)
    rng = np.random.default_rng(count + top_k)
    scores = rng.normal(0, 4, count).astype(np.float32)
    scores[rng.integers(0, count, max(1, count // 50))] = scores.max()     # ties at the top
    packed = np.array([aq_mi355.pack_best(float(v), t) for t, v in enumerate(scores)], dtype=np.uint64)
    packed[rng.integers(0, count, count // 10)] = 0                          # suppressed entries
    din, dout = ctx.to_device(packed), ctx.alloc(top_k * 8)
    ctx.packed_topk(din, count, top_k, dout)
    ctx.sync()
    got = _u64(dout, top_k)
    want = np.sort(packed)[::-1][:top_k]
    want = np.concatenate([want, np.zeros(top_k - want.size, np.uint64)])
    assert np.array_equal(got, want)
    din.free()
    dout.free()


@pytest.mark.parametrize("shape", ["by_rank", "by_rank_reversed", "nearly_empty", "empty", "one_score", "repeats"])
@pytest.mark.parametrize("count,top_k", [(262144, 40), (65536, 64), (9000, 8), (1048576, 3), (40000, 64), (5000, 50)])
def test_packed_topk_arranged_inputs(ctx, shape, count, top_k):
    """Inputs that defeat a threshold taken from per-segment maxima (scores arranged by rank, one score
    everywhere) or leave fewer candidates than top_k still give the sorted top_k, zero-padded."""
    say("packed topk arranged", shape, count, top_k)
    rng = np.random.default_rng(count * 7 + top_k)
    idx = np.arange(count, dtype=np.uint64)
    low = np.uint64(0xFFFFFFFF) - idx
    if shape == "by_rank":
        packed = ((np.uint64(0x90000000) - idx) << np.uint64(32)) | low
    elif shape == "by_rank_reversed":
        packed = ((np.uint64(0x80000000) + idx) << np.uint64(32)) | low
    elif shape == "nearly_empty":
        packed = np.zeros(count, np.uint64)
        where = rng.choice(count, top_k - 1, replace=False)
        packed[where] = (np.uint64(0xC0000000) << np.uint64(32)) | low[where]
    elif shape == "empty":
        packed = np.zeros(count, np.uint64)
    elif shape == "one_score":
        packed = (np.uint64(0xC1234567) << np.uint64(32)) | low
    else:
        packed = rng.integers(1, 50, count).astype(np.uint64) << np.uint64(40)   # the same value many times over
    din, dout = ctx.to_device(packed), ctx.to_device(np.full(top_k, 0xDEADBEEF, np.uint64))
    for _ in range(2):                                                           # the workspace is reused
        ctx.packed_topk(din, count, top_k, dout)
    ctx.sync()
    got = _u64(dout, top_k)
    want = np.sort(packed)[::-1][:top_k]
    assert np.array_equal(got, want)
    din.free()
    dout.free()


def test_head_top_k_pipeline_and_errors(ctx, orc):
    """scores -> top-k: the k best tokens of the projection, in order, without the logits leaving the device."""
    import aq_mi355
    say("head topk pipeline")
    K, N, gs, bits, k = 1536, 50000, 32, 4, 16
    words, s, b = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 104)
    x = F.synthetic_x(1, K, seed=F.BASE_SEED + 105)
    dw = DeviceAffine(ctx, words, s, b)
    dx, dsc, dtop = ctx.to_device(x), ctx.alloc(N * 8), ctx.alloc(k * 8)
    ctx.qmv_scores(dx, dw.w, dw.s, dw.b, dsc, 1, K, N, gs, bits)
    ctx.packed_topk(dsc, N, k, dtop)
    ctx.sync()
    top = _u64(dtop, k)
    logits = run_qmv(ctx, x, dw, 1, K, N, gs, bits, True)[0]
    order = np.lexsort((np.arange(N), -logits.astype(np.float64)))[:k]
    assert [(_unpack(p)[0]) for p in top] == order.tolist()
    assert [np.float32(_unpack(p)[1]) for p in top] == [logits[i] for i in order]
    buf = ctx.alloc(4096)
    for call, code in [(lambda: ctx.qmv_greedy(buf, buf, buf, buf, None, 1, 64, 8), aq_mi355.AQ_ERR_ARG),
                       (lambda: ctx.qmv_greedy(buf, buf, buf, buf, buf, 1, 64, 8, 3), aq_mi355.AQ_ERR_SHAPE),
                       (lambda: ctx.qmv_greedy(buf, buf, buf, buf, buf, 1, 64, 8, 64, 4, None, 2), aq_mi355.AQ_ERR_ARG),
                       (lambda: ctx.qmv_scores(buf, buf, buf, buf, buf, 1, 0, 8), aq_mi355.AQ_ERR_SHAPE),
                       (lambda: ctx.packed_topk(buf, 10, 0, buf), aq_mi355.AQ_ERR_SHAPE),
                       (lambda: ctx.packed_topk(buf, 10, 65, buf), aq_mi355.AQ_ERR_UNSUPPORTED),
                       (lambda: ctx.packed_topk(None, 10, 4, buf), aq_mi355.AQ_ERR_ARG)]:
        with pytest.raises(aq_mi355.AqError) as e:
            call()
        assert e.value.code == code
    ctx.qmv_greedy(None, None, None, None, None, 0, 64, 8)     # no rows: nothing to do
    best = ctx.to_device(np.full(1, 7, np.uint64))
    ctx.qmv_greedy(None, None, None, None, best, 1, 64, 0)     # no vocabulary: best is cleared, no result
    ctx.sync()
    assert _u64(best, 1)[0] == 0
    for t in (dx, dsc, dtop, buf, best):
        t.free()
    dw.free()


def _sample(ctx, top, temperature, top_p, softcap, draw):
    dtop, dout = ctx.to_device(np.ascontiguousarray(top, np.uint64)), ctx.to_device(np.full(1, 0xDEAD, np.uint64))
    ctx.packed_topk_sample(dtop, len(top), temperature, top_p, softcap, draw, dout)
    ctx.sync()
    got = int(_u64(dout, 1)[0])
    dtop.free()
    dout.free()
    return got


def test_packed_topk_sample_against_oracle(ctx, orc):
    """The device sampler picks the oracle's candidate: the scenario of the reference's hardware test (through the
    device top-k, against the host sampler over soft-capped logits too), then random lists with holes, every
    temperature / top-p mode and out-of-range draws."""
    import aq_mi355
    say("packed topk sample")
    V = 262144
    logits = np.full(V, -100, np.float32)
    for rank in range(64):
        logits[200000 + rank * 17] = 60 - rank / 2
    packed = np.array([aq_mi355.pack_best(float(v), t) for t, v in enumerate(logits)], dtype=np.uint64)
    host = orc.softcap_logits(logits, 30)
    din = ctx.to_device(packed)
    for k in (40, 64):
        dtop, dout = ctx.alloc(k * 8), ctx.alloc(8)
        ctx.packed_topk(din, V, k, dtop)
        for top_p in (1.0, 0.95):
            for draw in (0, 0.1, 0.5, 0.9, 0.999999):
                ctx.packed_topk_sample(dtop, k, 1.0, top_p, 30.0, draw, dout)
                ctx.sync()
                got = int(_u64(dout, 1)[0])
                assert got == orc.packed_topk_sample(_u64(dtop, k), 1.0, top_p, 30.0, draw), (k, top_p, draw)
                assert _unpack(got)[0] == orc.host_sample(host, 1.0, k, top_p, draw)[0], (k, top_p, draw)
        dtop.free()
        dout.free()
    din.free()
    rng = np.random.default_rng(77)
    for case in range(60):
        k = int(rng.integers(1, 129))
        scores = np.sort(rng.normal(0, 3, k).astype(np.float32))[::-1]
        top = np.array([aq_mi355.pack_best(float(s), int(t)) for s, t in zip(scores, rng.permutation(100000)[:k])], np.uint64)
        top[rng.random(k) < 0.15] = 0
        temperature = float(rng.choice([0.0, 0.3, 1.0, 2.5]))
        top_p = float(rng.choice([0.0, 0.5, 0.9, 1.0]))
        softcap = float(rng.choice([0.0, 2.0, 30.0]))
        for draw in (-0.5, 0.0, float(rng.random()), float(rng.random()), 0.999999999, 1.0, 3.0):
            want = orc.packed_topk_sample(top, temperature, top_p, softcap, draw)
            assert _sample(ctx, top, temperature, top_p, softcap, draw) == want, (case, k, temperature, top_p, softcap, draw)
    assert _sample(ctx, np.zeros(5, np.uint64), 1.0, 1.0, 0.0, 0.5) == 0
    huge = np.array([aq_mi355.pack_best(3e38, 1), aq_mi355.pack_best(-3e38, 2)], np.uint64)     # weight 1 and exp(-inf) = 0
    assert _sample(ctx, huge, 1e-3, 1.0, 0.0, 0.999) == orc.packed_topk_sample(huge, 1e-3, 1.0, 0.0, 0.999) == int(huge[0])
    buf = ctx.alloc(1024)
    for call, code in [(lambda: ctx.packed_topk_sample(buf, 0, 1.0, 1.0, 0.0, 0.5, buf), aq_mi355.AQ_ERR_SHAPE),
                       (lambda: ctx.packed_topk_sample(buf, 129, 1.0, 1.0, 0.0, 0.5, buf), aq_mi355.AQ_ERR_UNSUPPORTED),
                       (lambda: ctx.packed_topk_sample(None, 4, 1.0, 1.0, 0.0, 0.5, buf), aq_mi355.AQ_ERR_ARG),
                       (lambda: ctx.packed_topk_sample(buf, 4, -1.0, 1.0, 0.0, 0.5, buf), aq_mi355.AQ_ERR_ARG),
                       (lambda: ctx.packed_topk_sample(buf, 4, 1.0, 1.5, 0.0, 0.5, buf), aq_mi355.AQ_ERR_ARG),
                       (lambda: ctx.packed_topk_sample(buf, 4, 1.0, 1.0, float("inf"), 0.5, buf), aq_mi355.AQ_ERR_ARG),
                       (lambda: ctx.packed_topk_sample(buf, 4, 1.0, 1.0, 0.0, float("nan"), buf), aq_mi355.AQ_ERR_ARG)]:
        with pytest.raises(aq_mi355.AqError) as e:
            call()
        assert e.value.code == code
    buf.free()


def test_sampling_pipeline_captured(ctx, orc):
    """scores -> top-k -> sampler recorded into one graph (after an eager call has sized the scratch) and replayed with
    eager work in between: every replay gives the eager token, which is the oracle's choice over the device's list."""
    say("sampling pipeline captured")
    K, N, gs, bits, k = 1536, 32768, 32, 4, 40
    words, s, b = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 106)
    dw = DeviceAffine(ctx, words, s, b)
    xs = [ctx.to_device(F.synthetic_x(1, K, seed=F.BASE_SEED + 107 + i)) for i in range(2)]
    dsc, dtop, dbest, dx = ctx.alloc(N * 8), ctx.alloc(k * 8), ctx.alloc(8), ctx.alloc(K * 2)

    def pipeline():
        ctx.qmv_scores(dx, dw.w, dw.s, dw.b, dsc, 1, K, N, gs, bits)
        ctx.packed_topk(dsc, N, k, dtop)
        ctx.packed_topk_sample(dtop, k, 0.9, 0.9, 30.0, 0.61, dbest)

    want = []
    for x in xs:                                   # eager, per input
        ctx._check(ctx.lib.aq_d2d(ctx.handle, dx.ptr, x.ptr, K * 2))
        pipeline()
        ctx.sync()
        got = int(_u64(dbest, 1)[0])
        assert got == orc.packed_topk_sample(_u64(dtop, k), 0.9, 0.9, 30.0, 0.61) and got != 0
        want.append(got)
    ctx.capture_begin()
    pipeline()
    graph = ctx.capture_end()
    for i in range(4):
        ctx._check(ctx.lib.aq_d2d(ctx.handle, dx.ptr, xs[i % 2].ptr, K * 2))
        ctx.fill_zero(dbest)
        ctx.graph_launch(graph)
        ctx.sync()
        assert int(_u64(dbest, 1)[0]) == want[i % 2], i
    ctx.graph_destroy(graph)
    for t in xs + [dsc, dtop, dbest, dx]:
        t.free()
    dw.free()


def test_graph_is_refused_once_the_workspace_has_moved(orc):
    """A captured graph carries the address of the context's workspace.  When a later call makes the workspace
    grow (the old block is freed), launching that graph must be refused, not run; a graph that never touched the
    workspace still launches."""
    import aq_mi355
    say("graph vs workspace growth")
    c = aq_mi355.Context(0)
    try:
        K, N, k = 1024, 4096, 8
        words, s, b = F.synthetic_affine(N, K, 4, 64, seed=F.BASE_SEED + 120)
        dw = DeviceAffine(c, words, s, b)
        dx = c.to_device(F.synthetic_x(1, K, seed=F.BASE_SEED + 121))
        dsc, dtop, dy = c.alloc(N * 8), c.alloc(k * 8), c.alloc(N * 2)
        c.qmv_scores(dx, dw.w, dw.s, dw.b, dsc, 1, K, N, 64, 4)
        c.packed_topk(dsc, N, k, dtop)          # eager: sizes the workspace
        c.sync()
        want = _u64(dtop, k).copy()
        c.capture_begin()
        c.packed_topk(dsc, N, k, dtop)
        with_ws = c.capture_end()
        c.capture_begin()
        c.qmv(dx, dw.w, dw.s, dw.b, dy, 1, K, N, 64, 4)
        without_ws = c.capture_end()
        c.graph_launch(with_ws)
        c.sync()
        assert np.array_equal(_u64(dtop, k), want)
        c.reserve_workspace_bytes(64 << 20)      # the workspace moves
        with pytest.raises(aq_mi355.AqError) as e:
            c.graph_launch(with_ws)
        assert e.value.code == aq_mi355.AQ_ERR_UNSUPPORTED and "workspace" in str(e.value)
        c.graph_launch(without_ws)               # no workspace inside: still fine
        c.sync()
        c.capture_begin()                        # captured again over the new block: runs
        c.packed_topk(dsc, N, k, dtop)
        again = c.capture_end()
        c.fill_zero(dtop)
        c.graph_launch(again)
        c.sync()
        assert np.array_equal(_u64(dtop, k), want)
        for g in (with_ws, without_ws, again):
            c.graph_destroy(g)
        for t in (dx, dsc, dtop, dy):
            t.free()
        dw.free()
    finally:
        c.close()


@pytest.mark.parametrize("bits,gs,K,N,exact", [(4, 64, 2048, 1000, True), (4, 64, 4096, 5000, True), (4, 64, 14336, 300, False),
                                               (4, 32, 1536, 4099, False), (8, 64, 512, 50, False), (4, 64, 256, 10, False),
                                               (6, 32, 192, 301, False)])
def test_greedy_over_a_candidate_list(ctx, orc, bits, gs, K, N, exact):
    """aq_qmv_greedy_selected (rocm_mlx_q4_projection_selected_greedy, affine_projection_fused.hipinc:485-546): the winner
    is the oracle's greedy token over the logits with every row outside the list suppressed; ids out of range are
    skipped, duplicates are harmless, equal scores go to the lowest id, an empty or all-invalid list gives 0.  exact:
    shapes whose gathered and dense kernels compute the same bytes (the device's own logits decide); elsewhere the
    float64 reference decides, within the matvec tolerance."""
    say("selected greedy", bits, gs, K, N)
    rng = np.random.default_rng(K + N)
    if 32 % bits == 0:
        words, s, b = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 140)
    else:
        words = F.pack_codes(rng.integers(0, 1 << bits, size=(N, K)), bits)
        s = F.f32_to_bf16_bits((np.abs(rng.normal(0, 0.02, (N, K // gs))) + 1e-3).astype(np.float32))
        b = F.f32_to_bf16_bits(rng.normal(0, 0.05, (N, K // gs)).astype(np.float32))
    # rows 3 and 7 equal row 5: equal scores, the lowest id among the listed ones must win when they lead
    for dup in (3, 7):
        if N > 8:
            words[dup], s[dup], b[dup] = words[5], s[5], b[5]
    x = F.synthetic_x(1, K, seed=F.BASE_SEED + 141)
    dw = DeviceAffine(ctx, words, s, b)
    ref = F.reference_f64(x, words, s, b, bits, gs, K)[0]
    logits = run_qmv(ctx, x, dw, 1, K, N, gs, bits, True)[0]
    dx = ctx.to_device(np.ascontiguousarray(x, np.uint16))
    best = ctx.to_device(np.full(1, 0xDEADBEEF, np.uint64))
    top = int(np.argmax(ref))
    lists = [rng.integers(0, N, size=n).tolist() for n in (1, 7, 40, min(N, 600))]
    lists.append([top, -1, N, N + 5, top, 2 ** 31 - 1])               # ids out of range around the best row
    if N > 8:
        lists.append([7, 5, 3, 7])                                     # three equal rows: id 3 wins
        lists.append(sorted(set(range(N)) - {top})[:2000])             # everything but the best row
    lists.append([-5, N, N + 1])                                       # nothing valid
    for cand in lists:
        dc = ctx.to_device(np.asarray(cand, np.int32))
        ctx.qmv_greedy_selected(dx, dw.w, dw.s, dw.b, dc, len(cand), best, K, N, gs, bits)
        ctx.sync()
        got = int(_u64(best, 1)[0])
        valid = sorted({c for c in cand if 0 <= c < N})
        if not valid:
            assert got == 0
            continue
        tok, score = _unpack(got)
        assert tok in valid
        others = np.array(sorted(set(range(N)) - set(valid)), np.int32)
        if exact:
            want, want_score = orc.greedy_sample_suppress(logits, others)
            assert (tok, score) == (want, want_score), (cand[:8], tok, want)
        else:
            assert abs(score - ref[tok]) <= MAX_ABS + 2e-3 * abs(ref[tok])
            assert ref[tok] >= max(ref[v] for v in valid) - 2 * (MAX_ABS + 2e-3 * abs(ref[tok]))
        if cand == [7, 5, 3, 7]:
            assert tok == 3
        dc.free()
    # an empty list and an empty vocabulary: "no result"
    ctx.qmv_greedy_selected(dx, dw.w, dw.s, dw.b, None, 0, best, K, N, gs, bits)
    ctx.sync()
    assert int(_u64(best, 1)[0]) == 0
    import aq_mi355
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.qmv_greedy_selected(dx, dw.w, dw.s, dw.b, None, 3, best, K, N, gs, bits)
    assert e.value.code == aq_mi355.AQ_ERR_ARG
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.qmv_greedy_selected(dx, dw.w, dw.s, dw.b, best, 70000, best, K, N, gs, bits)
    assert e.value.code == aq_mi355.AQ_ERR_UNSUPPORTED
    for t in (dx, best):
        t.free()
    dw.free()
