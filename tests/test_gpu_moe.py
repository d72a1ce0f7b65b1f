"""GPU parity of the device MoE router and combine, and of a whole routed-expert block that never leaves
the device (router -> gate|up gather with GELU -> down gather -> combine), through the C ABI against the
CPU oracle.  Expert ids must match exactly; weights to fp32 rounding of the device exp."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import MAX_ABS, DeviceAffine, say

pytestmark = pytest.mark.gpu


def _route(ctx, logits, top_k, scales=None, normalise=True, bf16=False):
    import aq_mi355
    rows, experts = logits.shape
    dl = ctx.to_device(F.f32_to_bf16_bits(logits) if bf16 else np.ascontiguousarray(logits, np.float32))
    ds = None if scales is None else ctx.to_device(np.ascontiguousarray(scales, np.float32))
    di, dw, dt = ctx.alloc(rows * top_k * 4), ctx.alloc(rows * top_k * 4), ctx.alloc(rows * top_k * 4)
    ctx.moe_route(dl, rows, experts, top_k, di, dw, dt, ds, normalise, aq_mi355.AQ_LOGITS_BF16 if bf16 else 0)
    ctx.sync()
    ids = di.download(np.int32, rows * top_k).reshape(rows, top_k)
    w = dw.download(np.float32, rows * top_k).reshape(rows, top_k)
    tok = dt.download(np.int32, rows * top_k).reshape(rows, top_k)
    for t in (dl, ds, di, dw, dt):
        if t is not None:
            t.free()
    return ids, w, tok


def test_route_reference_known_answers(ctx, orc):
    """go/engine/hip/hip_qwen3_moe_router_test.go:19-73, hip_moe_launch_test.go:1369-1400, 1861-1882."""
    say("moe route KATs")
    ids, w, tok = _route(ctx, np.array([[1, 3, 2, 0]], np.float32), 2)
    s1 = 1 / (1 + np.exp(-1.0))
    assert ids.tolist() == [[1, 2]] and tok.tolist() == [[0, 0]]
    assert abs(w[0, 0] - s1) < 1e-6 and abs(w[0, 1] - (1 - s1)) < 1e-6
    ids, w, _ = _route(ctx, np.array([[1, 3, 2, 0]], np.float32), 2, normalise=False)
    total = np.exp(1.0) + np.exp(3.0) + np.exp(2.0) + 1
    assert ids.tolist() == [[1, 2]]
    assert abs(w[0, 0] - np.exp(3.0) / total) < 1e-6 and abs(w[0, 1] - np.exp(2.0) / total) < 1e-6
    scores = np.array([[1, 4, 2, 3], [5, 5, -1, 0], [-2, 1, 7, 3]], np.float32)
    scales = np.array([1, 0.5, 2, 1.5], np.float32)
    ids, w, tok = _route(ctx, scores, 2, scales)
    oi, ow = orc.moe_route(scores, 2, scales)
    assert np.array_equal(ids, oi) and ids.tolist() == [[1, 3], [0, 1], [2, 3]]
    assert np.abs(w - ow).max() < 1e-6
    assert tok.tolist() == [[0, 0], [1, 1], [2, 2]]
    assert _route(ctx, np.array([[0.1, 2, 1, -1]], np.float32), 2)[0].tolist() == [[1, 2]]


@pytest.mark.parametrize("normalise", [True, False])
def test_route_hardware_fixture_128_experts(ctx, orc, normalise):
    """go/engine/hip/hip_hardware_test.go:1197-1220: heavy ties, resolved towards the lower expert id."""
    say("moe route 128 experts", normalise)
    lg = np.array([[np.float32((e * 37) % 23) / np.float32(8) for e in range(128)]], np.float32)
    ids, w, _ = _route(ctx, lg, 8, normalise=normalise)
    oi, ow = orc.moe_route(lg, 8, normalise=normalise)
    assert np.array_equal(ids, oi)
    assert np.abs(w - ow).max() <= 2e-6 * ow.max() + 1e-9


@pytest.mark.parametrize("experts,top_k,rows", [(128, 8, 8), (4, 4, 3), (64, 1, 5), (65, 2, 9), (200, 6, 37), (256, 32, 2),
                                                (1000, 64, 3), (1024, 8, 130), (8, 2, 2048)])
def test_route_random_against_oracle(ctx, orc, experts, top_k, rows):
    say("moe route random", experts, top_k, rows)
    rng = np.random.default_rng(experts * 7 + top_k)
    lg = rng.normal(0, 2, (rows, experts)).astype(np.float32)
    if experts > 70:
        lg[:, 3] = lg[:, 67]   # equal scores held by different lanes and slots
    sc = rng.uniform(0.5, 2, experts).astype(np.float32)
    for norm in (True, False):
        for scales in (None, sc):
            ids, w, tok = _route(ctx, lg, top_k, scales, norm)
            oi, ow = orc.moe_route(lg, top_k, scales, norm)
            assert np.array_equal(ids, oi), (norm, scales is None)
            assert (np.abs(w - ow) <= 4e-6 * np.abs(ow) + 1e-9).all()
            assert np.array_equal(tok, np.repeat(np.arange(rows), top_k).reshape(rows, top_k))
    # bf16 scores: the oracle on the widened values
    lb = F.bf16_bits_to_f32(F.f32_to_bf16_bits(lg)).reshape(rows, experts)
    ids, w, _ = _route(ctx, lg, top_k, None, True, bf16=True)
    oi, ow = orc.moe_route(lb, top_k)
    assert np.array_equal(ids, oi) and (np.abs(w - ow) <= 4e-6 * np.abs(ow) + 1e-9).all()


def test_route_nan_scores_rank_last_and_errors(ctx):
    import aq_mi355
    say("moe route nan/err")
    lg = np.array([[np.nan, 1.0, np.nan, 0.5, 2.0]], np.float32)
    ids, w, _ = _route(ctx, lg, 3)
    assert ids.tolist() == [[4, 1, 3]] and np.isfinite(w).all() and abs(w.sum() - 1) < 1e-6
    buf = ctx.alloc(4096)
    for kw, code in [(dict(E=0), aq_mi355.AQ_ERR_SHAPE), (dict(k=0), aq_mi355.AQ_ERR_SHAPE), (dict(k=9), aq_mi355.AQ_ERR_SHAPE),
                     (dict(E=2000, k=2), aq_mi355.AQ_ERR_UNSUPPORTED), (dict(E=128, k=65), aq_mi355.AQ_ERR_UNSUPPORTED),
                     (dict(rows=-1), aq_mi355.AQ_ERR_SHAPE)]:
        with pytest.raises(aq_mi355.AqError) as e:
            ctx.moe_route(buf, kw.get("rows", 1), kw.get("E", 8), kw.get("k", 2), buf, buf)
        assert e.value.code == code, kw
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.moe_route(None, 1, 8, 2, buf, buf)
    assert e.value.code == aq_mi355.AQ_ERR_ARG
    ctx.moe_route(None, 0, 8, 2, None, None)   # no rows: nothing to do
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.moe_combine(buf, buf, buf, 1, 0, 8)
    assert e.value.code == aq_mi355.AQ_ERR_SHAPE
    ctx.moe_combine(None, None, None, 0, 2, 8)
    buf.free()


@pytest.mark.parametrize("rows,top_k,n", [(8, 8, 2816), (1, 1, 7), (3, 2, 33), (64, 4, 1000)])
def test_combine_against_oracle(ctx, orc, rows, top_k, n):
    import aq_mi355
    say("moe combine", rows, top_k, n)
    rng = np.random.default_rng(rows + n)
    y = rng.normal(0, 1, (rows * top_k, n)).astype(np.float32)
    w = rng.uniform(0, 1, rows * top_k).astype(np.float32)
    yb = F.f32_to_bf16_bits(y)
    ybf = F.bf16_bits_to_f32(yb).reshape(rows * top_k, n)
    dw = ctx.to_device(w)
    d32, d16 = ctx.to_device(y), ctx.to_device(yb)
    o32, o16 = ctx.alloc(rows * n * 4), ctx.alloc(rows * n * 2)
    # fp32 in, fp32 out: bit-exact (fp32 multiply, then fp32 adds in rank order)
    ctx.moe_combine(d32, dw, o32, rows, top_k, n, aq_mi355.AQ_IN_F32 | aq_mi355.AQ_OUT_F32)
    ctx.sync()
    assert np.array_equal(o32.download(np.float32, rows * n).reshape(rows, n), orc.moe_combine(y, w, rows, top_k, n))
    # bf16 in, bf16 out: the RNE of the same fp32 sums
    ctx.moe_combine(d16, dw, o16, rows, top_k, n, 0)
    ctx.sync()
    want = orc.moe_combine(ybf, w, rows, top_k, n)
    assert np.array_equal(o16.download(np.uint16, rows * n).reshape(rows, n), F.f32_to_bf16_bits(want).reshape(rows, n))
    # bf16 at every step
    ctx.moe_combine(d16, dw, o16, rows, top_k, n, aq_mi355.AQ_BF16_STEPS)
    ctx.sync()
    want = orc.moe_combine(ybf, w, rows, top_k, n, bf16_steps=True)
    assert np.array_equal(o16.download(np.uint16, rows * n).reshape(rows, n), F.f32_to_bf16_bits(want).reshape(rows, n))
    for t in (dw, d32, d16, o32, o16):
        t.free()


def _gelu64(v):
    return 0.5 * v * (1 + np.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))


def test_routed_expert_block_stays_on_device(ctx, orc):
    """cfg 4 geometry at a reduced expert count: scores -> aq_moe_route -> aq_gather_qmv_gate_up (GELU) ->
    aq_gather_qmv (down) -> aq_moe_combine, captured into one graph; against a float64 chain on the oracle's
    routing, with the intermediate roundings the device path makes (bf16 h, bf16 route rows)."""
    import aq_mi355
    say("moe block on device")
    E, tokens, top_k, DM, DFF, gs, bits = 16, 8, 4, 1024, 512, 64, 4
    routes = tokens * top_k
    rng = np.random.default_rng(F.BASE_SEED + 95)
    logits = rng.normal(0, 1.5, (tokens, E)).astype(np.float32)
    scales = rng.uniform(0.8, 1.2, E).astype(np.float32)
    gu = F.synthetic_affine(E * 2 * DFF, DM, bits, gs, seed=F.BASE_SEED + 96)
    dn = F.synthetic_affine(E * DM, DFF, bits, gs, seed=F.BASE_SEED + 97)
    x = F.f32_to_bf16_bits(rng.normal(0, 0.3, (tokens, DM)).astype(np.float32))
    dgu, ddn = DeviceAffine(ctx, *gu), DeviceAffine(ctx, *dn)
    dx, dl, ds = ctx.to_device(x), ctx.to_device(logits), ctx.to_device(scales)
    d_ids, d_w, d_tok = ctx.alloc(routes * 4), ctx.alloc(routes * 4), ctx.alloc(routes * 4)
    d_iota = ctx.to_device(np.arange(routes, dtype=np.int32))
    dh, dy, dout = ctx.alloc(routes * DFF * 2), ctx.alloc(routes * DM * 2), ctx.alloc(tokens * DM * 4)

    def block():
        ctx.moe_route(dl, tokens, E, top_k, d_ids, d_w, d_tok, ds, True)
        ctx.gather_qmv_gate_up(dx, dgu.w, dgu.s, dgu.b, d_tok, d_ids, dh, routes, tokens, DM, DFF, E, 2 * DFF, 0, DFF, gs, bits,
                               aq_mi355.AQ_ACT_GELU_TANH)
        ctx.gather_qmv(dh, ddn.w, ddn.s, ddn.b, d_iota, d_ids, dy, routes, routes, DFF, DM, E, DM, 0, gs, bits)
        ctx.moe_combine(dy, d_w, dout, tokens, top_k, DM, aq_mi355.AQ_OUT_F32)

    block()
    ctx.sync()
    eager = dout.download(np.float32, tokens * DM).reshape(tokens, DM).copy()
    ids = d_ids.download(np.int32, routes).reshape(tokens, top_k)
    oi, ow = orc.moe_route(logits, top_k, scales)
    assert np.array_equal(ids, oi)
    # float64 chain with the device path's storage roundings
    wgu = F.numpy_dequant(gu[0], gu[1], gu[2], bits, gs, DM).astype(np.float64).reshape(E, 2 * DFF, DM)
    wdn = F.numpy_dequant(dn[0], dn[1], dn[2], bits, gs, DFF).astype(np.float64).reshape(E, DM, DFF)
    xf = F.bf16_bits_to_f32(x).astype(np.float64).reshape(tokens, DM)
    ref = np.zeros((tokens, DM))
    for t in range(tokens):
        for r in range(top_k):
            e = oi[t, r]
            h = _gelu64(wgu[e, :DFF] @ xf[t]) * (wgu[e, DFF:] @ xf[t])
            h = F.bf16_bits_to_f32(F.f32_to_bf16_bits(h.astype(np.float32))).astype(np.float64)
            y = wdn[e] @ h
            y = F.bf16_bits_to_f32(F.f32_to_bf16_bits(y.astype(np.float32))).astype(np.float64)
            ref[t] += y * float(ow[t, r])
    err = np.abs(eager - ref)
    # bf16 storage of h and of the route rows dominates: a relative 2^-8 of each, through |w_down| sums
    assert err.max() <= 4 * MAX_ABS + 2.0 ** -7 * np.abs(ref).max(), err.max()
    assert np.linalg.norm(eager - ref) / np.linalg.norm(ref) <= 1e-2
    ctx.capture_begin()
    block()
    graph = ctx.capture_end()
    for i in range(3):
        ctx.fill_zero(dout)
        ctx.graph_launch(graph)
        ctx.sync()
        assert np.array_equal(dout.download(np.float32, tokens * DM).reshape(tokens, DM), eager), i
    ctx.graph_destroy(graph)
    for t in (dx, dl, ds, d_ids, d_w, d_tok, d_iota, dh, dy, dout):
        t.free()
    dgu.free()
    ddn.free()
