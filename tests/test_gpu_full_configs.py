"""The benchmark configurations at their stated sizes, through the launch forms the bench times.

cfg 4: 128 experts (gate|up slab: 507 MB of codes), 8 tokens x top-8.
cfg 1: the multi-matrix launches q|k|v and gate|up = 2 x 14336 rows.
Checked against the oracle library itself (fp32-accumulated reference, gather) and a float64 chain.
"""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, MAX_ABS, check_accumulators, check_bf16_store, run_qmv, say

pytestmark = pytest.mark.gpu


def _gelu64(v):
    return 0.5 * v * (1 + np.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))


def _expert_f64(t, e, rows, K):
    """float64 weights of expert e of a stacked affine tensor t = (words, scales, biases) with `rows` rows per expert."""
    sl = slice(e * rows, (e + 1) * rows)
    return F.numpy_dequant(t[0][sl], t[1][sl], t[2][sl], 4, 64, K).astype(np.float64)


def test_cfg4_at_128_experts(ctx, orc):
    """gather_qmv, the fused gate|up gather and the whole routed block with E = 128, in-projection slab
    [128, 2 x 1408, 2816] and down slab [128, 2816, 1408]; the routes include experts 0, 64 and 127 (the
    sweep of go/engine/metal/qmv_gather_test.go:87-129 and the slice identity of moe_quant_test.go:1143-1185
    at the size BASELINE's cfg 4 states)."""
    import aq_mi355
    E, tokens, top_k, DM, DFF, gs, bits = 128, 8, 8, 2816, 1408, 64, 4
    routes = tokens * top_k
    rng = np.random.default_rng(F.BASE_SEED + 404)
    say("cfg4 E=128: building slabs")
    gu = F.synthetic_affine(E * 2 * DFF, DM, bits, gs, seed=F.BASE_SEED + 405)
    dn = F.synthetic_affine(E * DM, DFF, bits, gs, seed=F.BASE_SEED + 406)
    assert gu[0].nbytes == E * 2 * DFF * DM // 2   # 507 MB of codes in one slab
    ids = np.stack([rng.permutation(E)[:top_k] for _ in range(tokens)]).astype(np.int32)
    # the first expert, one in the upper half of the slab, and the last
    for t, pos, e in ((0, 0, 0), (3, 5, 64), (7, 7, 127)):
        dup = np.nonzero(ids[t] == e)[0]
        if len(dup):
            ids[t, dup[0]] = ids[t, pos]
        ids[t, pos] = e
    assert all(len(set(ids[t])) == top_k for t in range(tokens))
    flat = ids.reshape(-1).copy()
    assert (flat >= 64).sum() >= 16
    tok_of = np.repeat(np.arange(tokens), top_k).astype(np.int32)
    iota = np.arange(routes, dtype=np.int32)
    x = F.synthetic_x(tokens, DM, seed=F.BASE_SEED + 407)
    xf = F.bf16_bits_to_f32(x).astype(np.float64).reshape(tokens, DM)

    dgu, ddn = DeviceAffine(ctx, *gu), DeviceAffine(ctx, *dn)
    dx, d_ids, d_tok, d_iota = ctx.to_device(x), ctx.to_device(flat), ctx.to_device(tok_of), ctx.to_device(iota)

    # ---- float64 references per route (one dequantised expert at a time) ----
    g_ref, u_ref = np.zeros((routes, DFF)), np.zeros((routes, DFF))
    for e in np.unique(flat):
        w = _expert_f64(gu, e, 2 * DFF, DM)
        for z in np.nonzero(flat == e)[0]:
            g_ref[z] = w[:DFF] @ xf[tok_of[z]]
            u_ref[z] = w[DFF:] @ xf[tok_of[z]]

    # ---- aq_gather_qmv on the gate half and on the up half (row bases inside the fused slab) ----
    say("cfg4 E=128: gather gate / up")
    acc = {}
    for name, base, ref in (("gate", 0, g_ref), ("up", DFF, u_ref)):
        dy = ctx.alloc(routes * DFF * 4)
        ctx.fill_zero(dy)
        ctx.gather_qmv(dx, dgu.w, dgu.s, dgu.b, d_tok, d_ids, dy, routes, tokens, DM, DFF, E, 2 * DFF, base, gs, bits,
                       aq_mi355.AQ_OUT_F32)
        ctx.sync()
        acc[name] = dy.download(np.float32, routes * DFF).reshape(routes, DFF)
        check_accumulators(acc[name], ref, "cfg4 gather " + name)
        dy.free()
    assert ctx.last_variant(0).startswith("qmvd_"), ctx.last_variant(0)
    # a subset of routes against the oracle library, incl. the routes on experts 0, 64 and 127
    sub = np.array([0, 3 * top_k + 5, 7 * top_k + 7, 9, 30, 50])
    for name, base in (("gate", 0), ("up", DFF)):
        r64, _ = orc.gather_qmv(x, tokens, gu[0], gu[1], gu[2], tok_of[sub], flat[sub], len(sub), E, 2 * DFF, base, DFF, DM, gs, bits)
        check_accumulators(acc[name][sub], r64, "cfg4 gather %s vs oracle" % name)
    # bf16 store; byte identity with aq_qmv on the sliced expert (experts 0, 64, 127)
    dyb = ctx.alloc(routes * DFF * 2)
    ctx.gather_qmv(dx, dgu.w, dgu.s, dgu.b, d_tok, d_ids, dyb, routes, tokens, DM, DFF, E, 2 * DFF, DFF, gs, bits)
    ctx.sync()
    up_bits = dyb.download(np.uint16, routes * DFF).reshape(routes, DFF)
    assert np.array_equal(up_bits, F.f32_to_bf16_bits(acc["up"]).reshape(routes, DFF))
    for z in (0, 3 * top_k + 5, 7 * top_k + 7):
        e = flat[z]
        sl = slice(e * 2 * DFF + DFF, (e + 1) * 2 * DFF)
        one = DeviceAffine(ctx, gu[0][sl], gu[1][sl], gu[2][sl])
        yb = run_qmv(ctx, x[tok_of[z]:tok_of[z] + 1], one, 1, DM, DFF, gs, bits, False)
        assert np.array_equal(yb[0], up_bits[z]), ("slice identity", z, e)
        one.free()
    dyb.free()

    # ---- fused gate|up gather (GELU-tanh) ----
    say("cfg4 E=128: fused gate|up gather")
    dh32 = ctx.alloc(routes * DFF * 4)
    ctx.gather_qmv_gate_up(dx, dgu.w, dgu.s, dgu.b, d_tok, d_ids, dh32, routes, tokens, DM, DFF, E, 2 * DFF, 0, DFF, gs, bits,
                           aq_mi355.AQ_ACT_GELU_TANH, aq_mi355.AQ_OUT_F32)
    ctx.sync()
    assert ctx.last_variant(0) == "gather_gate_up_diag", ctx.last_variant(0)
    h32 = dh32.download(np.float32, routes * DFF).reshape(routes, DFF)
    h_ref = _gelu64(g_ref) * u_ref
    # the matvec bounds carried through act(g) * u: |d(act(g) u)| <= |u| 1.13 dg + |act(g)| du
    bound = MAX_ABS * (1.13 * np.abs(u_ref) + np.abs(_gelu64(g_ref))) + 1e-5
    assert (np.abs(h32 - h_ref) <= bound).all(), float((np.abs(h32 - h_ref) - bound).max())
    want = orc.act_multiply(aq_mi355.AQ_ACT_GELU_TANH, acc["gate"].reshape(-1), acc["up"].reshape(-1)).reshape(routes, DFF)
    assert np.abs(h32 - want).max() <= 1e-5 * max(1.0, np.abs(want).max())
    dh32.free()

    # ---- the routed block: router -> fused gather -> down gather -> combine ----
    say("cfg4 E=128: routed block")
    logits = rng.normal(0, 1.5, (tokens, E)).astype(np.float32)
    logits[0, 0] += 20.0      # make sure the first, a middle and the last expert are routed to
    logits[3, 64] += 20.0
    logits[7, 127] += 20.0
    dl = ctx.to_device(logits)
    r_ids, r_w, r_tok = ctx.alloc(routes * 4), ctx.alloc(routes * 4), ctx.alloc(routes * 4)
    dh, dy, dout = ctx.alloc(routes * DFF * 2), ctx.alloc(routes * DM * 2), ctx.alloc(tokens * DM * 4)
    ctx.moe_route(dl, tokens, E, top_k, r_ids, r_w, r_tok, None, True)
    ctx.gather_qmv_gate_up(dx, dgu.w, dgu.s, dgu.b, r_tok, r_ids, dh, routes, tokens, DM, DFF, E, 2 * DFF, 0, DFF, gs, bits,
                           aq_mi355.AQ_ACT_GELU_TANH)
    ctx.gather_qmv(dh, ddn.w, ddn.s, ddn.b, d_iota, r_ids, dy, routes, routes, DFF, DM, E, DM, 0, gs, bits)
    ctx.moe_combine(dy, r_w, dout, tokens, top_k, DM, aq_mi355.AQ_OUT_F32)
    ctx.sync()
    got = dout.download(np.float32, tokens * DM).reshape(tokens, DM)
    oi, ow = orc.moe_route(logits, top_k, None)
    assert np.array_equal(r_ids.download(np.int32, routes).reshape(tokens, top_k), oi)
    assert oi[0, 0] == 0 and oi[3, 0] == 64 and oi[7, 0] == 127
    # the down gather alone against the oracle library on the device's own h (three routes)
    h_dev = dh.download(np.uint16, routes * DFF)
    y_dev = F.bf16_bits_to_f32(dy.download(np.uint16, routes * DM)).reshape(routes, DM)
    subz = np.array([0, 3 * top_k, 7 * top_k])
    r64, _ = orc.gather_qmv(h_dev, routes, dn[0], dn[1], dn[2], iota[subz], oi.reshape(-1)[subz], len(subz), E, DM, 0, DM, DFF, gs, bits)
    for i, z in enumerate(subz):
        check_bf16_store(F.f32_to_bf16_bits(y_dev[z]), r64[i], "cfg4 down route %d vs oracle" % z)
    ref = np.zeros((tokens, DM))
    for e in np.unique(oi):
        wg = _expert_f64(gu, e, 2 * DFF, DM)
        wd = _expert_f64(dn, e, DM, DFF)
        for t, r in zip(*np.nonzero(oi == e)):
            h = _gelu64(wg[:DFF] @ xf[t]) * (wg[DFF:] @ xf[t])
            h = F.bf16_bits_to_f32(F.f32_to_bf16_bits(h.astype(np.float32))).astype(np.float64)
            y = wd @ h
            y = F.bf16_bits_to_f32(F.f32_to_bf16_bits(y.astype(np.float32))).astype(np.float64)
            ref[t] += y * float(ow[t, r])
    err = np.abs(got - ref)
    assert err.max() <= 4 * MAX_ABS + 2.0 ** -7 * np.abs(ref).max(), err.max()
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) <= 1e-2
    for t in (dx, d_ids, d_tok, d_iota, dl, r_ids, r_w, r_tok, dh, dy, dout):
        t.free()
    dgu.free()
    ddn.free()


# the third form crosses the size from which a launch loads its weights with the non-temporal hint (16 MB of codes):
# the launch of both matrices is above it, the single calls it is compared with are below
@pytest.mark.parametrize("name,Ns", [("q|k|v", (4096, 1024, 1024)), ("gate|up", (14336, 14336)), ("q|o", (4096, 4200))])
def test_cfg1_multi_launch_forms(ctx, orc, name, Ns):
    """The launches the cfg 1 bench times: aq_qmv_multi over q|k|v and over gate|up = 2 x 14336 rows at K = 4096.
    Byte-identical to one aq_qmv per matrix (ConcatQuantRows' contract, go/model/quant_weight.go:32-44), and every
    member within the stated bounds of the oracle's fp32-accumulated reference (hip_projection_reference.go:92-116)."""
    import aq_mi355
    say("cfg1 multi", name)
    K = 4096
    x = F.synthetic_x(1, K, seed=F.BASE_SEED + 1)
    xf = F.bf16_bits_to_f32(x[0])
    dx = ctx.to_device(x)
    mats = [F.synthetic_affine(n, K, 4, 64, seed=F.BASE_SEED + 500 + 7 * i + n) for i, n in enumerate(Ns)]
    dws = [DeviceAffine(ctx, *m) for m in mats]
    for f32 in (True, False):
        esz = 4 if f32 else 2
        ys = [ctx.alloc(n * esz) for n in Ns]
        for t in ys:
            ctx.fill_zero(t)
        ctx.qmv_multi(dx, [d.w for d in dws], [d.s for d in dws], [d.b for d in dws], ys, list(Ns), 1, K, 64, 4,
                      aq_mi355.AQ_OUT_F32 if f32 else 0)
        ctx.sync()
        assert ctx.last_variant(0) == "qmv_multi_diag", ctx.last_variant(0)
        for i, n in enumerate(Ns):
            got = ys[i].download(np.float32 if f32 else np.uint16, n).reshape(1, n)
            want = run_qmv(ctx, x, dws[i], 1, K, n, 64, 4, f32)
            assert np.array_equal(got.view(np.uint32 if f32 else np.uint16), want.view(np.uint32 if f32 else np.uint16)), (name, i, f32)
            ref32 = orc.hip_reference_projection(xf, mats[i][0], mats[i][1], mats[i][2], n, K, 64, 4)
            if f32:
                check_accumulators(got, ref32, "cfg1 %s member %d vs oracle" % (name, i))
                check_accumulators(got, F.reference_f64(x, *mats[i], 4, 64, K), "cfg1 %s member %d vs f64" % (name, i))
            else:
                check_bf16_store(got, ref32, "cfg1 %s member %d bf16" % (name, i))
        for t in ys:
            t.free()
    dx.free()
    for d in dws:
        d.free()
