"""GPU parity of the activation-fused MLP entry points (gate|up with GELU-tanh / SiLU epilogue, plain and
expert-gathered; projections that form their gated input while staging it; the stand-alone act_mul),
called through the C ABI and checked against the CPU oracle.

Bars: a fused gate|up output equals act(g) * u for the fp32 sums g, u that the unfused aq_qmv /
aq_gather_qmv produce (same streaming order, so the same sums) to fp32 rounding of the activation, and sits
within the stated matvec tolerance of the float64 reference propagated through the activation; the x-load
fused projections are byte-identical to aq_act_mul followed by the plain projection."""
import contextlib

import numpy as np
import pytest

import fixtures as F
from gpu_util import MAX_ABS, REL, DeviceAffine, check_accumulators, run_qmv, say

pytestmark = pytest.mark.gpu

ACTS = [1, 2]


def _act64(act, v):
    v = np.asarray(v, dtype=np.float64)
    if act == 1:
        return 0.5 * v * (1 + np.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))
    return v / (1 + np.exp(-v))


def _check_fused(got, g_gpu, u_gpu, g64, u64, act, orc, what):
    """got: fused fp32 output; g_gpu/u_gpu: the unfused device sums; g64/u64: float64 reference sums."""
    want = orc.act_multiply(act, g_gpu, u_gpu)
    # fp32 rounding of the activation; for negative gates 1 + tanh cancels in fp32 (the reference's own
    # formula, math.hipinc:3-9), an absolute error of about an fp32 ulp of 1 times |g * u| / 2
    tight = np.abs(got.astype(np.float64) - want) <= 4e-6 * np.abs(want) + 2.5e-7 * np.maximum(1.0, np.abs(g_gpu * u_gpu))
    assert tight.all(), "%s: fused epilogue differs from act(g)*u of the unfused sums by %.3e" % (
        what, np.abs(got - want).max())
    # against the float64 reference: the matvec bounds on g and u, carried through act (|act'| <= 1.13)
    ref = _act64(act, g64) * u64
    bound = MAX_ABS * (1.13 * np.abs(u64) + np.abs(_act64(act, g64)) + MAX_ABS) + REL * np.abs(ref)
    assert (np.abs(got - ref) <= bound).all(), what
    denom = np.linalg.norm(ref)
    if denom > 0:
        assert np.linalg.norm(got - ref) / denom <= REL, what


class _dot2_family:
    """Pins the unfused calls to the dot2 kernel family the fused kernels are built from, so that both
    sides add up in the same order."""

    def __init__(self, ctx, bits, gather):
        import aq_mi355
        self.ctx = ctx
        name = "qmv_b%d_m1_r1_w4_d2_g%d_x0" % (bits, 1 if gather else 0)
        self.idx = aq_mi355.variant_names(aq_mi355.OP_QMV).index(name)

    def __enter__(self):
        self.ctx.force_variant(0, self.idx)

    def __exit__(self, *exc):
        self.ctx.force_variant(0, -1)


def _run_gate_up(ctx, x, dg, du, M, K, N, gs, bits, act, f32=True):
    import aq_mi355
    dx = ctx.to_device(np.ascontiguousarray(x, dtype=np.uint16))
    dy = ctx.alloc(M * N * (4 if f32 else 2))
    ctx.fill_zero(dy)
    ctx.qmv_gate_up(dx, (dg.w, dg.s, dg.b), (du.w, du.s, du.b), dy, M, K, N, gs, bits, act,
                    aq_mi355.AQ_OUT_F32 if f32 else 0)
    ctx.sync()
    out = dy.download(np.float32 if f32 else np.uint16, M * N).reshape(M, N)
    dx.free()
    dy.free()
    return out


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("bits,gs,M,K,N", [(4, 64, 1, 4096, 14336), (4, 64, 1, 2048, 1001), (4, 64, 1, 2816, 1408),
                                           (8, 64, 1, 2560, 640), (4, 32, 1, 512, 40), (4, 128, 1, 1024, 7),
                                           (8, 32, 1, 256, 3), (4, 64, 1, 14336, 256), (4, 64, 3, 4096, 203),
                                           (4, 64, 4, 3072, 48), (4, 64, 1, 8192, 130), (4, 64, 2, 2048, 77)])
def test_gate_up_single_row(ctx, orc, act, bits, gs, M, K, N):
    say("gate_up", act, bits, gs, M, K, N)
    gw, gsb, gb = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 70)
    uw, usb, ub = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 71)
    x = F.synthetic_x(M, K, seed=F.BASE_SEED + 72)
    dg, du = DeviceAffine(ctx, gw, gsb, gb), DeviceAffine(ctx, uw, usb, ub)
    got = _run_gate_up(ctx, x, dg, du, M, K, N, gs, bits, act)
    # 4-bit group-64 codes with K a multiple of 256 in 2..8 steps of 1024: the diagonal-MFMA pair kernel (up to 4 rows), whose two sums
    # are those of the library's own choice for a plain call; otherwise the dot2 pair kernel (one row)
    diag = bits == 4 and gs == 64 and K % 256 == 0 and 2 <= (K + 1023) // 1024 <= 8
    assert ctx.last_variant(0) == ("qmv_gate_up_diag" if diag else "qmv_gate_up_dot2")
    if diag:
        g_gpu = run_qmv(ctx, x, dg, M, K, N, gs, bits, True)
        assert ctx.last_variant(0).startswith("qmvd_")
        u_gpu = run_qmv(ctx, x, du, M, K, N, gs, bits, True)
    else:
        with _dot2_family(ctx, bits, False):
            g_gpu = run_qmv(ctx, x, dg, M, K, N, gs, bits, True)
            u_gpu = run_qmv(ctx, x, du, M, K, N, gs, bits, True)
    _check_fused(got, g_gpu, u_gpu, F.reference_f64(x, gw, gsb, gb, bits, gs, K), F.reference_f64(x, uw, usb, ub, bits, gs, K),
                 act, orc, "gate_up")
    out = _run_gate_up(ctx, x, dg, du, M, K, N, gs, bits, act, f32=False)
    assert np.array_equal(out, F.f32_to_bf16_bits(got).reshape(M, N))  # the store is the RNE of the same value
    dg.free()
    du.free()


def test_gate_up_row_concatenated_slab(ctx, orc):
    """One [2N, K] gate|up tensor (model.ConcatQuantRows): up = slab + N rows."""
    say("gate_up slab")
    K, N, gs, bits = 1024, 96, 64, 4
    w, s, b = F.synthetic_affine(2 * N, K, bits, gs, seed=F.BASE_SEED + 73)
    x = F.synthetic_x(1, K, seed=F.BASE_SEED + 74)
    slab = DeviceAffine(ctx, w, s, b)
    wpr, gpr = K * bits // 32, K // gs

    class View:
        pass
    up = View()
    up.w, up.s, up.b = slab.w.ptr + N * wpr * 4, slab.s.ptr + N * gpr * 2, slab.b.ptr + N * gpr * 2
    got = _run_gate_up(ctx, x, slab, up, 1, K, N, gs, bits, 1)
    both = run_qmv(ctx, x, slab, 1, K, 2 * N, gs, bits, True)
    want = orc.act_multiply(1, both[:, :N], both[:, N:])
    assert (np.abs(got - want) <= 4e-6 * np.abs(want) + 2.5e-7 * np.maximum(1.0, np.abs(both[:, :N] * both[:, N:]))).all()
    slab.free()


@pytest.mark.parametrize("gs", [32, 64])
def test_gate_up_reference_hardware_fixture(ctx, orc, gs):
    """go/engine/hip/hip_hardware_test.go:2318-2407: device result within 0.03 of the CPU expectation.  The
    fixture's x is fp32 with bf16-exact values ((c%23-11)/128), so the bf16 boundary loses nothing."""
    say("gate_up hw fixture", gs)
    fx = F.hw_fixture_q4_gelu_cols2560(gs)
    xb = F.f32_to_bf16_bits(fx["x"])
    assert np.array_equal(F.bf16_bits_to_f32(xb), fx["x"])
    proj = lambda m: orc.hip_reference_projection(fx["x"], m["packed"], m["scales"], m["biases"], fx["rows"], fx["cols"], gs, 4)
    want = orc.act_multiply(orc.ACT_GELU_TANH, proj(fx["gate"]), proj(fx["up"]))
    dg = DeviceAffine(ctx, fx["gate"]["packed"], fx["gate"]["scales"], fx["gate"]["biases"])
    du = DeviceAffine(ctx, fx["up"]["packed"], fx["up"]["scales"], fx["up"]["biases"])
    got = _run_gate_up(ctx, xb.reshape(1, -1), dg, du, 1, fx["cols"], fx["rows"], gs, 4, 1).reshape(-1)
    assert np.abs(got - want).max() <= fx["tol"]
    assert np.abs(got - want).max() <= 1e-5
    dg.free()
    du.free()


@pytest.mark.parametrize("bits,gs,M,K,N", [(6, 32, 1, 192, 11), (4, 64, 3, 512, 64), (4, 64, 20, 1024, 130),
                                           (4, 64, 70, 512, 96), (3, 64, 2, 256, 9)])
def test_gate_up_unfused_shapes(ctx, orc, bits, gs, M, K, N):
    """Widths, groups and row counts the one-launch kernels do not take run as two projections and an
    element-wise step; same contract."""
    say("gate_up unfused", bits, gs, M, K, N)
    rng = np.random.default_rng(bits * 100 + M)
    mk = lambda: (F.pack_codes(rng.integers(0, 1 << bits, size=(N, K)), bits),
                  F.f32_to_bf16_bits((np.abs(rng.normal(0, 0.02, (N, K // gs))) + 1e-3).astype(np.float32)),
                  F.f32_to_bf16_bits(rng.normal(0, 0.05, (N, K // gs)).astype(np.float32)))
    (gw, gsb, gb), (uw, usb, ub) = mk(), mk()
    x = F.synthetic_x(M, K, seed=F.BASE_SEED + 75)
    dg, du = DeviceAffine(ctx, gw, gsb, gb), DeviceAffine(ctx, uw, usb, ub)
    got = _run_gate_up(ctx, x, dg, du, M, K, N, gs, bits, 1)
    g_gpu = run_qmv(ctx, x, dg, M, K, N, gs, bits, True)
    u_gpu = run_qmv(ctx, x, du, M, K, N, gs, bits, True)
    _check_fused(got, g_gpu, u_gpu, F.reference_f64(x, gw, gsb, gb, bits, gs, K), F.reference_f64(x, uw, usb, ub, bits, gs, K),
                 1, orc, "gate_up unfused")
    out = _run_gate_up(ctx, x, dg, du, M, K, N, gs, bits, 1, f32=False)
    assert np.array_equal(out, F.f32_to_bf16_bits(got).reshape(M, N))
    dg.free()
    du.free()


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("bits,gs,M,K,N", [(4, 64, 256, 4096, 520), (4, 64, 2048, 2048, 1024), (8, 64, 100, 1024, 203),
                                           (4, 64, 40, 1024, 300), (4, 128, 64, 512, 96), (4, 64, 33, 320, 77)])
def test_gate_up_prefill_rows(ctx, orc, act, bits, gs, M, K, N):
    """More than 32 rows (rocm_mlx_q4_gelu_tanh_multiply_batch, affine_gelu_tanh.hipinc:921-1109): the `up` projection
    runs on the matmul tiles and their stores apply act(gate) * up, over every tile family (fp16-operand tiles, bf16-code
    tiles, few-rows kernels with their K-split sum) and ragged N.  Checked against the device's own two projections."""
    say("gate_up prefill", act, bits, gs, M, K, N)
    gw, gsb, gb = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 170)
    uw, usb, ub = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 171)
    x = F.synthetic_x(M, K, seed=F.BASE_SEED + 172)
    dg, du = DeviceAffine(ctx, gw, gsb, gb), DeviceAffine(ctx, uw, usb, ub)
    got = _run_gate_up(ctx, x, dg, du, M, K, N, gs, bits, act)
    assert ctx.last_variant(0) == "qmv_gate_up_tiles"
    g_gpu = run_qmv(ctx, x, dg, M, K, N, gs, bits, True)
    u_gpu = run_qmv(ctx, x, du, M, K, N, gs, bits, True)
    _check_fused(got, g_gpu, u_gpu, F.reference_f64(x, gw, gsb, gb, bits, gs, K), F.reference_f64(x, uw, usb, ub, bits, gs, K),
                 act, orc, "gate_up prefill")
    out = _run_gate_up(ctx, x, dg, du, M, K, N, gs, bits, act, f32=False)
    assert np.array_equal(out, F.f32_to_bf16_bits(got).reshape(M, N))
    dg.free()
    du.free()


def _gather_inputs(ctx, E, expert_rows, K, bits, gs, x_rows, lhs, rhs, seed):
    words, s, b = F.synthetic_affine(E * expert_rows, K, bits, gs, seed=seed)
    x = F.synthetic_x(x_rows, K, seed=seed + 1)
    dev = dict(w=DeviceAffine(ctx, words, s, b), x=ctx.to_device(x), rhs=ctx.to_device(np.asarray(rhs, np.int32)),
               lhs=None if lhs is None else ctx.to_device(np.asarray(lhs, np.int32)))
    return words, s, b, x, dev


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("bits,K,N,batched", [(4, 2816, 1408, True), (4, 512, 40, False), (8, 1024, 64, True),
                                              (4, 1408, 70, True), (4, 4096, 40, False)])
def test_gather_gate_up_fused_slab(ctx, orc, act, bits, K, N, batched):
    """Experts hold a fused gate|up slab of 2N rows; expert ids and token rows are read on the device."""
    import aq_mi355
    say("gather gate_up", act, bits, K, N, batched)
    E, tokens, topk, gs = 6, 4, 3, 64
    routes = tokens * topk
    rng = np.random.default_rng(F.BASE_SEED + 76)
    rhs = np.concatenate([rng.permutation(E)[:topk] for _ in range(tokens)]).astype(np.int32)
    lhs = np.repeat(np.arange(tokens), topk).astype(np.int32) if batched else None
    x_rows = tokens if batched else 1
    words, s, b, x, dev = _gather_inputs(ctx, E, 2 * N, K, bits, gs, x_rows, lhs, rhs, F.BASE_SEED + 77)
    dw = dev["w"]
    dy = ctx.alloc(routes * N * 4)
    ctx.fill_zero(dy)
    ctx.gather_qmv_gate_up(dev["x"], dw.w, dw.s, dw.b, dev["lhs"], dev["rhs"], dy, routes, x_rows, K, N, E, 2 * N, 0, N, gs,
                           bits, act, aq_mi355.AQ_OUT_F32)
    ctx.sync()
    # 4-bit codes with K a multiple of 128 in 2..8 steps of 1024: the gathered diagonal-MFMA pair kernel, whose sums
    # are those of the library's own choice for a plain gather; otherwise the dot2 pair kernel
    diag = bits == 4 and K % 128 == 0 and 2 <= (K + 1023) // 1024 <= 8
    assert ctx.last_variant(0) == ("gather_gate_up_diag" if diag else "gather_gate_up_dot2")
    got = dy.download(np.float32, routes * N).reshape(routes, N)
    parts = []
    import contextlib
    with (contextlib.nullcontext() if diag else _dot2_family(ctx, bits, True)):
        for base in (0, N):
            ctx.fill_zero(dy)
            ctx.gather_qmv(dev["x"], dw.w, dw.s, dw.b, dev["lhs"], dev["rhs"], dy, routes, x_rows, K, N, E, 2 * N, base, gs,
                           bits, aq_mi355.AQ_OUT_F32)
            ctx.sync()
            assert ctx.last_variant(0).startswith("qmvd_") == diag
            parts.append(dy.download(np.float32, routes * N).reshape(routes, N))
    wq = F.numpy_dequant(words, s, b, bits, gs, K).astype(np.float64).reshape(E, 2 * N, K)
    xf = F.bf16_bits_to_f32(x).astype(np.float64).reshape(x_rows, K)
    xr = lambda z: xf[lhs[z]] if batched else xf[0]
    g64 = np.stack([wq[rhs[z], :N] @ xr(z) for z in range(routes)])
    u64 = np.stack([wq[rhs[z], N:] @ xr(z) for z in range(routes)])
    _check_fused(got, parts[0], parts[1], g64, u64, act, orc, "gather gate_up")
    # the oracle's own gather, a few routes
    sub = [0, routes // 2, routes - 1]
    og, _ = orc.gather_qmv(x, x_rows, words, s, b, None if lhs is None else lhs[sub], rhs[sub], len(sub), E, 2 * N, 0, N, K, gs, bits)
    ou, _ = orc.gather_qmv(x, x_rows, words, s, b, None if lhs is None else lhs[sub], rhs[sub], len(sub), E, 2 * N, N, N, K, gs, bits)
    check_accumulators(parts[0][sub], og, "gate sums vs oracle gather")
    check_accumulators(parts[1][sub], ou, "up sums vs oracle gather")
    for t in (dy, dev["x"], dev["rhs"], dev["lhs"]):
        if t is not None:
            t.free()
    dw.free()


@pytest.mark.parametrize("K", [512, 1408])
def test_gather_gate_up_bad_ids_and_errors(ctx, K):
    import aq_mi355
    say("gather gate_up bad ids", K)
    E, N = 4, 32
    words, s, b, x, dev = _gather_inputs(ctx, E, 2 * N, K, 4, 64, 1, None, [1, 9, -2], F.BASE_SEED + 78)
    dw = dev["w"]
    dy = ctx.alloc(3 * N * 4)
    ctx.gather_qmv_gate_up(dev["x"], dw.w, dw.s, dw.b, None, dev["rhs"], dy, 3, 1, K, N, E, 2 * N, 0, N, 64, 4, 1,
                           aq_mi355.AQ_OUT_F32)
    ctx.sync()
    out = dy.download(np.float32, 3 * N).reshape(3, N)
    assert np.all(out[1] == 0) and np.all(out[2] == 0) and np.any(out[0] != 0)
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.gather_qmv_gate_up(dev["x"], dw.w, dw.s, dw.b, None, dev["rhs"], dy, 3, 1, K, N, E, 2 * N, 0, N + 1, 64, 4, 1)
    assert e.value.code == aq_mi355.AQ_ERR_SHAPE
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.gather_qmv_gate_up(dev["x"], dw.w, dw.s, dw.b, None, dev["rhs"], dy, 3, 1, K, N, E, 2 * N, 0, N, 64, 4, 7)
    assert e.value.code == aq_mi355.AQ_ERR_UNSUPPORTED
    ctx.gather_qmv_gate_up(dev["x"], dw.w, dw.s, dw.b, None, dev["rhs"], dy, 0, 1, K, N, E, 2 * N, 0, N, 64, 4, 1)  # no routes
    for t in (dy, dev["x"], dev["rhs"]):
        t.free()
    dw.free()


@pytest.mark.parametrize("act", ACTS)
def test_act_mul_vs_oracle(ctx, orc, act):
    say("act_mul", act)
    rng = np.random.default_rng(F.BASE_SEED + 79 + act)
    for n in (1, 7, 4096, 100003):
        g = F.f32_to_bf16_bits(rng.normal(0, 2, n).astype(np.float32))
        u = F.f32_to_bf16_bits(rng.normal(0, 1.5, n).astype(np.float32))
        dg, du, dy = ctx.to_device(g), ctx.to_device(u), ctx.alloc(n * 2)
        ctx.act_mul(dg, du, dy, n, act)
        ctx.sync()
        got = dy.download(np.uint16, n)
        want = orc.act_gate_mul_bf16(act, g, u)
        key = lambda v: np.where(v.astype(np.int32) & 0x8000, -(v.astype(np.int32) & 0x7FFF), v.astype(np.int32) & 0x7FFF)
        d = np.abs(key(got) - key(want))
        absd = np.abs(F.bf16_bits_to_f32(got).astype(np.float64) - F.bf16_bits_to_f32(want).astype(np.float64))
        # the device tanh/exp and libm may differ in the last fp32 place: a bf16 rounding boundary may flip
        assert ((d <= 1) | (absd <= 1e-6)).all(), n
        assert np.mean(d == 0) > 0.98 or n < 100
        for t in (dg, du, dy):
            t.free()


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("bits,gs,M,K,N", [(4, 64, 1, 14336, 4096), (4, 64, 1, 1408, 2816), (8, 64, 1, 1024, 100),
                                           (4, 32, 1, 256, 9), (4, 64, 3, 512, 64), (6, 32, 1, 192, 11)])
def test_qmv_act_equals_act_mul_then_qmv(ctx, orc, act, bits, gs, M, K, N):
    """The down projection that gates its own input: byte-identical to the two-step chain, and within the
    matvec tolerance of the float64 reference on the oracle's gated input."""
    import aq_mi355
    say("qmv_act", act, bits, gs, M, K, N)
    rng = np.random.default_rng(F.BASE_SEED + 80)
    if 32 % bits == 0:
        words, s, b = F.synthetic_affine(N, K, bits, gs, seed=F.BASE_SEED + 81)
    else:
        words = F.pack_codes(rng.integers(0, 1 << bits, size=(N, K)), bits)
        s = F.f32_to_bf16_bits((np.abs(rng.normal(0, 0.02, (N, K // gs))) + 1e-3).astype(np.float32))
        b = F.f32_to_bf16_bits(rng.normal(0, 0.05, (N, K // gs)).astype(np.float32))
    g = F.f32_to_bf16_bits(rng.normal(0, 1.5, (M, K)).astype(np.float32))
    u = F.f32_to_bf16_bits(rng.normal(0, 1.0, (M, K)).astype(np.float32))
    dw = DeviceAffine(ctx, words, s, b)
    dg, du = ctx.to_device(g), ctx.to_device(u)
    dy = ctx.alloc(M * N * 4)
    ctx.fill_zero(dy)
    ctx.qmv_act(dg, du, dw.w, dw.s, dw.b, dy, M, K, N, gs, bits, act, aq_mi355.AQ_OUT_F32)
    ctx.sync()
    fused = dy.download(np.float32, M * N).reshape(M, N)
    if M == 1 and bits in (4, 8):
        assert ctx.last_variant(0) == "qmv_act_dot2"
    dgated = ctx.alloc(M * K * 2)
    ctx.act_mul(dg, du, dgated, M * K, act)
    ctx.fill_zero(dy)
    with (_dot2_family(ctx, bits, False) if M == 1 and bits in (4, 8) else contextlib.nullcontext()):
        ctx.qmv(dgated, dw.w, dw.s, dw.b, dy, M, K, N, gs, bits, aq_mi355.AQ_OUT_F32)
    ctx.sync()
    chain = dy.download(np.float32, M * N).reshape(M, N)
    assert np.array_equal(fused.view(np.uint32), chain.view(np.uint32))
    gated_dev = dgated.download(np.uint16, M * K).reshape(M, K)
    ref_dev = F.reference_f64(gated_dev, words, s, b, bits, gs, K)
    check_accumulators(fused, ref_dev, "qmv_act vs float64 on the device's gated input")
    # against the oracle's gated input: the few inputs whose bf16 rounding differs move the sums a little
    gated_orc = orc.act_gate_mul_bf16(act, g, u)
    assert np.mean(gated_orc == gated_dev) > 0.98
    ref = F.reference_f64(gated_orc, words, s, b, bits, gs, K)
    assert np.abs(fused - ref).max() <= MAX_ABS
    for t in (dg, du, dy, dgated):
        t.free()
    dw.free()


@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("bits,K,N", [(4, 1408, 2816), (8, 512, 48), (6, 192, 11)])
def test_gather_qmv_act_equals_chain(ctx, orc, act, bits, K, N):
    """lthn_gather_qmv_gelu: the routed down projection with gate/up rows indexed by lhs."""
    import aq_mi355
    say("gather_qmv_act", act, bits, K, N)
    E, routes, gs = 5, 12, 64 if bits != 6 else 32
    rng = np.random.default_rng(F.BASE_SEED + 82)
    rhs = rng.integers(0, E, routes).astype(np.int32)
    lhs = rng.permutation(routes).astype(np.int32)
    if 32 % bits == 0:
        words, s, b = F.synthetic_affine(E * N, K, bits, gs, seed=F.BASE_SEED + 83)
    else:
        words = F.pack_codes(rng.integers(0, 1 << bits, size=(E * N, K)), bits)
        s = F.f32_to_bf16_bits((np.abs(rng.normal(0, 0.02, (E * N, K // gs))) + 1e-3).astype(np.float32))
        b = F.f32_to_bf16_bits(rng.normal(0, 0.05, (E * N, K // gs)).astype(np.float32))
    g = F.f32_to_bf16_bits(rng.normal(0, 1.5, (routes, K)).astype(np.float32))
    u = F.f32_to_bf16_bits(rng.normal(0, 1.0, (routes, K)).astype(np.float32))
    dw = DeviceAffine(ctx, words, s, b)
    dg, du, dl, dr = ctx.to_device(g), ctx.to_device(u), ctx.to_device(lhs), ctx.to_device(rhs)
    dy = ctx.alloc(routes * N * 4)
    ctx.fill_zero(dy)
    ctx.gather_qmv_act(dg, du, dw.w, dw.s, dw.b, dl, dr, dy, routes, routes, K, N, E, N, 0, gs, bits, act, aq_mi355.AQ_OUT_F32)
    ctx.sync()
    fused = dy.download(np.float32, routes * N).reshape(routes, N)
    if bits in (4, 8):
        assert ctx.last_variant(0) == "gather_act_dot2"
    dgated = ctx.alloc(routes * K * 2)
    ctx.act_mul(dg, du, dgated, routes * K, act)
    ctx.fill_zero(dy)
    with (_dot2_family(ctx, bits, True) if bits in (4, 8) else contextlib.nullcontext()):
        ctx.gather_qmv(dgated, dw.w, dw.s, dw.b, dl, dr, dy, routes, routes, K, N, E, N, 0, gs, bits, aq_mi355.AQ_OUT_F32)
    ctx.sync()
    chain = dy.download(np.float32, routes * N).reshape(routes, N)
    assert np.array_equal(fused.view(np.uint32), chain.view(np.uint32))
    gated_dev = dgated.download(np.uint16, routes * K).reshape(routes, K)
    wq = F.numpy_dequant(words, s, b, bits, gs, K).astype(np.float64).reshape(E, N, K)
    xf = F.bf16_bits_to_f32(gated_dev).astype(np.float64)
    ref = np.stack([wq[rhs[z]] @ xf[lhs[z]] for z in range(routes)])
    check_accumulators(fused, ref, "gather_qmv_act")
    for t in (dg, du, dl, dr, dy, dgated):
        t.free()
    dw.free()


def test_fused_act_zero_sizes_and_errors(ctx):
    import aq_mi355
    say("fused act zero/err")
    buf = ctx.alloc(1 << 16)
    trip = (buf, buf, buf)
    ctx.qmv_gate_up(None, (None,) * 3, (None,) * 3, None, 1, 64, 0, 64, 4, 1)   # N == 0
    ctx.qmv_gate_up(None, (None,) * 3, (None,) * 3, None, 0, 64, 8, 64, 4, 1)   # M == 0
    ctx.qmv_act(None, None, None, None, None, None, 1, 0, 8, 64, 4, 1)           # K == 0
    ctx.act_mul(None, None, None, 0, 1)
    for call, code in [
        (lambda: ctx.qmv_gate_up(buf, trip, trip, buf, 1, 64, 4, 64, 4, 0), aq_mi355.AQ_ERR_UNSUPPORTED),
        (lambda: ctx.qmv_gate_up(buf, trip, trip, buf, 1, 64, 4, 3, 4, 1), aq_mi355.AQ_ERR_SHAPE),
        (lambda: ctx.qmv_gate_up(buf, trip, trip, buf, 1, 64, 4, 64, 9, 1), aq_mi355.AQ_ERR_UNSUPPORTED),
        (lambda: ctx.qmv_gate_up(buf, trip, (None, buf, buf), buf, 1, 64, 4, 64, 4, 1), aq_mi355.AQ_ERR_ARG),
        (lambda: ctx.qmv_gate_up(buf, trip, trip, buf, 1, 0, 4, 64, 4, 1), aq_mi355.AQ_ERR_SHAPE),
        (lambda: ctx.qmv_act(buf, None, buf, buf, buf, buf, 1, 64, 4, 64, 4, 1), aq_mi355.AQ_ERR_ARG),
        (lambda: ctx.qmv_act(buf, buf, buf, buf, buf, buf, 1, 64, 4, 64, 4, 3), aq_mi355.AQ_ERR_UNSUPPORTED),
        (lambda: ctx.act_mul(buf, buf, buf, -1, 1), aq_mi355.AQ_ERR_SHAPE),
        (lambda: ctx.act_mul(buf, buf, buf, 8, 0), aq_mi355.AQ_ERR_UNSUPPORTED),
        (lambda: ctx.gather_qmv_act(buf, buf, buf, buf, buf, None, buf, buf, 3, 1, 64, 8, 4, 8, 4, 64, 4, 1), aq_mi355.AQ_ERR_SHAPE),
    ]:
        with pytest.raises(aq_mi355.AqError) as e:
            call()
        assert e.value.code == code
    buf.free()


def test_fused_mlp_block_in_a_graph(ctx, orc):
    """gate|up fused launch + gated down projection captured once and replayed: every replay equals the
    eager result (no workspace growth, no memset nodes)."""
    import aq_mi355
    say("fused mlp graph")
    K, F_, gs, bits = 1024, 2816, 64, 4
    gw, gsb, gb = F.synthetic_affine(F_, K, bits, gs, seed=F.BASE_SEED + 90)
    uw, usb, ub = F.synthetic_affine(F_, K, bits, gs, seed=F.BASE_SEED + 91)
    dwn, ds, db = F.synthetic_affine(K, F_, bits, gs, seed=F.BASE_SEED + 92)
    dg, du, dd = DeviceAffine(ctx, gw, gsb, gb), DeviceAffine(ctx, uw, usb, ub), DeviceAffine(ctx, dwn, ds, db)
    x = F.synthetic_x(1, K, seed=F.BASE_SEED + 93)
    dx, dh, dy = ctx.to_device(x), ctx.alloc(F_ * 2), ctx.alloc(K * 4)

    def step():
        ctx.qmv_gate_up(dx, (dg.w, dg.s, dg.b), (du.w, du.s, du.b), dh, 1, K, F_, gs, bits, 1, 0)
        ctx.qmv(dh, dd.w, dd.s, dd.b, dy, 1, F_, K, gs, bits, aq_mi355.AQ_OUT_F32)
    step()
    ctx.sync()
    eager = dy.download(np.float32, K).copy()
    h = F.bf16_bits_to_f32(dh.download(np.uint16, F_)).astype(np.float64)
    g64 = F.reference_f64(x, gw, gsb, gb, bits, gs, K).reshape(-1)
    u64 = F.reference_f64(x, uw, usb, ub, bits, gs, K).reshape(-1)
    hr = _act64(1, g64) * u64
    assert (np.abs(h - hr) <= 2e-2 + 2.0 ** -8 * np.abs(hr)).all()   # the matvec bound plus one bf16 rounding
    ctx.capture_begin()
    step()
    graph = ctx.capture_end()
    for i in range(3):
        ctx.fill_zero(dy)
        ctx.graph_launch(graph)
        ctx.sync()
        assert np.array_equal(dy.download(np.float32, K), eager), i
    ctx.graph_destroy(graph)
    for t in (dx, dh, dy):
        t.free()
    for t in (dg, du, dd):
        t.free()
