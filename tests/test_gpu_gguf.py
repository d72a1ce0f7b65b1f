"""GGUF blocks -> affine tensors on the device (aq_gguf_to_affine) against the CPU oracle, bit for bit, and the
repacked tensors through the projection kernels against ggml's own dequantisation of the same blocks."""
import numpy as np
import pytest

import fixtures as F
import gguf_blocks as G
from gpu_util import DeviceAffine, check_accumulators, run_qmv, say

pytestmark = pytest.mark.gpu

TYPES = [G.F32, G.Q4_0, G.Q4_1, G.Q8_0, G.Q4_K, G.Q5_K, G.Q6_K]


def _repack(ctx, gguf_type, rows, cols, data, offset=0):
    """Device repack of host bytes `data`; offset shifts the device copy of the blocks off its alignment."""
    import aq_mi355
    lay = aq_mi355.gguf_affine_layout(gguf_type, rows, cols)
    src = ctx.alloc(data.nbytes + 16)
    ctx._check(ctx.lib.aq_h2d(ctx.handle, src.ptr + offset, data.ctypes.data, data.nbytes))
    w, s, b = ctx.alloc(lay.packed_bytes), ctx.alloc(lay.scales_bytes), ctx.alloc(lay.scales_bytes)
    for t in (w, s, b):                      # stale contents must not survive
        t.upload(np.full(t.nbytes, 0xA5, np.uint8))
    ctx.gguf_to_affine(gguf_type, src.ptr + offset, data.nbytes, rows, cols, w, s, b)
    ctx.sync()
    out = (w.download(np.uint32).reshape(rows, lay.packed_cols), s.download(np.uint16).reshape(rows, lay.groups),
           b.download(np.uint16).reshape(rows, lay.groups))
    for t in (src, w, s, b):
        t.free()
    return out, lay


@pytest.mark.parametrize("gguf_type", TYPES)
@pytest.mark.parametrize("rows,blocks,offset", [(1, 1, 0), (3, 5, 0), (37, 9, 0), (64, 16, 2), (5, 3, 1), (700, 4, 0)])
def test_repack_matches_oracle_bit_for_bit(ctx, orc, gguf_type, rows, blocks, offset):
    cols = blocks * G.BLOCK[gguf_type][0]
    if gguf_type == G.F32 and offset % 4:
        offset = 4
    say("gguf repack", G.NAMES[gguf_type], rows, cols, offset)
    data = G.random_blocks(gguf_type, rows, cols, seed=F.BASE_SEED + 300 + gguf_type + rows)
    (w, s, b), lay = _repack(ctx, gguf_type, rows, cols, data, offset)
    ow, os_, ob = orc.gguf_to_affine(gguf_type, rows, cols, data)
    assert (lay.bits, lay.group_size) == G.AFFINE[gguf_type]
    assert np.array_equal(w, ow), "codes"
    assert np.array_equal(s, os_), "scales"
    assert np.array_equal(b, ob), "biases"


@pytest.mark.parametrize("gguf_type,rows,cols", [(G.Q4_0, 512, 2048), (G.Q4_1, 300, 1536), (G.Q8_0, 256, 1024),
                                                 (G.Q4_K, 512, 2048), (G.Q5_K, 200, 768), (G.Q6_K, 384, 1024),
                                                 (G.F32, 128, 512)])
def test_projection_over_repacked_tensor(ctx, gguf_type, rows, cols):
    """blocks -> device repack -> aq_qmv, against x @ W^T with W dequantised by ggml's rules (bf16-exact block scales,
    so the affine triple stands for exactly those weights; F32 input: against the quantiser's own dequantisation,
    which sits within half a step of the source)."""
    say("gguf projection", G.NAMES[gguf_type], rows, cols)
    import aq_mi355
    data = G.random_blocks(gguf_type, rows, cols, seed=F.BASE_SEED + 330 + gguf_type, exact=True)
    lay = aq_mi355.gguf_affine_layout(gguf_type, rows, cols)
    src = ctx.to_device(data)
    w, s, b = ctx.alloc(lay.packed_bytes), ctx.alloc(lay.scales_bytes), ctx.alloc(lay.scales_bytes)
    ctx.gguf_to_affine(gguf_type, src, data.nbytes, rows, cols, w, s, b)
    hw = w.download(np.uint32).reshape(rows, -1)
    hs, hb = s.download(np.uint16).reshape(rows, -1), b.download(np.uint16).reshape(rows, -1)
    dq = G.affine_dequant(hw, hs, hb, cols, lay.bits, lay.group_size)
    if gguf_type == G.F32:
        clean = data.view(np.float32).reshape(rows, cols).astype(np.float64)
        clean[~np.isfinite(clean)] = 0
        step = np.repeat(G.bf16_to_f64(hs), 32, axis=1)
        lo = np.repeat(G.bf16_to_f64(hb), 32, axis=1)
        # half a step, plus the bf16 rounding of the step (over up to 255 steps) and of the group minimum
        assert np.all(np.abs(dq - clean) <= step * (0.5 + 255 * 2.0 ** -8) + np.abs(lo) * 2.0 ** -8 + 1e-6)
        weights = dq
    else:
        weights = G.ggml_dequant(gguf_type, rows, cols, data)
        assert np.array_equal(dq, weights)
    norm = max(1.0, np.abs(weights).max())                       # keeps the sums in the range the bounds are stated for
    dev = DeviceAffine.__new__(DeviceAffine)
    dev.w, dev.s, dev.b = w, s, b
    for M in (1, 3):
        x = F.synthetic_x(M, cols, seed=F.BASE_SEED + 340 + M)
        ref = F.bf16_bits_to_f32(x).astype(np.float64).reshape(M, cols) @ weights.T
        got = run_qmv(ctx, x, dev, M, cols, rows, lay.group_size, lay.bits, True).astype(np.float64)
        check_accumulators(got / norm, ref / norm, G.NAMES[gguf_type])
    for t in (src, w, s, b):
        t.free()


def test_repack_captured_and_errors(ctx, orc):
    import aq_mi355
    say("gguf capture + errors")
    rows, cols = 16, 1024
    data = G.random_blocks(G.Q4_K, rows, cols, seed=F.BASE_SEED + 350)
    lay = aq_mi355.gguf_affine_layout(G.Q4_K, rows, cols)
    src = ctx.to_device(data)
    w, s, b = ctx.alloc(lay.packed_bytes), ctx.alloc(lay.scales_bytes), ctx.alloc(lay.scales_bytes)
    ctx.capture_begin()
    ctx.gguf_to_affine(G.Q4_K, src, data.nbytes, rows, cols, w, s, b)
    graph = ctx.capture_end()
    ow, os_, ob = orc.gguf_to_affine(G.Q4_K, rows, cols, data)
    for i in range(2):
        for t in (w, s, b):
            ctx.fill_zero(t)
        ctx.graph_launch(graph)
        ctx.sync()
        assert np.array_equal(w.download(np.uint32).reshape(rows, -1), ow), i
        assert np.array_equal(s.download(np.uint16).reshape(rows, -1), os_), i
        assert np.array_equal(b.download(np.uint16).reshape(rows, -1), ob), i
    ctx.graph_destroy(graph)
    n = data.nbytes
    for call, code in [(lambda: ctx.gguf_to_affine(G.Q4_K, src, n - 1, rows, cols, w, s, b), aq_mi355.AQ_ERR_SHAPE),
                       (lambda: ctx.gguf_to_affine(G.Q4_K, src, n, rows, cols + 32, w, s, b), aq_mi355.AQ_ERR_SHAPE),
                       (lambda: ctx.gguf_to_affine(G.Q4_K, src, n, 0, cols, w, s, b), aq_mi355.AQ_ERR_SHAPE),
                       (lambda: ctx.gguf_to_affine(7, src, n, rows, cols, w, s, b), aq_mi355.AQ_ERR_UNSUPPORTED),
                       (lambda: ctx.gguf_to_affine(G.Q4_K, None, n, rows, cols, w, s, b), aq_mi355.AQ_ERR_ARG),
                       (lambda: ctx.gguf_to_affine(G.Q4_K, src, n, rows, cols, w.ptr + 4, s, b), aq_mi355.AQ_ERR_ARG),
                       (lambda: ctx.gguf_to_affine(G.Q4_K, src, n, rows, cols, w, s.ptr + 1, b), aq_mi355.AQ_ERR_ARG)]:
        with pytest.raises(aq_mi355.AqError) as e:
            call()
        assert e.value.code == code
    for t in (src, w, s, b):
        t.free()


@pytest.mark.parametrize("gguf_type", [G.Q4_K, G.Q6_K])
def test_repack_full_size_projection_tensor(ctx, orc, gguf_type):
    """The gate projection's shape (14336 x 4096), bit for bit against the oracle."""
    rows, cols = 14336, 4096
    say("gguf repack full size", G.NAMES[gguf_type], rows, cols)
    data = G.random_blocks(gguf_type, rows, cols, seed=F.BASE_SEED + 360 + gguf_type)
    (w, s, b), _ = _repack(ctx, gguf_type, rows, cols, data)
    ow, os_, ob = orc.gguf_to_affine(gguf_type, rows, cols, data)
    assert np.array_equal(w, ow) and np.array_equal(s, os_) and np.array_equal(b, ob)


def test_gguf_lm_head_to_greedy_token(ctx, orc):
    """A Q4_0 vocabulary projection as a GGUF file ships it -> device repack -> aq_qmv_greedy (group 32: the
    diagonal-MFMA head kernel) -> the token ggml's dequantisation of the same blocks makes the winner."""
    import aq_mi355
    rows, cols = 32768, 1536
    say("gguf lm_head greedy", rows, cols)
    data = G.random_blocks(G.Q4_0, rows, cols, seed=F.BASE_SEED + 370, exact=True)
    lay = aq_mi355.gguf_affine_layout(G.Q4_0, rows, cols)
    src = ctx.to_device(data)
    w, s, b = ctx.alloc(lay.packed_bytes), ctx.alloc(lay.scales_bytes), ctx.alloc(lay.scales_bytes)
    ctx.gguf_to_affine(G.Q4_0, src, data.nbytes, rows, cols, w, s, b)
    x = F.synthetic_x(1, cols, seed=F.BASE_SEED + 371)
    dx, best, scores = ctx.to_device(x), ctx.alloc(8), ctx.alloc(rows * 8)
    ctx.qmv_greedy(dx, w, s, b, best, 1, cols, rows, lay.group_size, lay.bits)
    assert ctx.last_variant(0) == "qmv_greedy_diag"
    ctx.qmv_scores(dx, w, s, b, scores, 1, cols, rows, lay.group_size, lay.bits)
    ctx.sync()
    packed = scores.download(np.uint64, rows)
    got = int(best.download(np.uint64, 1)[0])
    assert got == int(packed.max())
    tok, score = aq_mi355.unpack_best(got)
    ref = F.bf16_bits_to_f32(x).astype(np.float64).reshape(cols) @ G.ggml_dequant(G.Q4_0, rows, cols, data).T
    norm = np.abs(ref).max()
    assert abs(score - ref[tok]) <= 2e-3 * norm and ref[tok] >= ref.max() - 4e-3 * norm
    for t in (src, w, s, b, dx, best, scores):
        t.free()


@pytest.mark.parametrize("gguf_type", [G.Q4_K, G.Q6_K, G.Q8_0])
def test_gguf_expert_stack_to_gather(ctx, orc, gguf_type):
    """A stacked expert tensor [E, rows, cols] of GGUF blocks (as *_exps.weight ships) -> one repack over E * rows rows
    -> aq_gather_qmv with the expert ids on the device, against ggml's dequantisation of the chosen experts' rows."""
    import aq_mi355
    E, rows, cols, routes, x_rows = 6, 96, 1024, 9, 3
    say("gguf experts gather", G.NAMES[gguf_type], E, rows, cols)
    data = G.random_blocks(gguf_type, E * rows, cols, seed=F.BASE_SEED + 380 + gguf_type, exact=True)
    lay = aq_mi355.gguf_affine_layout(gguf_type, E * rows, cols)
    src = ctx.to_device(data)
    w, s, b = ctx.alloc(lay.packed_bytes), ctx.alloc(lay.scales_bytes), ctx.alloc(lay.scales_bytes)
    ctx.gguf_to_affine(gguf_type, src, data.nbytes, E * rows, cols, w, s, b)
    rng = np.random.default_rng(9)
    rhs = rng.integers(0, E, routes).astype(np.int32)
    lhs = rng.integers(0, x_rows, routes).astype(np.int32)
    x = F.synthetic_x(x_rows, cols, seed=F.BASE_SEED + 381)
    dx, dl, dr = ctx.to_device(x), ctx.to_device(lhs), ctx.to_device(rhs)
    out_dim, row_base = 64, 32
    dy = ctx.alloc(routes * out_dim * 4)
    ctx.gather_qmv(dx, w, s, b, dl, dr, dy, routes, x_rows, cols, out_dim, E, rows, row_base, lay.group_size, lay.bits,
                   aq_mi355.AQ_OUT_F32)
    ctx.sync()
    got = dy.download(np.float32, routes * out_dim).reshape(routes, out_dim).astype(np.float64)
    weights = G.ggml_dequant(gguf_type, E * rows, cols, data).reshape(E, rows, cols)
    xf = F.bf16_bits_to_f32(x).astype(np.float64).reshape(x_rows, cols)
    ref = np.stack([weights[rhs[z], row_base:row_base + out_dim] @ xf[lhs[z]] for z in range(routes)])
    norm = max(1.0, np.abs(weights).max())
    check_accumulators(got / norm, ref / norm, G.NAMES[gguf_type])
    # and against the oracle's gather over the oracle's repack of the same blocks
    ow, os_, ob = orc.gguf_to_affine(gguf_type, E * rows, cols, data)
    ref64, _ = orc.gather_qmv(x, x_rows, ow, os_, ob, lhs, rhs, routes, E, rows, row_base, out_dim, cols, lay.group_size, lay.bits)
    check_accumulators(got / norm, np.asarray(ref64, np.float64).reshape(routes, out_dim) / norm, G.NAMES[gguf_type] + " oracle")
    for t in (src, w, s, b, dx, dl, dr, dy):
        t.free()
