"""The tile-major device layout (aq_tile_weights / aq_untile_weights / AQ_W_TILED): the layout against an independent
numpy statement of it, the exact inverse, and every call that takes the flag against the same call on the MLX arrays,
byte for byte (same kernels, same order of additions); one full-size case against the float64 reference."""
import numpy as np
import pytest

import aq_mi355
import fixtures as F
from gpu_util import DeviceAffine, check_accumulators, say

pytestmark = pytest.mark.gpu

T = aq_mi355.AQ_W_TILED
F32 = aq_mi355.AQ_OUT_F32

# N ragged against the 16-row sets; K: one short step, whole steps, three-chunk steps (2816), a last chunk of one half
# (3200 = 25 halves), the long K of the down projection, the longest K the one-row kernels take, K beyond them
SHAPES = [(16, 1152), (40, 2048), (33, 2816), (64, 3200), (100, 4096), (48, 14336), (256, 1408), (17, 16384), (50, 1152),
          (20, 128), (35, 17408)]


def _tiled(ctx, N, K, seed):
    w, s, b = F.synthetic_affine(N, K, 4, 64, seed=seed)
    d = DeviceAffine(ctx, w, s, b)
    t = ctx.tile_weights(d.w, d.s, d.b, N, K)
    return (w, s, b), d, t


@pytest.mark.parametrize("N,K", SHAPES)
def test_layout_matches_numpy_and_inverts(ctx, N, K):
    say("tile layout", N, K)
    (w, s, b), d, t = _tiled(ctx, N, K, N + K)
    ctx.sync()
    got = t.download(np.uint8)
    ref = F.tile_major(w, s, b, N, K)
    assert got.size == ref.size == aq_mi355.tiled_bytes(N, K)
    assert (got == ref).all()
    w2, s2, b2 = ctx.alloc(w.nbytes), ctx.alloc(s.nbytes), ctx.alloc(b.nbytes)
    for z in (w2, s2, b2):
        ctx.fill_zero(z)
    ctx.untile_weights(t, N, K, w2, s2, b2)
    ctx.sync()
    assert (w2.download(np.uint32) == w.reshape(-1)).all()
    assert (s2.download(np.uint16) == s.reshape(-1)).all()
    assert (b2.download(np.uint16) == b.reshape(-1)).all()


@pytest.mark.parametrize("N,K", SHAPES)
def test_qmv_bytes_equal_the_mlx_layout(ctx, N, K):
    """One to eight rows run on the diagonal-MFMA kernels straight from the tiles (where those take K); more rows, and
    K they do not take, rebuild the MLX arrays in the workspace: either way the same bytes."""
    (w, s, b), d, t = _tiled(ctx, N, K, 3 * N + K)
    for M in (1, 2, 3, 4, 5, 8, 9, 16, 33):
        say("tiled qmv", N, K, M)
        x = ctx.to_device(F.synthetic_x(M, K, seed=3 + M))
        for flags in (F32, 0):
            y0, y1 = ctx.alloc(M * N * 4), ctx.alloc(M * N * 4)
            ctx.fill_zero(y0)
            ctx.fill_zero(y1)
            ctx.qmv(x, d.w, d.s, d.b, y0, M, K, N, 64, 4, flags)
            v0 = ctx.last_variant(0)
            ctx.qmv(x, t, None, None, y1, M, K, N, 64, 4, flags | T)
            v1 = ctx.last_variant(0)
            ctx.sync()
            assert v0 == v1
            assert (y0.download(np.uint32) == y1.download(np.uint32)).all(), (v0, M, flags)
        if M == 1 and 1024 < K <= 16384:
            assert v1.startswith("qmvd_"), v1


def test_headline_shape_against_the_reference(ctx):
    """cfg 1's gate projection at full size from the tiles: accumulators against float64, bytes against the MLX layout."""
    N, K = 14336, 4096
    (w, s, b), d, t = _tiled(ctx, N, K, 11)
    x_bits = F.synthetic_x(1, K, seed=12)
    x = ctx.to_device(x_bits)
    y0, y1 = ctx.alloc(N * 4), ctx.alloc(N * 4)
    ctx.qmv(x, d.w, d.s, d.b, y0, 1, K, N, 64, 4, F32)
    ctx.qmv(x, t, None, None, y1, 1, K, N, 64, 4, F32 | T)
    ctx.sync()
    a0, a1 = y0.download(np.float32), y1.download(np.float32)
    assert (a0.view(np.uint32) == a1.view(np.uint32)).all()
    check_accumulators(a1, F.reference_f64(x_bits, w, s, b, 4, 64, K), "tiled " + ctx.last_variant(0))


def test_multi_and_gate_up_bytes_equal_the_mlx_layout(ctx):
    K = 2048
    Ns = [48, 16, 80]
    mats = [_tiled(ctx, n, K, 40 + n) for n in Ns]
    for M in (1, 3, 4, 6):
        say("tiled multi", M)
        x = ctx.to_device(F.synthetic_x(M, K, seed=60 + M))
        ys0 = [ctx.alloc(M * n * 4) for n in Ns]
        ys1 = [ctx.alloc(M * n * 4) for n in Ns]
        ctx.qmv_multi(x, [m[1].w for m in mats], [m[1].s for m in mats], [m[1].b for m in mats], ys0, Ns, M, K, 64, 4, F32)
        ctx.qmv_multi(x, [m[2] for m in mats], [None] * 3, [None] * 3, ys1, Ns, M, K, 64, 4, F32 | T)
        ctx.sync()
        for a, b_ in zip(ys0, ys1):
            assert (a.download(np.uint32) == b_.download(np.uint32)).all(), M
    N = 48
    gate, up = _tiled(ctx, N, K, 71), _tiled(ctx, N, K, 72)
    for act in (aq_mi355.AQ_ACT_GELU_TANH, aq_mi355.AQ_ACT_SILU):
        for M in (1, 2, 4, 5):  # (five rows: no fused kernel, the unfused route through the workspace)
            say("tiled gate_up", act, M)
            x = ctx.to_device(F.synthetic_x(M, K, seed=80 + M))
            y0, y1 = ctx.alloc(M * N * 4), ctx.alloc(M * N * 4)
            ctx.qmv_gate_up(x, (gate[1].w, gate[1].s, gate[1].b), (up[1].w, up[1].s, up[1].b), y0, M, K, N, 64, 4, act, F32)
            ctx.qmv_gate_up(x, (gate[2], None, None), (up[2], None, None), y1, M, K, N, 64, 4, act, F32 | T)
            ctx.sync()
            assert (y0.download(np.uint32) == y1.download(np.uint32)).all(), (act, M)


def test_fused_slab_tiles_as_one(ctx):
    """A row-concatenated gate|up slab (model.ConcatQuantRows, go/model/quant_weight.go:45-63) tiled as ONE tensor: the
    up half starts at a whole set of rows, so its tiles are a pointer offset into the tiled slab."""
    N, K = 64, 2048
    w, s, b = F.synthetic_affine(2 * N, K, 4, 64, seed=91)
    d = DeviceAffine(ctx, w, s, b)
    t = ctx.tile_weights(d.w, d.s, d.b, 2 * N, K)
    up_off = aq_mi355.tiled_bytes(N, K)
    assert 2 * up_off == aq_mi355.tiled_bytes(2 * N, K)
    x = ctx.to_device(F.synthetic_x(1, K, seed=92))
    y0, y1 = ctx.alloc(N * 4), ctx.alloc(N * 4)
    row_w, row_s = K // 2, K // 64 * 2
    ctx.qmv_gate_up(x, (d.w, d.s, d.b), (d.w.ptr + N * row_w, d.s.ptr + N * row_s, d.b.ptr + N * row_s), y0, 1, K, N, 64, 4,
                    aq_mi355.AQ_ACT_GELU_TANH, F32)
    ctx.qmv_gate_up(x, (t, None, None), (t.ptr + up_off, None, None), y1, 1, K, N, 64, 4, aq_mi355.AQ_ACT_GELU_TANH, F32 | T)
    ctx.sync()
    assert (y0.download(np.uint32) == y1.download(np.uint32)).all()


def test_captured_and_replayed(ctx):
    N, K = 96, 4096
    (w, s, b), d, t = _tiled(ctx, N, K, 5)
    x = ctx.to_device(F.synthetic_x(2, K, seed=6))
    y0, y1 = ctx.alloc(2 * N * 2), ctx.alloc(2 * N * 2)
    ctx.qmv(x, d.w, d.s, d.b, y0, 2, K, N, 64, 4, 0)
    ctx.sync()
    ctx.capture_begin()
    ctx.qmv(x, t, None, None, y1, 2, K, N, 64, 4, T)
    g = ctx.capture_end()
    for _ in range(3):
        ctx.fill_zero(y1)
        ctx.graph_launch(g)
        ctx.sync()
        assert (y0.download(np.uint16) == y1.download(np.uint16)).all()
    ctx.graph_destroy(g)


def test_geometries_without_a_tile_major_form(ctx):
    assert aq_mi355.tiled_bytes(64, 4096, 64, 8) == -1
    assert aq_mi355.tiled_bytes(64, 4096, 32, 4) == -1
    assert aq_mi355.tiled_bytes(64, 4096 + 64, 64, 4) == -1
    assert aq_mi355.tiled_bytes(0, 4096, 64, 4) == -1
    assert aq_mi355.tiled_bytes(14336, 4096) == 33030144  # as many bytes as the three MLX arrays
    assert aq_mi355.tiled_bytes(17, 4096) == 2 * 36864     # rows padded to whole sets of 16
    buf = ctx.alloc(1 << 16)
    for (K, gs, bits) in ((4096, 64, 8), (4096, 32, 4), (4096 + 64, 64, 4)):
        with pytest.raises(aq_mi355.AqError) as e:
            ctx.qmv(buf, buf, None, None, buf, 1, K, 2, gs, bits, T)
        assert e.value.code == aq_mi355.AQ_ERR_UNSUPPORTED
        rc = ctx.lib.aq_tile_weights(ctx.handle, buf.ptr, buf.ptr, buf.ptr, 2, K, gs, bits, buf.ptr)
        assert rc == aq_mi355.AQ_ERR_UNSUPPORTED
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.qmv(buf, buf.ptr + 4, None, None, buf, 1, 2048, 2, 64, 4, T)  # a tile-major tensor is 16-byte aligned
    assert e.value.code == aq_mi355.AQ_ERR_ARG
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.qmv(buf, buf, None, None, buf, 1, 2048, 2, 64, 4, 0)          # without the flag scales and biases are needed
    assert e.value.code == aq_mi355.AQ_ERR_ARG
