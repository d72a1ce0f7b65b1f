"""GPU: a checkpoint file -> the library's loader -> device slabs -> the kernels, against the oracle on the
bytes that were written into the file."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import check_accumulators, say
from test_loader import affine_entry, write_safetensors

pytestmark = pytest.mark.gpu


def _download(ctx, ptr, nbytes):
    out = np.zeros(nbytes, np.uint8)
    ctx._check(ctx.lib.aq_d2h(ctx.handle, out.ctypes.data, ptr, nbytes))
    return out


def test_loaded_linear_runs_on_the_device(ctx, orc, tmp_path):
    import aq_mi355
    say("loader -> qmv")
    cases = {"q": (64, 512, 4, 64), "k": (24, 256, 8, 64), "v": (16, 192, 6, 32)}
    tensors, want = {}, {}
    for name, (N, K, bits, gs) in cases.items():
        t, w = affine_entry(name, N, K, bits, gs, seed=30 + len(tensors))
        tensors.update(t)
        want[name] = w
    path = str(tmp_path / "m.safetensors")
    write_safetensors(path, tensors)
    f = aq_mi355.SafetensorsFile(path)
    for name, (N, K, bits, gs) in cases.items():
        lin = f.load_linear(name, K)
        dev = ctx.upload_linear(lin)
        assert (dev.rows, dev.in_dim, dev.group_size, dev.bits, dev.experts) == (N, K, gs, bits, 0)
        w, s, b = want[name]
        assert np.array_equal(_download(ctx, dev.weight, w.nbytes), w.view(np.uint8).reshape(-1))
        x = F.synthetic_x(1, K, seed=40)
        dx, dy = ctx.to_device(x), ctx.alloc(N * 4)
        ctx.qmv(dx, dev.weight, dev.scales, dev.biases, dy, 1, K, N, gs, bits, aq_mi355.AQ_OUT_F32)
        ctx.sync()
        check_accumulators(dy.download(np.float32, N), F.reference_f64(x, w, s, b, bits, gs, K), "loaded " + name)
        ctx.free_device_linear(dev)
        assert dev.weight is None
        dx.free()
        dy.free()
    # a dense weight has no affine arrays to upload
    tensors2 = {"d.weight": ("BF16", [4, 8], np.zeros((4, 8), np.uint16))}
    path2 = str(tmp_path / "d.safetensors")
    write_safetensors(path2, tensors2)
    f2 = aq_mi355.SafetensorsFile(path2)
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.upload_linear(f2.load_linear("d", 8))
    assert e.value.code == aq_mi355.AQ_ERR_UNSUPPORTED
    f2.close()
    f.close()


def test_loaded_linear_in_the_tile_major_layout(ctx, tmp_path):
    """file -> loader -> upload -> aq_tile_device_linear -> kernel with AQ_W_TILED: the bytes of the same call on the
    arrays as uploaded; a fused gate|up slab tiled as one tensor; what has no tile-major form is refused and left alone."""
    import aq_mi355
    say("loader -> tile-major -> qmv")
    N, K = 80, 1152
    tensors = {}
    for i, name in enumerate(("gate", "up", "odd")):
        t, _ = affine_entry(name, N, K, 8 if name == "odd" else 4, 64, seed=70 + i)
        tensors.update(t)
    path = str(tmp_path / "t.safetensors")
    write_safetensors(path, tensors)
    f = aq_mi355.SafetensorsFile(path)
    x = F.synthetic_x(3, K, seed=71)
    dx = ctx.to_device(x)
    gate, up = f.load_linear("gate", K), f.load_linear("up", K)
    dev = ctx.upload_linear(gate)
    want, got = ctx.alloc(3 * N * 2), ctx.alloc(3 * N * 2)
    ctx.qmv(dx, dev.weight, dev.scales, dev.biases, want, 3, K, N, 64, 4, 0)
    ctx.tile_device_linear(dev)
    assert dev.scales is None and dev.biases is None and dev.weight
    ctx.qmv(dx, dev.weight, None, None, got, 3, K, N, 64, 4, aq_mi355.AQ_W_TILED)
    ctx.sync()
    assert np.array_equal(got.download(np.uint16, 3 * N), want.download(np.uint16, 3 * N))
    with pytest.raises(aq_mi355.AqError):       # a second time: nothing left to tile
        ctx.tile_device_linear(dev)
    ctx.free_device_linear(dev)
    # the fused gate|up slab as one tile-major tensor
    slab = ctx.upload_fused_gate_up(gate, up)
    rows = slab.rows // 2
    row_bytes, sb_bytes = K // 2, (K // 64) * 2
    ctx.qmv_gate_up(dx, (slab.weight, slab.scales, slab.biases),
                    (slab.weight + rows * row_bytes, slab.scales + rows * sb_bytes, slab.biases + rows * sb_bytes), want, 1, K, N, 64, 4)
    ctx.tile_device_linear(slab)
    half = aq_mi355.tiled_bytes(rows, K, 64, 4)
    ctx.qmv_gate_up(dx, (slab.weight, None, None), (slab.weight + half, None, None), got, 1, K, N, 64, 4,
                    flags=aq_mi355.AQ_W_TILED)
    ctx.sync()
    assert np.array_equal(got.download(np.uint16, N), want.download(np.uint16, N))
    ctx.free_device_linear(slab)
    odd = ctx.upload_linear(f.load_linear("odd", K))
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.tile_device_linear(odd)
    assert e.value.code == aq_mi355.AQ_ERR_UNSUPPORTED and odd.scales
    ctx.free_device_linear(odd)
    for t in (dx, want, got):
        t.free()
    f.close()


@pytest.mark.parametrize("experts", [0, 5])
def test_fused_gate_up_slab_upload(ctx, orc, tmp_path, experts):
    """Separate gate / up tensors become one [E, gate rows | up rows] slab during the upload; the fused
    kernels on that slab agree with the same kernels on separately uploaded parts, and the slab's bytes are
    model.ConcatQuantRows of each expert's pair."""
    import aq_mi355
    say("loader fused gate_up", experts)
    N, K, bits, gs = 40, 256, 4, 64
    tg, (gw, gsb, gb) = affine_entry("e.gate_proj", N, K, bits, gs, seed=50, experts=experts)
    tu, (uw, usb, ub) = affine_entry("e.up_proj", N, K, bits, gs, seed=51, experts=experts)
    path = str(tmp_path / "moe.safetensors")
    write_safetensors(path, {**tg, **tu})
    f = aq_mi355.SafetensorsFile(path)
    gate, up = f.load_linear("e.gate_proj", K), f.load_linear("e.up_proj", K)
    slab = ctx.upload_fused_gate_up(gate, up)
    E = max(experts, 1)
    assert (slab.rows, slab.experts, slab.bits, slab.group_size) == (2 * N, experts, bits, gs)
    wpr, gpr = K * bits // 32, K // gs
    want_w = np.concatenate([gw.reshape(E, N, wpr), uw.reshape(E, N, wpr)], axis=1)
    want_s = np.concatenate([gsb.reshape(E, N, gpr), usb.reshape(E, N, gpr)], axis=1)
    want_b = np.concatenate([gb.reshape(E, N, gpr), ub.reshape(E, N, gpr)], axis=1)
    assert np.array_equal(_download(ctx, slab.weight, want_w.nbytes), want_w.view(np.uint8).reshape(-1))
    assert np.array_equal(_download(ctx, slab.scales, want_s.nbytes), want_s.view(np.uint8).reshape(-1))
    assert np.array_equal(_download(ctx, slab.biases, want_b.nbytes), want_b.view(np.uint8).reshape(-1))
    if experts == 0:
        # byte-identical to model.ConcatQuantRows through the host mirror
        lib = aq_mi355.load()
        import ctypes
        po, so, bo = np.zeros(want_w.nbytes, np.uint8), np.zeros(want_s.nbytes, np.uint8), np.zeros(want_b.nbytes, np.uint8)
        od = ctypes.c_int(0)
        u8 = lambda a: np.ascontiguousarray(a).view(np.uint8).reshape(-1)
        assert lib.aqh_concat_quant_rows(u8(gw).ctypes.data, gw.nbytes, u8(gsb).ctypes.data, gsb.nbytes, u8(gb).ctypes.data, N,
                                         u8(uw).ctypes.data, uw.nbytes, u8(usb).ctypes.data, usb.nbytes, u8(ub).ctypes.data, N,
                                         K, K, bits, bits, gs, gs, po.ctypes.data, so.ctypes.data, bo.ctypes.data,
                                         ctypes.byref(od)) == 0
        assert od.value == 2 * N and np.array_equal(po, u8(want_w)) and np.array_equal(so, u8(want_s))
    routes = 7
    rng = np.random.default_rng(52)
    rhs = rng.integers(0, E, routes).astype(np.int32)
    x = F.synthetic_x(1, K, seed=53)
    dx, dr, dy = ctx.to_device(x), ctx.to_device(rhs), ctx.alloc(routes * N * 4)
    ctx.gather_qmv_gate_up(dx, slab.weight, slab.scales, slab.biases, None, dr, dy, routes, 1, K, N, E, 2 * N, 0, N, gs, bits,
                           aq_mi355.AQ_ACT_GELU_TANH, aq_mi355.AQ_OUT_F32)
    ctx.sync()
    got = dy.download(np.float32, routes * N).reshape(routes, N)
    wq = F.numpy_dequant(want_w.reshape(E * 2 * N, wpr), want_s.reshape(E * 2 * N, gpr), want_b.reshape(E * 2 * N, gpr), bits,
                         gs, K).astype(np.float64).reshape(E, 2 * N, K)
    xf = F.bf16_bits_to_f32(x).astype(np.float64).reshape(K)
    g = np.stack([wq[e, :N] @ xf for e in rhs])
    u = np.stack([wq[e, N:] @ xf for e in rhs])
    want = orc.act_multiply(orc.ACT_GELU_TANH, g.astype(np.float32), u.astype(np.float32))
    assert np.abs(got - want).max() <= 1e-2 * (1 + np.abs(u).max())
    # geometry mismatch between the parts is refused
    up.bits = 8
    with pytest.raises(aq_mi355.AqError):
        ctx.upload_fused_gate_up(gate, up)
    ctx.free_device_linear(slab)
    for t in (dx, dr, dy):
        t.free()
    f.close()
