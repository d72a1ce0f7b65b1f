"""Rows of an M-row call carry the bytes of single-row calls (go/engine/metal/qmv_rows.go:14-24): the reference holds its
flat tile (M <= 4) and its wide tile (M 5..8) to that at (out, in) = (512, 1024), (3840, 7680) and (704, 2816)
(go/engine/metal/qmv_rows_test.go:33-100); here the same for 2..8 rows of 4-bit group-64 codes at those shapes, at the
down-projection shape whose K is 14 steps long, at a K beyond the diagonal kernels and at a K that is no multiple of
128 - the shapes where a call of several rows and a call of one row are served by different launch plans."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, say

pytestmark = pytest.mark.gpu

SHAPES = [(512, 1024), (3840, 7680), (704, 2816), (4096, 14336), (14336, 4096), (272, 16384), (144, 16384 + 256),
          (96, 1024 + 64), (200, 640)]


@pytest.mark.parametrize("N,K", SHAPES)
def test_rows_have_the_bytes_of_single_row_calls(ctx, N, K):
    w, s, b = F.synthetic_affine(N, K, 4, 64, seed=1000 + N + K)
    d = DeviceAffine(ctx, w, s, b)
    x_bits = F.synthetic_x(8, K, seed=2000 + K)
    x = ctx.to_device(x_bits)
    single = np.zeros((8, N), dtype=np.uint16)
    y1 = ctx.alloc(N * 2)
    for m in range(8):
        ctx.fill_zero(y1)
        ctx.qmv(x.ptr + m * K * 2, d.w, d.s, d.b, y1, 1, K, N, 64, 4, 0)
        ctx.sync()
        single[m] = y1.download(np.uint16)
    one_row_kernel = ctx.last_variant(0)
    for M in range(2, 9):
        say("rows", N, K, M)
        y = ctx.alloc(M * N * 2)
        ctx.fill_zero(y)
        ctx.qmv(x, d.w, d.s, d.b, y, M, K, N, 64, 4, 0)
        ctx.sync()
        got = y.download(np.uint16).reshape(M, N)
        assert (got == single[:M]).all(), (N, K, M, one_row_kernel, ctx.last_variant(0), int((got != single[:M]).sum()))
        y.free()
