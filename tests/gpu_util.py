"""Helpers shared by the GPU parity tests: tolerance checks stated once, device round trips."""
import sys

import numpy as np

import fixtures as F

MAX_ABS = 1e-2   # max-abs-err bound on the fp32 accumulator vs the fp32-weight reference
REL = 2e-3       # rel-err bound (elementwise where |ref| >= 1, and as an L2 ratio overall)
BF16_ABS = 2e-3  # absolute escape of the one-ulp bf16 store check, for outputs near zero


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def check_accumulators(got_f32, ref_f64, what):
    got = np.asarray(got_f32, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref_f64, dtype=np.float64).reshape(-1)
    assert got.shape == ref.shape, what
    err = np.abs(got - ref)
    assert np.isfinite(got).all(), what
    assert err.max() <= MAX_ABS, "%s: max-abs-err %.3e > %.0e" % (what, err.max(), MAX_ABS)
    big = np.abs(ref) >= 1.0
    if big.any():
        rel = (err[big] / np.abs(ref[big])).max()
        assert rel <= REL, "%s: rel-err %.3e > %.0e" % (what, rel, REL)
    denom = np.linalg.norm(ref)
    if denom > 0:
        assert np.linalg.norm(got - ref) / denom <= REL, what
    return err.max()


def check_bf16_store(got_bits, ref_f64, what):
    """bf16 outputs must sit within one bf16 ulp of bf16(reference).  Near zero a bf16 ulp is finer
    than any fp32 summation-order difference, so a store also passes when it is within BF16_ABS of
    the reference in absolute terms (a fifth of the stated max-abs-err bound)."""
    got_bits = np.asarray(got_bits, dtype=np.uint16).reshape(-1)
    ref_bits = F.f32_to_bf16_bits(np.asarray(ref_f64, dtype=np.float64).reshape(-1).astype(np.float32))
    # monotone integer key of a bf16 pattern, so adjacent values differ by 1
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    d = np.abs(key(got_bits) - key(ref_bits))
    absd = np.abs(F.bf16_bits_to_f32(got_bits).astype(np.float64) - F.bf16_bits_to_f32(ref_bits).astype(np.float64))
    bad = (d > 1) & (absd > BF16_ABS)
    assert not bad.any(), "%s: bf16 store is %d ulp from bf16(reference)" % (what, d[bad].max())


class DeviceAffine:
    """An affine tensor resident on the device."""

    def __init__(self, ctx, words, s_bits, b_bits):
        self.w = ctx.to_device(np.ascontiguousarray(words, dtype=np.uint32))
        self.s = ctx.to_device(np.ascontiguousarray(s_bits, dtype=np.uint16))
        self.b = ctx.to_device(np.ascontiguousarray(b_bits, dtype=np.uint16))

    def free(self):
        for t in (self.w, self.s, self.b):
            t.free()


def run_qmv(ctx, x_bits, dw, M, K, N, gs, bits, f32, fn="qmv"):
    import aq_mi355
    dx = ctx.to_device(np.ascontiguousarray(x_bits, dtype=np.uint16))
    dy = ctx.alloc(M * N * (4 if f32 else 2))
    ctx.fill_zero(dy)
    getattr(ctx, fn)(dx, dw.w, dw.s, dw.b, dy, M, K, N, gs, bits, aq_mi355.AQ_OUT_F32 if f32 else 0)
    ctx.sync()
    out = dy.download(np.float32 if f32 else np.uint16, M * N).reshape(M, N)
    dx.free()
    dy.free()
    return out
