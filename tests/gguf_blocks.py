"""GGUF block tensors for the repack tests: random blocks per format, and ggml's own dequantisation rules
(dequantize_row_q4_0 / q4_1 / q8_0 / q4_K / q5_K / q6_K as ggml publishes them) written with numpy as an
independent witness of where every code of a block belongs and what it is worth."""
import numpy as np

F32, Q4_0, Q4_1, Q8_0, Q4_K, Q5_K, Q6_K = 0, 2, 3, 8, 12, 13, 14
BLOCK = {F32: (32, 128), Q4_0: (32, 18), Q4_1: (32, 20), Q8_0: (32, 34), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210)}
AFFINE = {F32: (8, 32), Q4_0: (4, 32), Q4_1: (4, 32), Q8_0: (8, 32), Q4_K: (4, 32), Q5_K: (6, 32), Q6_K: (6, 16)}
NAMES = {F32: "F32", Q4_0: "Q4_0", Q4_1: "Q4_1", Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K"}


def _halves(rng, n, exact):
    """n fp16 bit patterns.  exact: +-2^e * {1..15}/8-free values whose products with 7-bit integers fit bf16."""
    if exact:
        v = rng.choice([-1.0, 1.0], n) * np.exp2(rng.integers(-9, 2, n)).astype(np.float64)
        return v.astype(np.float16).view(np.uint16)
    v = rng.normal(0, 0.05, n).astype(np.float16)
    v[rng.integers(0, n, max(1, n // 16))] = np.float16(6e-6)       # subnormal halves
    return v.view(np.uint16)


def random_blocks(gguf_type, rows, cols, seed, exact=False):
    """uint8 bytes of a [rows, cols] tensor of this type."""
    rng = np.random.default_rng(seed)
    bc, bb = BLOCK[gguf_type]
    n = rows * (cols // bc)
    if gguf_type == F32:
        v = rng.normal(0, 1.5, (rows, cols)).astype(np.float32)
        v[rng.integers(0, rows, 3), rng.integers(0, cols, 3)] = [np.nan, np.inf, -np.inf]
        v[0, :32] = 0.75                                         # a constant group: scale 1, codes 0
        if cols >= 64:
            v[0, 32:64] = np.arange(32, dtype=np.float32)        # the reference's fixture
        return v.view(np.uint8).reshape(-1).copy()
    blk = rng.integers(0, 256, (n, bb), dtype=np.uint8)
    if gguf_type in (Q4_0, Q8_0):
        blk[:, 0:2] = _halves(rng, n, exact).view(np.uint8).reshape(n, 2)
    elif gguf_type in (Q4_1, Q4_K, Q5_K):
        blk[:, 0:2] = _halves(rng, n, exact).view(np.uint8).reshape(n, 2)
        blk[:, 2:4] = _halves(rng, n, exact).view(np.uint8).reshape(n, 2)
    else:
        blk[:, 208:210] = _halves(rng, n, exact).view(np.uint8).reshape(n, 2)
    return blk.reshape(-1)


def _f16(b2):
    return np.ascontiguousarray(b2).view(np.float16).astype(np.float64).reshape(-1)


def _scale_min_k4(q):
    """get_scale_min_k4 for j = 0..7 over [n, 12] bytes -> two [n, 8] arrays."""
    q = q.astype(np.int64)
    sc = np.empty((q.shape[0], 8), np.int64)
    mn = np.empty_like(sc)
    for j in range(8):
        if j < 4:
            sc[:, j], mn[:, j] = q[:, j] & 63, q[:, j + 4] & 63
        else:
            sc[:, j] = (q[:, j + 4] & 0xF) | ((q[:, j - 4] >> 6) << 4)
            mn[:, j] = (q[:, j + 4] >> 4) | ((q[:, j] >> 6) << 4)
    return sc, mn


def ggml_dequant(gguf_type, rows, cols, data):
    """float64 [rows, cols] by ggml's dequantize_row_* rules."""
    bc, bb = BLOCK[gguf_type]
    n = rows * (cols // bc)
    blk = np.asarray(data, np.uint8).reshape(n, bb)
    y = np.empty((n, bc), np.float64)
    if gguf_type == Q4_0:
        d = _f16(blk[:, 0:2])[:, None]
        qs = blk[:, 2:18].astype(np.int64)
        y[:, :16], y[:, 16:] = ((qs & 0xF) - 8) * d, ((qs >> 4) - 8) * d
    elif gguf_type == Q4_1:
        d, m = _f16(blk[:, 0:2])[:, None], _f16(blk[:, 2:4])[:, None]
        qs = blk[:, 4:20].astype(np.int64)
        y[:, :16], y[:, 16:] = (qs & 0xF) * d + m, (qs >> 4) * d + m
    elif gguf_type == Q8_0:
        y[:] = blk[:, 2:34].view(np.int8).astype(np.float64) * _f16(blk[:, 0:2])[:, None]
    elif gguf_type in (Q4_K, Q5_K):
        d, dmin = _f16(blk[:, 0:2]), _f16(blk[:, 2:4])
        sc, mn = _scale_min_k4(blk[:, 4:16])
        if gguf_type == Q4_K:
            qh, ql = None, blk[:, 16:144].astype(np.int64)
        else:
            qh, ql = blk[:, 16:48].astype(np.int64), blk[:, 48:176].astype(np.int64)
        for j in range(4):                              # 64 values: low nibbles, then high nibbles, of 32 bytes
            q = ql[:, 32 * j:32 * j + 32]
            lo, hi = q & 0xF, q >> 4
            if qh is not None:
                lo = lo + np.where(qh & (1 << (2 * j)), 16, 0)
                hi = hi + np.where(qh & (2 << (2 * j)), 16, 0)
            y[:, 64 * j:64 * j + 32] = (d * sc[:, 2 * j])[:, None] * lo - (dmin * mn[:, 2 * j])[:, None]
            y[:, 64 * j + 32:64 * j + 64] = (d * sc[:, 2 * j + 1])[:, None] * hi - (dmin * mn[:, 2 * j + 1])[:, None]
    elif gguf_type == Q6_K:
        d = _f16(blk[:, 208:210])
        scales = blk[:, 192:208].view(np.int8).astype(np.float64)
        for half in range(2):
            ql = blk[:, 64 * half:64 * half + 64].astype(np.int64)
            qh = blk[:, 128 + 32 * half:160 + 32 * half].astype(np.int64)
            sc = scales[:, 8 * half:8 * half + 8]
            l = np.arange(32)
            isub = l // 16
            q1 = ((ql[:, :32] & 0xF) | (((qh >> 0) & 3) << 4)) - 32
            q2 = ((ql[:, 32:] & 0xF) | (((qh >> 2) & 3) << 4)) - 32
            q3 = ((ql[:, :32] >> 4) | (((qh >> 4) & 3) << 4)) - 32
            q4 = ((ql[:, 32:] >> 4) | (((qh >> 6) & 3) << 4)) - 32
            base = 128 * half
            for k, q in enumerate((q1, q2, q3, q4)):
                y[:, base + 32 * k:base + 32 * k + 32] = d[:, None] * sc[:, isub + 2 * k] * q
    else:
        raise ValueError(gguf_type)
    return y.reshape(rows, cols)


def unpack_codes(words, cols, bits):
    """[rows, cols] codes of packed uint32 rows (LSB-first bit fields that may straddle words)."""
    rows = words.shape[0]
    bitsarr = np.unpackbits(np.ascontiguousarray(words).view(np.uint8).reshape(rows, -1), axis=1, bitorder="little")
    fields = bitsarr[:, :cols * bits].reshape(rows, cols, bits).astype(np.int64)
    return (fields << np.arange(bits)).sum(axis=2)


def bf16_to_f64(u16):
    return (np.asarray(u16, np.uint32) << 16).view(np.float32).astype(np.float64)


def affine_dequant(words, scales, biases, cols, bits, group):
    codes = unpack_codes(words, cols, bits)
    return np.repeat(bf16_to_f64(scales), group, axis=1) * codes + np.repeat(bf16_to_f64(biases), group, axis=1)
