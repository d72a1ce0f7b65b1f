"""Deterministic inputs for the parity tests.

Two kinds:
  * the formula fixtures the reference's own tests build (each function names the Go test it
    re-derives; every value is a closed formula, so they can be regenerated anywhere);
  * the seeded synthetic distributions of the benchmark configs (numpy PCG64).
All byte layouts are the MLX group-affine ones: packed uint32 LSB-first along K, bf16 scales/biases.
"""
import numpy as np


# ---- bf16 helpers (numpy, independent of both the oracle and the library) ---------------------

def f32_to_bf16_bits(a):
    """Round-to-nearest-even float32 -> bf16 bit patterns (uint16); NaN kept quiet."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return (r & 0xFFFF).astype(np.uint16)


def bf16_bits_to_f32(h):
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def pack_codes(codes, bits):
    """codes [N, K] (ints < 2**bits) -> uint32 [N, K*bits/32], LSB-first, codes may straddle words."""
    codes = np.asarray(codes, dtype=np.uint64)
    n, k = codes.shape
    assert (k * bits) % 32 == 0
    words = np.zeros((n, k * bits // 32), dtype=np.uint64)
    for col in range(k):
        bit = col * bits
        wi, sh = bit // 32, bit % 32
        v = codes[:, col] & ((1 << bits) - 1)
        words[:, wi] |= (v << sh) & 0xFFFFFFFF
        if sh + bits > 32:
            words[:, wi + 1] |= v >> (32 - sh)
    return words.astype(np.uint32)


def pack_codes_fast(codes, bits):
    """Vectorised pack for word-clean widths (1, 2, 4, 8)."""
    assert 32 % bits == 0
    per = 32 // bits
    codes = np.asarray(codes, dtype=np.uint32)
    n, k = codes.shape
    c = codes.reshape(n, k // per, per)
    shifts = (np.arange(per, dtype=np.uint32) * bits).astype(np.uint32)
    return np.bitwise_or.reduce(c << shifts, axis=2).astype(np.uint32)


def unpack_codes(words, bits, k):
    """Inverse of pack_codes: uint32 [N, W] -> codes [N, K] (python ints via uint64 math)."""
    words = np.asarray(words, dtype=np.uint64)
    n = words.shape[0]
    out = np.zeros((n, k), dtype=np.uint32)
    for col in range(k):
        bit = col * bits
        wi, sh = bit // 32, bit % 32
        v = words[:, wi] >> sh
        if sh + bits > 32:
            v = v | (words[:, wi + 1] << (32 - sh))
        out[:, col] = (v & ((1 << bits) - 1)).astype(np.uint32)
    return out


def numpy_dequant(words, scales_bits, biases_bits, bits, group_size, k):
    """float32 scale*code + bias, written the way tools/mlxaffine_dequant.py:52-69 writes it
    (broadcast shifts, repeat scales along the group)."""
    words = np.asarray(words, dtype=np.uint32)
    n = words.shape[0]
    if 32 % bits == 0:
        per = 32 // bits
        shifts = np.arange(per, dtype=np.uint32) * bits
        codes = ((words[..., None] >> shifts) & ((1 << bits) - 1)).reshape(n, k)
    else:
        codes = unpack_codes(words, bits, k)
    s = bf16_bits_to_f32(scales_bits).reshape(n, k // group_size)
    b = bf16_bits_to_f32(biases_bits).reshape(n, k // group_size)
    return codes.astype(np.float32) * np.repeat(s, group_size, axis=1) + np.repeat(b, group_size, axis=1)


# ---- the reference's own formula fixtures ---------------------------------------------------

def quant_affine_fixture():
    """enginetest.quantAffineFixture (go/engine/enginetest/quant_parity.go:35-68):
    outDim=8, inDim=128, groupSize=64, bits=4."""
    out_dim, in_dim, gs, bits = 8, 128, 64, 4
    groups = in_dim // gs
    codes = np.zeros((out_dim, in_dim), dtype=np.uint32)
    scales = np.zeros((out_dim, groups), dtype=np.float32)
    biases = np.zeros((out_dim, groups), dtype=np.float32)
    for r in range(out_dim):
        for g in range(groups):
            scales[r, g] = np.float32(0.25) + np.float32(0.125) * np.float32(g + r)
            biases[r, g] = np.float32(-1) + np.float32(0.5) * np.float32((g + r) % 3)
            for j in range(gs):
                c = g * gs + j
                codes[r, c] = (c * 5 + r * 3 + 1) % 16
    x = np.array([np.float32(0.1) * np.float32((i % 7) - 3) for i in range(in_dim)], dtype=np.float32)
    return dict(x=f32_to_bf16_bits(x), packed=pack_codes_fast(codes, bits), scales=f32_to_bf16_bits(scales),
                biases=f32_to_bf16_bits(biases), codes=codes, out_dim=out_dim, in_dim=in_dim, group_size=gs, bits=bits)


def hw_fixture_q8_cols256():
    """TestHIPHardwareMLXAffineQ8ProjectionCols256Group32 (go/engine/hip/hip_hardware_test.go:1930-1965)."""
    rows, cols, gs, bits = 3, 256, 32, 8
    groups = cols // gs
    x = np.array([np.float32((c % 17) - 8) / np.float32(8) for c in range(cols)], dtype=np.float32)
    codes = np.array([[(r * 19 + c * 7) & 0xFF for c in range(cols)] for r in range(rows)], dtype=np.uint32)
    s = np.array([[np.float32(0.015625) * np.float32(r + g + 1) for g in range(groups)] for r in range(rows)], dtype=np.float32)
    b = np.array([[np.float32(-0.25) * np.float32(r + 1) for g in range(groups)] for r in range(rows)], dtype=np.float32)
    return dict(x=x, packed=pack_codes(codes, bits), scales=f32_to_bf16_bits(s), biases=f32_to_bf16_bits(b),
                codes=codes, rows=rows, cols=cols, group_size=gs, bits=bits, tol=0.01)


def hw_fixture_q8_cols3072():
    """TestHIPHardwareMLXAffineQ8ProjectionCols3072Group32 (go/engine/hip/hip_hardware_test.go:1985-2020)."""
    rows, cols, gs, bits = 5, 3072, 32, 8
    groups = cols // gs
    x = np.array([np.float32((c % 23) - 11) / np.float32(64) for c in range(cols)], dtype=np.float32)
    codes = np.array([[(r * 29 + c * 11) & 0xFF for c in range(cols)] for r in range(rows)], dtype=np.uint32)
    s = np.array([[np.float32(0.001953125) * np.float32((r + g) % 7 + 1) for g in range(groups)] for r in range(rows)], dtype=np.float32)
    b = np.array([[np.float32(-0.03125) * np.float32(r + 1) for g in range(groups)] for r in range(rows)], dtype=np.float32)
    return dict(x=x, packed=pack_codes(codes, bits), scales=f32_to_bf16_bits(s), biases=f32_to_bf16_bits(b),
                codes=codes, rows=rows, cols=cols, group_size=gs, bits=bits, tol=0.03)


def hw_fixture_q4_g64_tokens16():
    """The q4 group-64 17x704 batch-16 case (go/engine/hip/hip_hardware_test.go:7822-7878)."""
    rows, cols, gs, batch = 17, 704, 64, 16
    x0 = np.array([np.float32(i % 11 - 5) / np.float32(8) for i in range(cols)], dtype=np.float32)
    codes = np.array([(i * 7 + 3) % 16 for i in range(rows * cols)], dtype=np.uint32).reshape(rows, cols)
    ng = rows * (cols // gs)
    s = np.array([np.float32(i % 4 + 1) / np.float32(8) for i in range(ng)], dtype=np.float32)
    b = np.array([np.float32(i % 5 - 2) / np.float32(8) for i in range(ng)], dtype=np.float32)
    xs = np.stack([x0 * (np.float32(t + 1) / np.float32(batch)) for t in range(batch)]).astype(np.float32)
    return dict(x=xs, packed=pack_codes_fast(codes, 4), scales=f32_to_bf16_bits(s), biases=f32_to_bf16_bits(b),
                codes=codes, rows=rows, cols=cols, group_size=gs, bits=4, tokens=batch, tol=0.001)


def hw_fixture_q4_gelu_cols2560(group_size):
    """testHIPHardwareMLXAffineQ4GELUTanhCols2560 (go/engine/hip/hip_hardware_test.go:2318-2407): rows=32,
    cols=2560, 4 bit, gate built with (valueStride 5, scaleBase 2^-9), up with (7, 0.00146484375); the
    reference accepts the device result within 0.03 of gelu_tanh(gate)*up."""
    rows, cols, bits = 32, 2560, 4
    groups = cols // group_size
    x = np.array([np.float32((c % 23) - 11) / np.float32(128) for c in range(cols)], dtype=np.float32)

    def make(stride, base):
        r = np.arange(rows).reshape(-1, 1)
        c = np.arange(cols).reshape(1, -1)
        codes = ((r * stride + c * (stride + 2)) & 0x0F).astype(np.uint32)
        g = np.arange(groups).reshape(1, -1)
        s = (np.float32(base) * ((r + g) % 7 + 1).astype(np.float32)).astype(np.float32)
        b = (-np.float32(base) * ((r + g) % 3 + 1).astype(np.float32)).astype(np.float32)
        return dict(packed=pack_codes_fast(codes, bits), scales=f32_to_bf16_bits(s), biases=f32_to_bf16_bits(b), codes=codes)

    return dict(x=x, gate=make(5, 0.001953125), up=make(7, 0.00146484375), rows=rows, cols=cols, group_size=group_size,
                bits=bits, tol=0.03)


def synthetic_float32(n, salt):
    """metal test helper syntheticFloat32 (go/engine/metal/test_helpers_test.go:54-60)."""
    i = np.arange(n, dtype=np.int64)
    return (((i * salt + 7) % 101 - 50).astype(np.float32) * np.float32(0.03125)).astype(np.float32)


def gather_fixture(out_dim, in_dim, gs, bits, num_experts, expert_rows, batched_x, routes):
    """gatherRoutesParityCase inputs (go/engine/metal/qmv_gather_test.go:18-40)."""
    nbytes = num_experts * expert_rows * in_dim * bits // 8
    packed = ((np.arange(nbytes, dtype=np.int64) * 131 + 17) % 256).astype(np.uint8)
    nsb = num_experts * expert_rows * (in_dim // gs)
    scales = f32_to_bf16_bits(synthetic_float32(nsb, 11))
    biases = f32_to_bf16_bits(synthetic_float32(nsb, 13))
    x_rows = routes if batched_x else 1
    lhs = np.array([(i * 2) % x_rows for i in range(routes)], dtype=np.int32) if batched_x else None
    x = f32_to_bf16_bits(synthetic_float32(x_rows * in_dim, 7))
    rhs = np.array([(i * 3 + 1) % num_experts for i in range(routes)], dtype=np.int32)
    return dict(x=x, x_rows=x_rows, packed=packed.view(np.uint32), scales=scales, biases=biases, lhs=lhs, rhs=rhs)


def cbq_synth_w(out_dim, in_dim):
    """cbqSynthW (go/engine/metal/quant_seam_backend_test.go:21-29)."""
    i = np.arange(out_dim * in_dim, dtype=np.int64)
    return (((i % 17) - 8).astype(np.float32) * np.float32(0.037)).astype(np.float32)


def synth_weight(out_dim, in_dim):
    """synthWeight (go/model/quant/mlxaffine/mlxaffine_test.go:16-27)."""
    w = np.zeros((out_dim, in_dim), dtype=np.float32)
    for r in range(out_dim):
        amp = np.float32(0.01) + np.float32(0.5) * np.float32(r + 1) / np.float32(out_dim)
        bias = np.float32(0.1) * np.float32(r % 3 - 1)
        c = np.arange(in_dim)
        w[r] = bias + amp * np.sin((r * 7 + c).astype(np.float64) * 0.013).astype(np.float32)
    return w


# ---- seeded synthetic benchmark distributions -----------------------------------------------

BASE_SEED = 0xA0


def synthetic_affine(N, K, bits=4, group_size=64, seed=BASE_SEED):
    """Codes uniform, scale = bf16(|N(0,0.02)| + 1e-3), bias = bf16(-mid*scale + N(0,1e-3)) from the
    bf16-rounded scale (mid = 8 for 4 bit, 128 for 8 bit)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    words = rng.integers(0, 1 << 32, size=(N, K * bits // 32), dtype=np.uint64).astype(np.uint32)
    g = K // group_size
    s = (np.abs(rng.normal(0.0, 0.02, size=(N, g))) + 1e-3).astype(np.float32)
    s_bits = f32_to_bf16_bits(s)
    s_r = bf16_bits_to_f32(s_bits)
    mid = np.float32(1 << (bits - 1))
    b = (-mid * s_r + rng.normal(0.0, 1e-3, size=(N, g)).astype(np.float32)).astype(np.float32)
    return words, s_bits, f32_to_bf16_bits(b)


def synthetic_x(M, K, seed=BASE_SEED + 1000):
    rng = np.random.Generator(np.random.PCG64(seed))
    return f32_to_bf16_bits(rng.normal(0.0, 1.0, size=(M, K)).astype(np.float32))


def reference_f64(x_bits, words, s_bits, b_bits, bits, group_size, K):
    """y[M,N] in float64 from the numpy dequant (fp32 weights, exact) -- the fp32-weight, wide-accumulate
    reference the tolerance is stated against."""
    w = numpy_dequant(words, s_bits, b_bits, bits, group_size, K).astype(np.float64)
    x = bf16_bits_to_f32(x_bits).astype(np.float64).reshape(-1, K)
    return x @ w.T


# ---- tile-major device layout (4-bit, group 64), written independently of the library's kernels --------------------

def tile_cps(k):
    """Chunks of 256 codes per wavefront step for this K (3 where that shares K out evenly over 2 or 4 wavefronts)."""
    chunks = (k + 255) // 256
    nw4 = ((chunks + 3) // 4 + 1) & ~1
    return 3 if (nw4 <= 4 and (chunks + 2) // 3 <= nw4) else 4


def tile_major(words, s_bits, b_bits, n, k):
    """MLX arrays of a 4-bit group-64 tensor -> the tile-major byte string aq_tile_weights must produce.

    Sets of 16 rows (zero-padded); per set, steps of `cps` chunks of 256 codes; per step 1 KiB of scales and biases
    (lane l = (row l % 16, chunk l // 16 of the step): four scales then four biases, zeros where there is no group),
    then 1 KiB per 128-code half (lane l: bytes [16 (l // 16), +16) of that half of row l % 16)."""
    assert k % 128 == 0
    cps = tile_cps(k)
    halves, groups = k // 128, k // 64
    chunks = (halves + 1) // 2
    steps = (chunks + cps - 1) // cps
    sets = (n + 15) // 16
    wb = np.zeros((sets * 16, k // 2), dtype=np.uint8)
    wb[:n] = np.ascontiguousarray(words, dtype=np.uint32).reshape(n, k // 8).view(np.uint8)
    sp = np.zeros((sets * 16, steps * cps * 4), dtype=np.uint16)
    bp = np.zeros_like(sp)
    sp[:n, :groups] = np.asarray(s_bits, dtype=np.uint16).reshape(n, groups)
    bp[:n, :groups] = np.asarray(b_bits, dtype=np.uint16).reshape(n, groups)
    out = []
    for st in range(sets):
        rows = slice(16 * st, 16 * st + 16)
        for step in range(steps):
            sb = np.zeros((4, 16, 8), dtype=np.uint16)  # [lane group j][row n][4 scales | 4 biases]
            for j in range(cps):
                g0 = 4 * (step * cps + j)
                sb[j, :, :4] = sp[rows, g0:g0 + 4]
                sb[j, :, 4:] = bp[rows, g0:g0 + 4]
            out.append(sb.tobytes())
            for h in range(2 * step * cps, min(2 * (step + 1) * cps, halves)):
                piece = wb[rows, 64 * h:64 * h + 64].reshape(16, 4, 16)  # [row][j][16 bytes]
                out.append(np.ascontiguousarray(piece.transpose(1, 0, 2)).tobytes())
    return np.frombuffer(b"".join(out), dtype=np.uint8)
