"""The oracle's GGUF -> affine repack pinned three ways: the reference's own known answers (the fixtures of
go/engine/hip/hip_gguf_affine_adapter_test.go:153-560, rebuilt here byte for byte), ggml's dequantisation
rules as an independent witness (the affine triple must dequantise to exactly what the block does when the
block's scales are bf16-exact, which fixes the position and value of every code and the sign and factor of every
scale and bias), and the half / bf16 conversions against numpy over every half and against the reference's
bit recipe.  The C ABI's layout query is checked against the same table (host code, no device)."""
import numpy as np
import pytest

import gguf_blocks as G
from oracle import orc


def _half(v):
    return np.frombuffer(np.float16(v).tobytes(), np.uint8)


def _bf(u16):
    return float(G.bf16_to_f64(np.array([u16], np.uint16))[0])


def _code(words, col, bits):
    return int(G.unpack_codes(np.asarray(words).reshape(1, -1), col + 1, bits)[0, col])


def _k_scales(block):
    for g in range(4):                      # hip_gguf_affine_adapter_test.go:157-164
        block[4 + g] = g + 1
        block[4 + g + 4] = g + 9
    for g in range(4, 8):
        block[4 + g + 4] = ((g + 9) << 4 | (g + 1)) & 0xFF


def test_q4_k_known_answer():
    block = np.zeros(144, np.uint8)
    block[0:2], block[2:4] = _half(0.5), _half(0.25)
    _k_scales(block)
    for pair in range(4):
        for col in range(32):
            block[16 + pair * 32 + col] = ((2 * pair + col) & 0xF) | (((2 * pair + 1 + col) & 0xF) << 4)
    assert orc.gguf_affine_layout(G.Q4_K, 1, 256) == (4, 32, 32, 8, 144)
    w, s, b = orc.gguf_to_affine(G.Q4_K, 1, 256, block)
    assert w.nbytes == 128 and s.nbytes == 16 and b.nbytes == 16
    assert w[0, 0] == 0x76543210 and w[0, 4] == 0x87654321
    assert (_bf(s[0, 0]), _bf(b[0, 0]), _bf(s[0, 4]), _bf(b[0, 4])) == (0.5, -2.25, 2.5, -3.25)


def test_q4_0_known_answer():
    block = np.zeros(18, np.uint8)
    block[0:2] = _half(0.25)
    for lane in range(16):
        block[2 + lane] = lane | (15 - lane) << 4
    assert orc.gguf_affine_layout(G.Q4_0, 1, 32)[:4] == (4, 32, 4, 1)
    w, s, b = orc.gguf_to_affine(G.Q4_0, 1, 32, block)
    assert [_code(w, c, 4) for c in (0, 7, 8, 15, 16, 23, 24, 31)] == [0, 7, 8, 15, 15, 8, 7, 0]
    assert (_bf(s[0, 0]), _bf(b[0, 0])) == (0.25, -2.0)


def test_q4_1_known_answer():
    block = np.zeros(20, np.uint8)
    block[0:2], block[2:4] = _half(0.5), _half(-1.25)
    for lane in range(16):
        block[4 + lane] = ((lane + 3) & 0xF) | ((lane + 11) & 0xF) << 4
    w, s, b = orc.gguf_to_affine(G.Q4_1, 1, 32, block)
    assert [_code(w, c, 4) for c in (0, 7, 8, 15, 16, 23, 24, 31)] == [3, 10, 11, 2, 11, 2, 3, 10]
    assert (_bf(s[0, 0]), _bf(b[0, 0])) == (0.5, -1.25)


def test_q5_k_known_answer():
    block = np.zeros(176, np.uint8)
    block[0:2], block[2:4] = _half(0.5), _half(0.25)
    _k_scales(block)
    for group in range(8):                  # the test's setQ5, :284-303
        for lane in range(32):
            value = (group + lane) & 0x1F
            il, high = group // 2, group % 2
            block[48 + 32 * il + lane] |= (value & 0xF) << (4 * high)
            if value & 0x10:
                block[16 + lane] |= 1 << (2 * il + high)
    assert orc.gguf_affine_layout(G.Q5_K, 1, 256) == (6, 32, 48, 8, 176)
    w, s, b = orc.gguf_to_affine(G.Q5_K, 1, 256, block)
    assert w.nbytes == 192
    assert [_code(w, c, 6) for c in (0, 15, 16, 3 * 32 + 17)] == [0, 15, 16, 20]
    assert (_bf(s[0, 0]), _bf(b[0, 0])) == (0.5, -2.25)
    codes = G.unpack_codes(w, 256, 6).reshape(8, 32)
    assert np.array_equal(codes, (np.arange(8)[:, None] + np.arange(32)) & 0x1F)


def test_q6_k_known_answer():
    block = np.zeros(210, np.uint8)
    block[208:210] = _half(0.25)
    block[192:208] = np.arange(2, 18, dtype=np.int8).view(np.uint8)
    block[192 + 5] = np.int8(-3).view(np.uint8)
    for group in range(16):                 # the test's setQ6, :343-362
        for lane in range(16):
            value = (32 + group + lane) & 0x3F
            ip, local = group // 8, group % 8
            off, quartile = (16 if local % 2 else 0), local // 2
            ql = ip * 64 + off + lane + (32 if quartile in (1, 3) else 0)
            block[ql] |= (value & 0xF) << (4 if quartile >= 2 else 0)
            block[128 + ip * 32 + off + lane] |= ((value >> 4) & 3) << (quartile * 2)
    assert orc.gguf_affine_layout(G.Q6_K, 1, 256) == (6, 16, 48, 16, 210)
    w, s, b = orc.gguf_to_affine(G.Q6_K, 1, 256, block)
    assert w.nbytes == 192 and s.nbytes == 32
    assert [_code(w, c, 6) for c in (0, 15, 5 * 16 + 2)] == [32, 47, 39]
    assert (_bf(s[0, 0]), _bf(b[0, 0]), _bf(s[0, 5]), _bf(b[0, 5])) == (0.5, -16.0, -0.75, 24.0)


def test_q8_0_known_answer_and_projection():
    block = np.zeros(34, np.uint8)
    block[0:2] = _half(0.5)
    block[2:34] = (np.arange(32) - 16).astype(np.int8).view(np.uint8)
    assert orc.gguf_affine_layout(G.Q8_0, 1, 32)[:4] == (8, 32, 8, 1)
    w, s, b = orc.gguf_to_affine(G.Q8_0, 1, 32, block)
    assert [_code(w, c, 8) for c in (0, 15, 16, 31)] == [112, 127, 128, 143]
    assert (_bf(s[0, 0]), _bf(b[0, 0])) == (0.5, -64.0)
    x = ((np.arange(32) % 7) - 3).astype(np.float32)            # :424-436: the projection over the repacked row
    want = float((x * (np.arange(32) - 16) * 0.5).sum())
    got = orc.hip_reference_projection(x, w.reshape(-1), s.reshape(-1), b.reshape(-1), 1, 32, 32, 8)
    assert abs(float(got[0]) - want) < 1e-4


def test_f32_known_answer_and_quantiser_rules():
    data = np.arange(32, dtype=np.float32)
    assert orc.gguf_affine_layout(G.F32, 1, 32) == (8, 32, 8, 1, 128)
    w, s, b = orc.gguf_to_affine(G.F32, 1, 32, data)
    assert _code(w, 0, 8) == 0 and _code(w, 31, 8) == 255
    assert abs(_bf(s[0, 0]) - 31.0 / 255.0) < 1e-3 and _bf(b[0, 0]) == 0.0
    # a constant group keeps scale 1 and codes 0; NaN and infinities count as 0; codes are round(half away)((v-min)/scale)
    v = np.full((2, 32), 0.75, np.float32)
    v[1] = np.linspace(-3, 5, 32, dtype=np.float32)
    v[1, 4], v[1, 9] = np.nan, np.inf
    w, s, b = orc.gguf_to_affine(G.F32, 2, 32, v)
    assert (_bf(s[0, 0]), _bf(b[0, 0])) == (1.0, 0.75) and not w[0].any()
    clean = np.where(np.isfinite(v[1]), v[1], np.float32(0))
    lo, hi = clean.min(), clean.max()
    scale = np.float32(hi - lo) / np.float32(255)
    q = (clean - lo) / scale
    want = np.minimum(np.floor(q.astype(np.float64) + 0.5), 255).astype(np.int64)
    assert np.array_equal(G.unpack_codes(w[1:2], 32, 8)[0], want)
    assert s[1, 0] == orc.gguf_f32_to_bf16(float(scale)) and b[1, 0] == orc.gguf_f32_to_bf16(float(lo))


@pytest.mark.parametrize("gguf_type", [G.Q4_0, G.Q4_1, G.Q8_0, G.Q4_K, G.Q5_K, G.Q6_K])
def test_affine_triple_dequantises_like_the_block(gguf_type):
    """bf16-exact block scales: scale*code + bias (affine) == ggml's value of the same element, exactly."""
    rows, cols = 5, 768
    data = G.random_blocks(gguf_type, rows, cols, seed=11 + gguf_type, exact=True)
    bits, group = G.AFFINE[gguf_type]
    w, s, b = orc.gguf_to_affine(gguf_type, rows, cols, data)
    assert w.shape == (rows, cols * bits // 32) and s.shape == (rows, cols // group)
    got = G.affine_dequant(w, s, b, cols, bits, group)
    want = G.ggml_dequant(gguf_type, rows, cols, data)
    assert np.array_equal(got, want)
    if gguf_type == G.Q5_K:
        assert G.unpack_codes(w, cols, 6).max() <= 31


@pytest.mark.parametrize("gguf_type", [G.Q4_0, G.Q4_1, G.Q8_0, G.Q4_K, G.Q5_K, G.Q6_K])
def test_general_blocks_within_bf16_rounding(gguf_type):
    """Arbitrary half scales (subnormal ones too): codes as before, values within the bf16 rounding of scale and bias."""
    rows, cols = 3, 512
    data = G.random_blocks(gguf_type, rows, cols, seed=31 + gguf_type)
    bits, group = G.AFFINE[gguf_type]
    w, s, b = orc.gguf_to_affine(gguf_type, rows, cols, data)
    got = G.affine_dequant(w, s, b, cols, bits, group)
    want = G.ggml_dequant(gguf_type, rows, cols, data)
    sref = np.repeat(np.abs(G.bf16_to_f64(s)), group, axis=1)
    bref = np.repeat(np.abs(G.bf16_to_f64(b)), group, axis=1)
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * (sref * ((1 << bits) - 1) + bref) + 1e-30)


def test_conversions_and_errors():
    halves = np.arange(65536, dtype=np.uint32)
    mine = np.array([np.float32(orc.gguf_f16_to_f32(int(h))) for h in halves[::7]], np.float32)
    ref = halves[::7].astype(np.uint16).view(np.float16).astype(np.float32)
    same = (mine.view(np.uint32) == ref.view(np.uint32)) | (np.isnan(mine) & np.isnan(ref))
    assert same.all()
    # float -> bf16: ties to even on the bit pattern, and (unlike a NaN-aware conversion) a NaN with a small payload
    # carries into infinity, as the reference's three-line recipe does
    assert orc.gguf_f32_to_bf16(1.0) == 0x3F80
    assert orc.gguf_f32_to_bf16(float(np.array([0x3F808000], np.uint32).view(np.float32)[0])) == 0x3F80     # tie -> even
    assert orc.gguf_f32_to_bf16(float(np.array([0x3F818000], np.uint32).view(np.float32)[0])) == 0x3F82     # tie -> even
    assert orc.gguf_f32_to_bf16(float(np.array([0x3F808001], np.uint32).view(np.float32)[0])) == 0x3F81
    for gguf_type, (bc, bb) in G.BLOCK.items():
        with pytest.raises(orc.OracleError) as e:
            orc.gguf_affine_layout(gguf_type, 2, bc + 16)
        assert e.value.code == orc.ORC_ERR_DIMS
        with pytest.raises(orc.OracleError) as e:
            orc.gguf_to_affine(gguf_type, 2, bc, np.zeros(2 * bb - 1, np.uint8))
        assert e.value.code == orc.ORC_ERR_SIZE
    for bad in (1, 6, 7, 10, 30):            # F16, Q5_0, Q5_1, Q2_K, BF16: not repacked
        with pytest.raises(orc.OracleError) as e:
            orc.gguf_affine_layout(bad, 1, 256)
        assert e.value.code == orc.ORC_ERR_BITS
    with pytest.raises(orc.OracleError):
        orc.gguf_affine_layout(G.Q4_0, 0, 32)


def test_library_layout_query_matches():
    import aq_mi355
    for gguf_type, (bc, _) in G.BLOCK.items():
        for rows, cols in ((1, bc), (7, 3 * bc), (4096, 14336 // bc * bc)):
            lay = aq_mi355.gguf_affine_layout(gguf_type, rows, cols)
            bits, group, pc, groups, src = orc.gguf_affine_layout(gguf_type, rows, cols)
            assert (lay.bits, lay.group_size, lay.packed_cols, lay.groups, lay.src_bytes) == (bits, group, pc, groups, src)
            assert lay.packed_bytes == rows * pc * 4 and lay.scales_bytes == rows * groups * 2
        with pytest.raises(aq_mi355.AqError) as e:
            aq_mi355.gguf_affine_layout(gguf_type, 2, bc + 16)
        assert e.value.code == aq_mi355.AQ_ERR_SHAPE
    with pytest.raises(aq_mi355.AqError) as e:
        aq_mi355.gguf_affine_layout(1, 2, 256)
    assert e.value.code == aq_mi355.AQ_ERR_UNSUPPORTED
