"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle and the
reference's fixtures.  Bar: dequantised weights bit-exact; fp32 accumulators within
max-abs-err 1e-2 and rel-err 2e-3 of the fp32-weight reference; bf16 stores within one bf16
ulp of bf16(reference)."""
import numpy as np
import pytest

import fixtures as F
from gpu_util import DeviceAffine, check_accumulators, check_bf16_store, run_qmv, say

pytestmark = pytest.mark.gpu


# ---- dequant: bit exact -----------------------------------------------------------------------

@pytest.mark.parametrize("N,K,bits,gs", [(8, 128, 4, 64), (33, 704, 4, 64), (64, 2048, 4, 64), (7, 256, 8, 32),
                                         (16, 512, 8, 64), (5, 640, 2, 64), (4, 128, 1, 128), (9, 512, 4, 128),
                                         (6, 192, 6, 32), (6, 256, 3, 64), (6, 256, 5, 64), (3, 64, 4, 16)])
def test_dequant_bit_exact(ctx, orc, N, K, bits, gs):
    say("dequant", N, K, bits, gs)
    rng = np.random.default_rng(N * 1000 + K + bits)
    codes = rng.integers(0, 1 << bits, size=(N, K)).astype(np.uint32)
    words = F.pack_codes(codes, bits)
    s = rng.integers(0, 65536, size=(N, K // gs)).astype(np.uint16)
    b = rng.integers(0, 65536, size=(N, K // gs)).astype(np.uint16)
    # any finite bf16 pattern, denormals and values whose product with a code overflows included;
    # inf/NaN inputs are left out (a NaN's payload is not part of the contract)
    s = np.where((s & 0x7F80) == 0x7F80, s & 0xBFFF, s).astype(np.uint16)
    b = np.where((b & 0x7F80) == 0x7F80, b & 0xBFFF, b).astype(np.uint16)
    dw = DeviceAffine(ctx, words, s, b)
    dout = ctx.alloc(N * K * 4)
    ctx.dequant_f32(dw.w, dw.s, dw.b, dout, N, K, gs, bits)
    ctx.sync()
    got = dout.download(np.uint32, N * K).reshape(N, K)
    if bits in (1, 2, 4, 8):
        want = orc.dequantize(words, s, b, N, K, bits, gs).view(np.uint32)
    else:  # straddling widths are outside DequantizeTensor: same formula over the word unpacker
        want = F.numpy_dequant(words, s, b, bits, gs, K).view(np.uint32)
    nan = np.isnan(want.view(np.float32))  # inf - inf: both sides must agree it is NaN
    assert np.array_equal(np.isnan(got.view(np.float32)), nan)
    assert np.array_equal(got[~nan], want[~nan])
    dw.free()
    dout.free()


def test_dequant_config0_bit_exact(ctx, orc):
    say("dequant cfg0 8192x2048")
    words, s, b = F.synthetic_affine(8192, 2048, 4, 64, seed=F.BASE_SEED)
    dw = DeviceAffine(ctx, words, s, b)
    dout = ctx.alloc(8192 * 2048 * 4)
    ctx.dequant_f32(dw.w, dw.s, dw.b, dout, 8192, 2048, 64, 4)
    ctx.sync()
    got = dout.download(np.uint32, 8192 * 2048)
    want = orc.dequantize(words, s, b, 8192, 2048, 4, 64).view(np.uint32).reshape(-1)
    assert np.array_equal(got, want)
    dw.free()
    dout.free()


# ---- qmv --------------------------------------------------------------------------------------

def _qmv_case(ctx, orc, M, K, N, bits, gs, seed, fn="qmv"):
    words, s, b = F.synthetic_affine(N, K, bits, gs, seed=seed)
    x = F.synthetic_x(M, K, seed=seed + 1)
    ref = F.reference_f64(x, words, s, b, bits, gs, K)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, gs, bits, True, fn)
    check_accumulators(acc, ref, "%s M=%d K=%d N=%d b=%d g=%d" % (fn, M, K, N, bits, gs))
    out = run_qmv(ctx, x, dw, M, K, N, gs, bits, False, fn)
    check_bf16_store(out, ref, "bf16 store")
    # the bf16 store is the RNE of the same accumulator
    assert np.array_equal(out, F.f32_to_bf16_bits(acc).reshape(M, N))
    dw.free()
    return acc, ref, (words, s, b, x)


def test_qmv_config0_vs_oracle(ctx, orc):
    """cfg 0: M=1, K=2048, N=8192, 4-bit g64 -- also against the reference's own CPU paths."""
    say("qmv cfg0")
    acc, ref, (words, s, b, x) = _qmv_case(ctx, orc, 1, 2048, 8192, 4, 64, F.BASE_SEED)
    xf = F.bf16_bits_to_f32(x).reshape(-1)
    fp32_ref = orc.hip_reference_projection(xf, words, s, b, 8192, 2048, 64, 4)       # fp32-accumulated
    host_ref = orc.matnt_quant_host(xf, words, s, b, 1, 2048, 8192, 64, 4).reshape(-1)  # matNTQuantHost
    check_accumulators(acc, fp32_ref, "vs hipReferenceMLXAffineProjection")
    check_accumulators(acc, host_ref, "vs matNTQuantHost")
    bf = orc.reference_affine_matvec(x, words, s, b, 8192, 2048, 64, 4).view(np.uint16)
    check_bf16_store(F.f32_to_bf16_bits(acc), F.bf16_bits_to_f32(bf).astype(np.float64), "vs ReferenceAffineMatVec")


@pytest.mark.parametrize("name,K,N", [("q", 4096, 4096), ("kv", 4096, 1024), ("gate_up", 4096, 14336), ("down", 14336, 4096)])
def test_qmv_config1_layer_shapes(ctx, orc, name, K, N):
    say("qmv cfg1", name)
    _qmv_case(ctx, orc, 1, K, N, 4, 64, F.BASE_SEED + 1)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M", [2, 3, 4, 8, 16, 32])
def test_qmv_config2_batched_rows(ctx, orc, bits, M):
    say("qmv cfg2", bits, M)
    _qmv_case(ctx, orc, M, 4096, 14336, bits, 64, F.BASE_SEED + 2)


@pytest.mark.parametrize("bits,gs,K,N,M", [(4, 64, 2816, 1408, 1), (4, 64, 1408, 2816, 1), (4, 64, 704, 17, 1), (4, 32, 256, 40, 1),
                                           (4, 128, 512, 24, 1), (8, 64, 512, 40, 1), (8, 32, 3072, 5, 1), (8, 128, 1024, 9, 2),
                                           (4, 64, 64, 3, 1), (4, 64, 512, 1, 4), (4, 64, 2048 + 64, 70, 3), (8, 64, 64, 2, 1)])
def test_qmv_ragged_and_thin_shapes(ctx, orc, bits, gs, K, N, M):
    say("qmv ragged", bits, gs, K, N, M)
    _qmv_case(ctx, orc, M, K, N, bits, gs, 77 + K + N)


@pytest.mark.parametrize("bits,gs,K,N,M", [(2, 64, 640, 9, 1), (3, 64, 256, 9, 1), (5, 64, 256, 9, 2), (6, 32, 192, 11, 1),
                                           (6, 16, 64, 5, 3), (4, 16, 64, 5, 1), (2, 128, 256, 24, 5),
                                           (6, 16, 1040, 33, 6), (6, 32, 4096, 70, 2), (6, 32, 1056, 7, 5), (6, 16, 16, 3, 1),
                                           (6, 64, 4096, 70, 1), (6, 64, 2112, 19, 3), (6, 128, 1280, 18, 4), (6, 64, 1088, 37, 7)])
def test_qmv_other_widths_generic_kernel(ctx, orc, bits, gs, K, N, M):
    say("qmv generic", bits, gs, K, N, M)
    rng = np.random.default_rng(bits * 100 + K)
    codes = rng.integers(0, 1 << bits, size=(N, K)).astype(np.uint32)
    words = F.pack_codes(codes, bits)
    _, s, b = F.synthetic_affine(N, K, 4, gs, seed=bits)
    x = F.synthetic_x(M, K, seed=bits + 5)
    ref = F.reference_f64(x, words, s, b, bits, gs, K)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, gs, bits, True)
    check_accumulators(acc, ref, "generic")
    # six-bit codes in groups of 16 / 32 (what GGUF Q6_K / Q5_K repack to) and 64 / 128 have a kernel of their own
    if bits == 6 and gs in (16, 32, 64, 128) and K % 16 == 0 and M <= 4:
        assert ctx.last_variant(0) == "qmv_six"
    else:                                # more than four rows go through the row-block loop, which reports its own name
        assert ctx.last_variant(0) in ("qmv_generic", "qmv_six")
    dw.free()


def _parse_variant(name):
    """-> (family, bits, rows it runs in one launch, gather)"""
    parts = dict((p.rstrip("0123456789"), int(p[len(p.rstrip("0123456789")):])) for p in name.split("_")[1:])
    if name.startswith("qmvb_"):
        return "blk", parts["b"], parts["m"], parts["g"]
    if name.startswith("qmvd_"):
        return "diag", parts["b"], parts["m"], parts["g"]
    if name.startswith("qmvt_"):
        return "tok", parts["b"], parts["m"], 0
    return "dot2", parts["b"], parts["m"], parts["g"]


def _blk_pieces(name):
    """K pieces per wavefront of a block-MFMA variant"""
    return int(name.split("_ki")[1].split("_")[0])


def test_qmv_every_variant(ctx, orc):
    """Each dot2 matvec kernel variant, forced, on a shape with a masked K tail (K = 44 group blocks) and ragged N."""
    import aq_mi355
    K, N = 2816, 150
    names = aq_mi355.variant_names(0)
    data = {}
    try:
        for idx, name in enumerate(names):
            fam, bits, m, gather = _parse_variant(name)
            if gather or fam != "dot2":
                continue  # covered by test_gather_every_variant and the other families' own tests
            say("variant", idx, name)
            if bits not in data:
                words, s, b = F.synthetic_affine(N, K, bits, 64, seed=500 + bits)
                x = F.synthetic_x(32, K, seed=600 + bits)
                data[bits] = (DeviceAffine(ctx, words, s, b), x, F.reference_f64(x, words, s, b, bits, 64, K))
            dw, x, ref = data[bits]
            ctx.force_variant(0, idx)
            acc = run_qmv(ctx, x[:m], dw, m, K, N, 64, bits, True)
            assert ctx.last_variant(0) == name
            check_accumulators(acc, ref[:m], name)
    finally:
        ctx.force_variant(0, -1)
    for dw, _, _ in data.values():
        dw.free()


def test_gather_every_variant(ctx, orc):
    """Each gather-capable kernel variant, forced, against the oracle (batched x, row_base slab offset)."""
    import aq_mi355
    names = aq_mi355.variant_names(0)
    E, routes, out_dim, in_dim, expert_rows, row_base = 4, 5, 40, 1408, 96, 32
    try:
        for idx, name in enumerate(names):
            fam, bits, m, gather = _parse_variant(name)
            if not gather or fam != "dot2":
                continue
            say("gather variant", idx, name)
            fx = F.gather_fixture(out_dim, in_dim, 64, bits, E, expert_rows, True, routes)
            # tame magnitudes: keep the fixture's codes, use benchmark-like scales
            _, s, b = F.synthetic_affine(E * expert_rows, in_dim, bits, 64, seed=40 + bits)
            fx["scales"], fx["biases"] = s, b
            ref64, _ = orc.gather_qmv(fx["x"], fx["x_rows"], fx["packed"], s, b, fx["lhs"], fx["rhs"], routes, E, expert_rows,
                                      row_base, out_dim, in_dim, 64, bits)
            ctx.force_variant(0, idx)
            acc, dw = _gather_run(ctx, fx, routes, E, expert_rows, row_base, out_dim, in_dim, 64, bits, True)
            assert ctx.last_variant(0) == name
            check_accumulators(acc, ref64, name)
            dw.free()
    finally:
        ctx.force_variant(0, -1)


def test_qmvb_every_variant(ctx, orc):
    """Each block-MFMA matvec variant, forced: K = 3 (4 bit) or 4 (8 bit) wavefronts x its pieces per wavefront, a row count
    that leaves the last round of workgroups ragged, the most activation rows it takes and one fewer."""
    import aq_mi355
    names = aq_mi355.variant_names(0)
    N = 4 * 523
    data = {}
    try:
        for idx, name in enumerate(names):
            fam, bits, m, gather = _parse_variant(name)
            if fam != "blk" or gather:
                continue
            ki = _blk_pieces(name)
            K = 1536 * ki if bits == 4 else 1024 * ki
            say("variant", idx, name, "K", K)
            if (bits, K) not in data:
                words, s, b = F.synthetic_affine(N, K, bits, 64, seed=510 + bits + ki)
                x = F.synthetic_x(16, K, seed=610 + bits + ki)
                data[(bits, K)] = (DeviceAffine(ctx, words, s, b), x, F.reference_f64(x, words, s, b, bits, 64, K))
            dw, x, ref = data[(bits, K)]
            ctx.force_variant(0, idx)
            for rows in sorted({m, max(1, m - 1)}):
                acc = run_qmv(ctx, x[:rows], dw, rows, K, N, 64, bits, True)
                assert ctx.last_variant(0) == name
                check_accumulators(acc, ref[:rows], "%s rows=%d" % (name, rows))
            # a shape outside the family is refused, not silently rerouted
            with pytest.raises(aq_mi355.AqError) as ei:
                run_qmv(ctx, x[:1, :K - 64], dw, 1, K - 64, N, 64, bits, True)
            assert ei.value.code == aq_mi355.AQ_ERR_ARG
    finally:
        ctx.force_variant(0, -1)
    for dw, _, _ in data.values():
        dw.free()


@pytest.mark.parametrize("M,K,N,gs,bits", [
    (2, 4096, 1024, 64, 4), (5, 4096, 1024, 64, 4), (16, 2048, 516, 64, 4), (24, 1024, 256, 64, 4),
    (3, 2048, 512, 32, 4), (4, 2048, 512, 128, 4), (7, 1024, 512, 64, 8), (2, 2048, 256, 32, 8),
    (4, 14336, 256, 64, 4), (9, 14336, 64, 64, 4)])
def test_qmv_small_m_default_path(ctx, orc, M, K, N, gs, bits):
    """2..24 activation rows through aq_qmv with nothing forced: fp32 outputs against the float64
    reference, bf16 stores against its rounding, over the group sizes and widths the block-MFMA
    family takes (and shapes that need several launches, or fall through to another family)."""
    say("small-M default", M, K, N, gs, bits)
    words, s, b = F.synthetic_affine(N, K, bits, gs, seed=77 + M)
    x = F.synthetic_x(M, K, seed=78 + M)
    ref = F.reference_f64(x, words, s, b, bits, gs, K)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, gs, bits, True)
    say("  ran on", ctx.last_variant(0), ctx.last_variant(1))
    check_accumulators(acc, ref, "small-M f32")
    out = run_qmv(ctx, x, dw, M, K, N, gs, bits, False)
    check_bf16_store(out, ref, "small-M bf16")
    dw.free()


def test_qmv_block_family_many_batches(ctx, orc):
    """A matrix tall enough that every workgroup of the block-MFMA kernel walks more row groups than one
    batch of staged scales holds (K = 512: one wavefront per workgroup, 4096 workgroups)."""
    M, K, N = 3, 512, 4 * 4096 * 19 + 8
    say("many batches", M, K, N)
    # (groups of 128: few rows of group-64 codes go to the kernels whose rows carry the bytes of single-row calls)
    words, s, b = F.synthetic_affine(N, K, 4, 128, seed=5)
    x = F.synthetic_x(M, K, seed=6)
    ref = F.reference_f64(x, words, s, b, 4, 128, K)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, 128, 4, True)
    assert ctx.last_variant(0).startswith("qmvb_"), ctx.last_variant(0)
    check_accumulators(acc, ref, "many batches")
    dw.free()


def test_qmvd_every_variant(ctx, orc):
    """Each diagonal-MFMA matvec variant, forced: 1..4 (1..8) activation rows, K = all the steps of 1024 codes (512 of
    8 bits) its wavefronts take and one step fewer (an idle wavefront), a last step of three chunks and of one chunk,
    a last chunk that is a single half of 128 codes (4 bit), ragged N; fp32 and bf16 stores; a K that is no multiple
    of 128, or more steps than the variant takes, is refused."""
    import aq_mi355
    names = aq_mi355.variant_names(0)
    N = 150
    data = {}
    try:
        for idx, name in enumerate(names):
            fam, bits, m, gather = _parse_variant(name)
            if fam != "diag" or gather:
                continue
            waves = int(name.split("_w")[1].split("_")[0])
            steps = waves * int(name.split("_d")[1].split("_")[0])
            wg_waves = waves * int(name.split("_r")[1].split("_")[0])
            unit = 256 if bits == 4 else 128              # codes of a chunk (128 bytes of a row)
            step = (3 if name.endswith("_c3") else 4) * unit  # codes per wavefront step
            gs = 32 if "_s32" in name else 64             # (group 32: K in whole chunks of 256 codes)
            ks = {step * steps, step * max(1, steps - 1), step * steps - unit, step * (steps - 1) + unit}
            if bits == 4:
                ks |= {step * steps - 128, step * (steps - 1) + 128}  # a last chunk of one half (8 bit: K in whole chunks)
            for K in sorted(ks):
                if gs == 32 and K % 256:
                    continue
                say("variant", idx, name, "K", K)
                if (K, gs, bits) not in data:
                    words, s, b = F.synthetic_affine(N, K, bits, gs, seed=530 + K // 128)
                    x = F.synthetic_x(8, K, seed=630 + K // 128)
                    data[(K, gs, bits)] = (DeviceAffine(ctx, words, s, b), x, F.reference_f64(x, words, s, b, bits, gs, K))
                dw, x, ref = data[(K, gs, bits)]
                ctx.force_variant(0, idx)
                for rows in ((1, 2) if m == 2 else (1, 2, 3, 4) if m == 4 else (1, 4, 5, 7, 8)):
                    k_steps = -(-(-(-K // unit)) // (3 if name.endswith("_c3") else 4))
                    lds_limit = (96 if k_steps <= 4 else 156) * 1024
                    sums = 96 if gs == 32 else 48 if bits == 4 else 32
                    if rows * K * 2 + rows * ((K + unit - 1) // unit) * sums + 128 + wg_waves * max(1, m // 4) * 256 > lds_limit:
                        # the activations of all rows and their group sums sit in LDS: beyond 96 KiB (two workgroups a
                        # CU; 156 KiB for K of more than four steps) the variant refuses
                        with pytest.raises(aq_mi355.AqError) as ei:
                            run_qmv(ctx, x[:rows], dw, rows, K, N, gs, bits, True)
                        assert ei.value.code == aq_mi355.AQ_ERR_ARG
                        continue
                    acc = run_qmv(ctx, x[:rows], dw, rows, K, N, gs, bits, True)
                    assert ctx.last_variant(0) == name
                    check_accumulators(acc, ref[:rows], "%s rows=%d" % (name, rows))
                out = run_qmv(ctx, x[:2], dw, 2, K, N, gs, bits, False)
                check_bf16_store(out, ref[:2], name)
            dw, x, ref = data[(step * steps, gs, bits)]
            for bad_k in (step * steps - 64, step * steps + unit):
                with pytest.raises(aq_mi355.AqError) as ei:
                    run_qmv(ctx, np.zeros((1, bad_k), np.uint16), dw, 1, bad_k, N, gs, bits, True)
                assert ei.value.code == aq_mi355.AQ_ERR_ARG
    finally:
        ctx.force_variant(0, -1)
    for dw, _, _ in data.values():
        dw.free()


def test_qmvd_gather_every_variant(ctx, orc):
    """Each gathered diagonal-MFMA variant, forced and as the default: K = all the steps its wavefronts take, a last
    chunk that is a single half of 128 codes, a last step of one chunk; batched x, a row_base inside the slab, ragged
    N, an expert id out of range (zeros for that route)."""
    import aq_mi355
    names = aq_mi355.variant_names(0)
    E, routes, out_dim, expert_rows, row_base = 4, 6, 40, 96, 32
    try:
        for idx, name in enumerate(names):
            fam, bits, m, gather = _parse_variant(name)
            if fam != "diag" or not gather:
                continue
            steps = int(name.split("_w")[1].split("_")[0]) * int(name.split("_d")[1].split("_")[0])
            step = 768 if name.endswith("_c3") else 1024
            for K in sorted({step * steps, step * steps - 128, step * (steps - 1) + 256, step * (steps - 1) + 128}):
                say("gather variant", idx, name, "K", K)
                fx = F.gather_fixture(out_dim, K, 64, bits, E, expert_rows, True, routes)
                _, s, b = F.synthetic_affine(E * expert_rows, K, bits, 64, seed=41 + bits)
                fx["scales"], fx["biases"] = s, b
                fx["rhs"] = fx["rhs"].copy()
                fx["rhs"][4] = E + 3  # no such expert
                ok = [z for z in range(routes) if z != 4]
                ref64, _ = orc.gather_qmv(fx["x"], fx["x_rows"], fx["packed"], s, b, fx["lhs"][ok], fx["rhs"][ok], len(ok), E,
                                          expert_rows, row_base, out_dim, K, 64, bits)
                for forced in (True, False):
                    ctx.force_variant(0, idx if forced else -1)
                    acc, dw = _gather_run(ctx, fx, routes, E, expert_rows, row_base, out_dim, K, 64, bits, True)
                    if forced:
                        assert ctx.last_variant(0) == name
                    elif K > 1024:
                        assert ctx.last_variant(0).startswith("qmvd_") and "_g1" in ctx.last_variant(0), ctx.last_variant(0)
                    check_accumulators(acc[ok], ref64, name)
                    assert np.all(acc[4] == 0)
                    dw.free()
                ctx.force_variant(0, idx)
            fx = F.gather_fixture(out_dim, step * steps + 128, 64, bits, E, expert_rows, True, routes)
            with pytest.raises(aq_mi355.AqError) as ei:
                _gather_run(ctx, fx, routes, E, expert_rows, row_base, out_dim, step * steps + 128, 64, bits, True)
            assert ei.value.code == aq_mi355.AQ_ERR_ARG
    finally:
        ctx.force_variant(0, -1)


def test_qmvd_is_the_default_for_few_rows(ctx, orc):
    """4-bit group-64 codes: 1..8 activation rows with K of 2..16 steps of 1024 codes land on the diagonal-MFMA kernels
    without forcing (beyond four steps: up to four rows a launch), rows beyond the last full 16 included; other K do
    not (8-bit codes: tests/test_gpu_diag8.py)."""
    for K, N in ((4096, 16 * 9 + 5), (3072, 64), (2048, 33)):
        words, s, b = F.synthetic_affine(N, K, 4, 64, seed=810 + K // 1024)
        x = F.synthetic_x(8, K, seed=820 + K // 1024)
        ref = F.reference_f64(x, words, s, b, 4, 64, K)
        dw = DeviceAffine(ctx, words, s, b)
        for rows in (1, 2, 3, 4, 5, 8):
            say("default few rows", K, N, rows)
            acc = run_qmv(ctx, x[:rows], dw, rows, K, N, 64, 4, True)
            assert ctx.last_variant(0).startswith("qmvd_"), ctx.last_variant(0)
            check_accumulators(acc, ref[:rows], "diag default K=%d rows=%d" % (K, rows))
            out = run_qmv(ctx, x[:rows], dw, rows, K, N, 64, 4, False)
            check_bf16_store(out, ref[:rows], "diag default bf16 K=%d rows=%d" % (K, rows))
        dw.free()
    for K in (5120, 7168, 14336, 16384, 2816, 11008, 1280, 1408, 2944):
        words, s, b = F.synthetic_affine(40, K, 4, 64, seed=840 + K // 1024)
        x = F.synthetic_x(1, K, seed=850 + K // 1024)
        dw = DeviceAffine(ctx, words, s, b)
        say("default one row", K)
        acc = run_qmv(ctx, x, dw, 1, K, 40, 64, 4, True)
        assert ctx.last_variant(0).startswith("qmvd_"), ctx.last_variant(0)
        check_accumulators(acc, F.reference_f64(x, words, s, b, 4, 64, K), "diag default K=%d" % K)
        dw.free()
    for K in (1536, 4096, 3072):  # group 32: up to two rows
        words, s, b = F.synthetic_affine(70, K, 4, 32, seed=860 + K // 256)
        x = F.synthetic_x(2, K, seed=870 + K // 256)
        ref = F.reference_f64(x, words, s, b, 4, 32, K)
        dw = DeviceAffine(ctx, words, s, b)
        for rows in (1, 2):
            say("default group 32", K, rows)
            acc = run_qmv(ctx, x[:rows], dw, rows, K, 70, 32, 4, True)
            assert ctx.last_variant(0).startswith("qmvd_") and "_s32" in ctx.last_variant(0), ctx.last_variant(0)
            check_accumulators(acc, ref[:rows], "diag g32 K=%d rows=%d" % (K, rows))
        dw.free()
    for K, rows in ((8192, 2), (14336, 4), (14336, 7), (16384, 8), (11008, 3)):
        words, s, b = F.synthetic_affine(40, K, 4, 64, seed=880 + K // 1024)
        x = F.synthetic_x(rows, K, seed=881 + K // 1024)
        dw = DeviceAffine(ctx, words, s, b)
        say("default rows at a long K", K, rows)
        acc = run_qmv(ctx, x, dw, rows, K, 40, 64, 4, True)
        assert ctx.last_variant(0).startswith("qmvd_b4_m4_"), ctx.last_variant(0)
        check_accumulators(acc, F.reference_f64(x, words, s, b, 4, 64, K), "diag default K=%d rows=%d" % (K, rows))
        dw.free()
    for K, bits, rows in ((17408, 4, 1), (1024, 4, 1), (3072, 8, 1), (17408, 4, 2), (2880, 4, 1)):
        words, s, b = F.synthetic_affine(32, K, bits, 64, seed=830)
        x = F.synthetic_x(rows, K, seed=831)
        dw = DeviceAffine(ctx, words, s, b)
        acc = run_qmv(ctx, x, dw, rows, K, 32, 64, bits, True)
        assert not ctx.last_variant(0).startswith("qmvd_"), ctx.last_variant(0)
        check_accumulators(acc, F.reference_f64(x, words, s, b, bits, 64, K), "not diag K=%d bits=%d" % (K, bits))
        dw.free()


def test_qmvd_default_paths_random_shapes(ctx, orc):
    """The library's own choice over seeded random shapes the diagonal-MFMA kernels take: K any multiple of 128 (group
    32: 256) from 1152 to 16384, ragged N, 1..8 (group 32: 1..2) activation rows; plain, multi-matrix and fused gate|up
    calls, each against the float64 reference, and the byte-identity contracts between them."""
    import aq_mi355
    rng = np.random.default_rng(20240607)
    for case in range(28):
        gs = 32 if case % 4 == 3 else 64
        K = int(rng.integers(1152 // 128, 16384 // 128 + 1)) * 128
        if gs == 32:
            K = max(1280, K // 256 * 256)
        if case % 7 == 0:
            K = int(rng.choice([2816, 1408, 3584, 5120, 11008, 14336]))
            gs = 64
        M = int(rng.integers(1, 3 if gs == 32 else 9))
        if K > 4096 and M > 1:
            M = 1 if gs == 64 else M
        N = int(rng.integers(1, 300))
        say("random diag shape", case, "K", K, "N", N, "M", M, "group", gs)
        words, s, b = F.synthetic_affine(N, K, 4, gs, seed=9000 + case)
        x = F.synthetic_x(M, K, seed=9100 + case)
        ref = F.reference_f64(x, words, s, b, 4, gs, K)
        dw = DeviceAffine(ctx, words, s, b)
        acc = run_qmv(ctx, x, dw, M, K, N, gs, 4, True)
        name = ctx.last_variant(0)
        if not (gs == 32 and K > 8192):
            assert name.startswith("qmvd_"), (name, K, N, M, gs)
        check_accumulators(acc, ref, "random shape %d (%s)" % (case, name))
        out = run_qmv(ctx, x, dw, M, K, N, gs, 4, False)
        assert np.array_equal(out, F.f32_to_bf16_bits(acc).reshape(M, N)), "bf16 store is not the RNE of the accumulator"
        # every row on its own: the same bytes
        if M > 1:
            one = run_qmv(ctx, x[M - 1:M], dw, 1, K, N, gs, 4, True)
            assert np.array_equal(one[0].view(np.uint32), acc[M - 1].view(np.uint32)), (K, N, M, gs)
        if gs == 64 and M <= 4:
            # two matrices in one launch, and the fused gate|up of the same two
            w2, s2, b2 = F.synthetic_affine(N, K, 4, gs, seed=9200 + case)
            dw2 = DeviceAffine(ctx, w2, s2, b2)
            dx = ctx.to_device(x)
            ys = [ctx.alloc(M * N * 4), ctx.alloc(M * N * 4)]
            ctx.qmv_multi(dx, [dw.w, dw2.w], [dw.s, dw2.s], [dw.b, dw2.b], ys, [N, N], M, K, gs, 4, aq_mi355.AQ_OUT_F32)
            ctx.sync()
            m0 = ys[0].download(np.float32, M * N).reshape(M, N)
            m1 = ys[1].download(np.float32, M * N).reshape(M, N)
            assert np.array_equal(m0.view(np.uint32), acc.view(np.uint32)), ("multi member 0", K, N, M)
            acc2 = run_qmv(ctx, x, dw2, M, K, N, gs, 4, True)
            assert np.array_equal(m1.view(np.uint32), acc2.view(np.uint32)), ("multi member 1", K, N, M)
            check_accumulators(acc2, F.reference_f64(x, w2, s2, b2, 4, gs, K), "random shape %d, second matrix" % case)
            for t in ys + [dx]:
                t.free()
            dw2.free()
        dw.free()


def test_qmvb_gather_every_variant(ctx, orc):
    """Each gather-capable block-MFMA variant, forced, against the oracle (batched x, row_base slab
    offset)."""
    import aq_mi355
    names = aq_mi355.variant_names(0)
    E, routes, out_dim, expert_rows, row_base = 4, 6, 40, 96, 32
    try:
        for idx, name in enumerate(names):
            fam, bits, m, gather = _parse_variant(name)
            if fam != "blk" or not gather:
                continue
            in_dim = (512 if bits == 4 else 256) * _blk_pieces(name) * 2
            say("gather variant", idx, name, "K", in_dim)
            fx = F.gather_fixture(out_dim, in_dim, 64, bits, E, expert_rows, True, routes)
            _, s, b = F.synthetic_affine(E * expert_rows, in_dim, bits, 64, seed=40 + bits)
            fx["scales"], fx["biases"] = s, b
            ref64, _ = orc.gather_qmv(fx["x"], fx["x_rows"], fx["packed"], s, b, fx["lhs"], fx["rhs"], routes, E, expert_rows,
                                      row_base, out_dim, in_dim, 64, bits)
            ctx.force_variant(0, idx)
            acc, dw = _gather_run(ctx, fx, routes, E, expert_rows, row_base, out_dim, in_dim, 64, bits, True)
            assert ctx.last_variant(0) == name
            check_accumulators(acc, ref64, name)
            dw.free()
    finally:
        ctx.force_variant(0, -1)


def test_qmv_rows_match_single_row_bytes(ctx, orc):
    """M-row qmv is byte-identical, row by row, to M single-row calls
    (the contract of go/engine/metal/qmv_rows_test.go:31-100)."""
    say("qmv rows == per-row")
    K, N = 2048, 520
    words, s, b = F.synthetic_affine(N, K, 4, 64, seed=91)
    x = F.synthetic_x(4, K, seed=92)
    dw = DeviceAffine(ctx, words, s, b)
    for M in (2, 3, 4):
        both = run_qmv(ctx, x[:M], dw, M, K, N, 64, 4, False)
        for m in range(M):
            one = run_qmv(ctx, x[m:m + 1], dw, 1, K, N, 64, 4, False)
            assert np.array_equal(both[m], one[0]), (M, m)
    dw.free()


def test_concat_rows_is_byte_identical(ctx, orc):
    """gate||up as one matvec equals the two matvecs (go/model/quant_weight.go:32-44)."""
    say("concat rows")
    K = 1024
    wa, sa, ba = F.synthetic_affine(96, K, 4, 64, seed=31)
    wb, sb_, bb = F.synthetic_affine(160, K, 4, 64, seed=32)
    x = F.synthetic_x(1, K, seed=33)
    da, db = DeviceAffine(ctx, wa, sa, ba), DeviceAffine(ctx, wb, sb_, bb)
    dc = DeviceAffine(ctx, np.concatenate([wa, wb]), np.concatenate([sa, sb_]), np.concatenate([ba, bb]))
    ya = run_qmv(ctx, x, da, 1, K, 96, 64, 4, False)
    yb = run_qmv(ctx, x, db, 1, K, 160, 64, 4, False)
    yc = run_qmv(ctx, x, dc, 1, K, 256, 64, 4, False)
    assert np.array_equal(yc[0, :96], ya[0]) and np.array_equal(yc[0, 96:], yb[0])
    for d in (da, db, dc):
        d.free()


@pytest.mark.parametrize("M,bits,Ns,K", [(1, 4, (96, 160, 40), 1024), (1, 4, (4096, 1024, 1024), 1024), (1, 4, (50,), 1024),
                                          (1, 4, (7, 9, 300, 64), 1024), (2, 4, (96, 160), 1024), (1, 8, (64, 200), 1024),
                                          (1, 4, (96, 0, 32), 1024), (1, 4, (96, 160, 40), 2048), (1, 4, (4096, 1024, 1030), 4096),
                                          (1, 4, (7, 300), 3072), (2, 4, (96, 160), 4096), (1, 8, (64, 200), 4096),
                                          (4, 4, (4096, 1024, 1030), 4096), (3, 4, (50, 40, 33, 20), 2816), (5, 4, (96, 160), 4096)])
def test_qmv_multi_matches_separate_calls(ctx, orc, M, bits, Ns, K):
    """aq_qmv_multi (q|k|v, gate|up in one launch) is byte-identical to one aq_qmv per matrix, the
    contract ConcatQuantRows states (go/model/quant_weight.go:32-44); members that the fused kernels
    do not take (more rows, 8 bit, empty) run as separate launches behind the same call."""
    import aq_mi355
    say("qmv multi", M, bits, Ns, K)
    x = F.synthetic_x(M, K, seed=333)
    dx = ctx.to_device(x)
    mats = [F.synthetic_affine(max(n, 1), K, bits, 64, seed=340 + i) for i, n in enumerate(Ns)]
    dws = [DeviceAffine(ctx, *m) for m in mats]
    for f32 in (False, True):
        esz = 4 if f32 else 2
        ys = [ctx.alloc(max(M * n, 1) * esz) for n in Ns]
        for t in ys:
            ctx.fill_zero(t)
        ctx.qmv_multi(dx, [d.w for d in dws], [d.s for d in dws], [d.b for d in dws], ys, list(Ns), M, K, 64, bits,
                      aq_mi355.AQ_OUT_F32 if f32 else 0)
        ctx.sync()
        fused_name = ctx.last_variant(0)
        for i, n in enumerate(Ns):
            if n == 0:
                continue
            got = ys[i].download(np.float32 if f32 else np.uint16, M * n).reshape(M, n)
            want = run_qmv(ctx, x, dws[i], M, K, n, 64, bits, f32)
            assert np.array_equal(got.view(np.uint32 if f32 else np.uint16), want.view(np.uint32 if f32 else np.uint16)), (i, n, f32)
            ref = F.reference_f64(x, mats[i][0][:n], mats[i][1][:n], mats[i][2][:n], bits, 64, K)
            if f32:
                check_accumulators(got, ref, "multi member %d" % i)
        if bits == 4 and all(n > 0 for n in Ns) and (M == 1 or (M <= 4 and K > 1024)):
            # K beyond one step of 1024 codes goes to the diagonal-MFMA kernels (up to four rows), like the single calls
            assert fused_name == ("qmv_multi_diag" if K > 1024 else "qmv_multi_dot2"), fused_name
        else:
            assert not fused_name.startswith("qmv_multi"), fused_name
        for t in ys:
            t.free()
    with pytest.raises(aq_mi355.AqError):
        ctx.qmv_multi(dx, [d.w for d in dws] * 5, [d.s for d in dws] * 5, [d.b for d in dws] * 5, [dx] * (5 * len(Ns)),
                      list(Ns) * 5, M, K, 64, bits, 0)
    dx.free()
    for d in dws:
        d.free()


def test_qmv_zero_sized_and_errors(ctx):
    import aq_mi355
    say("qmv zero/err")
    ctx.qmv(None, None, None, None, None, 1, 0, 8, 64, 4)   # K == 0: no-op
    ctx.qmv(None, None, None, None, None, 1, 64, 0, 64, 4)  # N == 0: no-op
    buf = ctx.alloc(4096)
    for kw, code in [(dict(K=64, gs=3), aq_mi355.AQ_ERR_SHAPE), (dict(K=64, bits=0), aq_mi355.AQ_ERR_UNSUPPORTED),
                     (dict(K=64, bits=9), aq_mi355.AQ_ERR_UNSUPPORTED), (dict(K=7, gs=7), aq_mi355.AQ_ERR_SHAPE),
                     (dict(K=-1), aq_mi355.AQ_ERR_SHAPE)]:
        with pytest.raises(aq_mi355.AqError) as e:
            ctx.qmv(buf, buf, buf, buf, buf, 1, kw.get("K", 64), 4, kw.get("gs", 64), kw.get("bits", 4))
        assert e.value.code == code, kw
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.qmv(None, buf, buf, buf, buf, 1, 64, 4, 64, 4)
    assert e.value.code == aq_mi355.AQ_ERR_ARG
    buf.free()


# ---- gather_qmv -------------------------------------------------------------------------------

def _gather_run(ctx, fx, routes, E, expert_rows, row_base, N, K, gs, bits, f32):
    import aq_mi355
    dx = ctx.to_device(fx["x"])
    dw = DeviceAffine(ctx, fx["packed"], fx["scales"], fx["biases"])
    dl = ctx.to_device(fx["lhs"]) if fx["lhs"] is not None else None
    dr = ctx.to_device(fx["rhs"])
    dy = ctx.alloc(routes * N * (4 if f32 else 2))
    ctx.fill_zero(dy)
    ctx.gather_qmv(dx, dw.w, dw.s, dw.b, dl, dr, dy, routes, fx["x_rows"], K, N, E, expert_rows, row_base, gs, bits,
                   aq_mi355.AQ_OUT_F32 if f32 else 0)
    ctx.sync()
    out = dy.download(np.float32 if f32 else np.uint16, routes * N).reshape(routes, N)
    for t in (dx, dl, dr, dy):
        if t is not None:
            t.free()
    return out, dw


@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
@pytest.mark.parametrize("name,out_dim,in_dim,gs,expert_rows,row_base,batched", [
    ("fast shared-x", 32, 512, 64, 32, 0, False), ("fast batched-x", 32, 512, 64, 32, 0, True),
    ("plain shared-x", 24, 256, 32, 24, 0, False), ("fast gate_up rowBase", 32, 512, 64, 64, 32, False)])
def test_gather_reference_cases(ctx, orc, bits, name, out_dim, in_dim, gs, expert_rows, row_base, batched):
    """The sweep of go/engine/metal/qmv_gather_test.go:87-129, device vs oracle, and byte-identity with the
    plain qmv on the expert slice (go/engine/metal/moe_quant_test.go:1143-1185)."""
    if in_dim * bits % 32:
        pytest.skip("packed-row alignment")
    say("gather", bits, name)
    E, routes = 4, 3
    fx = F.gather_fixture(out_dim, in_dim, gs, bits, E, expert_rows, batched, routes)
    ref64, _ = orc.gather_qmv(fx["x"], fx["x_rows"], fx["packed"], fx["scales"], fx["biases"], fx["lhs"], fx["rhs"], routes, E,
                              expert_rows, row_base, out_dim, in_dim, gs, bits)
    acc, dw = _gather_run(ctx, fx, routes, E, expert_rows, row_base, out_dim, in_dim, gs, bits, True)
    # these fixtures have |w| up to ~400 and outputs up to ~1e4: the stated bounds are relative to that scale
    scale = max(1.0, np.abs(ref64).max())
    check_accumulators(acc / scale, ref64 / scale, "gather f32")
    out, dw2 = _gather_run(ctx, fx, routes, E, expert_rows, row_base, out_dim, in_dim, gs, bits, False)
    assert np.array_equal(out, F.f32_to_bf16_bits(acc).reshape(routes, out_dim))
    # sliced plain qmv gives the same bytes
    wpr, gpr = in_dim * bits // 32, in_dim // gs
    W = fx["packed"].reshape(E, expert_rows, wpr)
    S = fx["scales"].reshape(E, expert_rows, gpr)
    B = fx["biases"].reshape(E, expert_rows, gpr)
    X = fx["x"].reshape(fx["x_rows"], in_dim)
    for z in range(routes):
        e = fx["rhs"][z]
        sl = slice(row_base, row_base + out_dim)
        ds = DeviceAffine(ctx, W[e, sl], S[e, sl], B[e, sl])
        xr = X[fx["lhs"][z]] if batched else X[0]
        one = run_qmv(ctx, xr.reshape(1, -1), ds, 1, in_dim, out_dim, gs, bits, False)
        assert np.array_equal(one[0], out[z]), (name, z)
        ds.free()
    dw.free()
    dw2.free()


def test_gather_config4_shape(ctx, orc):
    """cfg 4 geometry at a reduced expert count: 8 tokens x top-8 of 16 experts, in-proj [1408 x 2816]
    with lhs = route -> token, then down [2816 x 1408] with lhs = iota."""
    rng = np.random.default_rng(F.BASE_SEED + 4)
    E, tokens, topk = 16, 8, 8
    routes = tokens * topk
    ids = np.concatenate([rng.permutation(E)[:topk] for _ in range(tokens)]).astype(np.int32)
    for (N, K, lhs, x_rows) in [(1408, 2816, np.repeat(np.arange(tokens), topk).astype(np.int32), tokens),
                                (2816, 1408, np.arange(routes, dtype=np.int32), routes)]:
        say("gather cfg4", N, K)
        words, s, b = F.synthetic_affine(E * N, K, 4, 64, seed=F.BASE_SEED + 40 + N)
        x = F.synthetic_x(x_rows, K, seed=F.BASE_SEED + 41 + N)
        fx = dict(x=x, x_rows=x_rows, packed=words, scales=s, biases=b, lhs=lhs, rhs=ids)
        acc, dw = _gather_run(ctx, fx, routes, E, N, 0, N, K, 64, 4, True)
        wq = F.numpy_dequant(words, s, b, 4, 64, K).astype(np.float64).reshape(E, N, K)
        xf = F.bf16_bits_to_f32(x).astype(np.float64).reshape(x_rows, K)
        ref = np.stack([wq[ids[z]] @ xf[lhs[z]] for z in range(routes)])
        check_accumulators(acc, ref, "gather cfg4")
        # a subset of routes against the oracle itself
        sub = [0, 17, 63]
        r64, _ = orc.gather_qmv(x, x_rows, words, s, b, lhs[sub], ids[sub], len(sub), E, N, 0, N, K, 64, 4)
        check_accumulators(acc[sub], r64, "gather cfg4 vs oracle")
        dw.free()


def test_gather_out_of_range_ids_give_zeros(ctx):
    say("gather bad ids")
    fx = F.gather_fixture(32, 512, 64, 4, 4, 32, False, 3)
    fx["rhs"] = np.array([1, 9, -2], dtype=np.int32)
    out, dw = _gather_run(ctx, fx, 3, 4, 32, 0, 32, 512, 64, 4, True)
    assert np.all(out[1] == 0) and np.all(out[2] == 0) and np.any(out[0] != 0)
    dw.free()


def test_gather_errors(ctx):
    import aq_mi355
    buf = ctx.alloc(4096)
    with pytest.raises(aq_mi355.AqError) as e:
        ctx.gather_qmv(buf, buf, buf, buf, None, buf, buf, 3, 1, 64, 8, 4, 8, 4, 64, 4)  # row_base+N > expert_rows
    assert e.value.code == aq_mi355.AQ_ERR_SHAPE
    ctx.gather_qmv(buf, buf, buf, buf, None, buf, buf, 0, 1, 64, 8, 4, 8, 0, 64, 4)      # zero routes: no-op
    buf.free()


# ---- qmm --------------------------------------------------------------------------------------

@pytest.mark.parametrize("M,K,N,bits,gs", [(3, 512, 64, 4, 64), (5, 256, 40, 4, 64), (2, 128, 8, 8, 64), (33, 1024, 130, 4, 64),
                                           (64, 512, 256, 8, 64), (100, 2816, 96, 4, 64), (17, 704, 17, 4, 64), (40, 1408, 70, 4, 128),
                                           (130, 384, 33, 8, 128), (256, 1024, 512, 4, 64),
                                           # more than 64 rows, few 128 x 128 tiles, long K: K shared out over workgroups
                                           (130, 2048, 200, 4, 64), (100, 4096, 520, 8, 64), (200, 6144, 130, 4, 128)])
def test_qmm_small_cases(ctx, orc, M, K, N, bits, gs):
    say("qmm", M, K, N, bits, gs)
    _qmv_case(ctx, orc, M, K, N, bits, gs, 900 + M + N, fn="qmm")


def test_qmm_every_variant(ctx, orc):
    import aq_mi355
    names = aq_mi355.variant_names(1)
    M, N = 150, 200
    data = {}
    try:
        for idx, name in enumerate(names):
            say("qmm variant", idx, name)
            bits = int(name.split("_")[1][1:])
            # variants that stage scales through LDS take K in multiples of 512 (1536: three quads, the last
            # octet half used); the others get a K that ends in the middle of a quad
            staged = name.endswith("_q") or name.endswith("_pq")
            K = 1536 if staged else 704
            if (bits, K) not in data:
                words, s, b = F.synthetic_affine(N, K, bits, 64, seed=700 + bits)
                x = F.synthetic_x(M, K, seed=800 + bits)
                data[(bits, K)] = (DeviceAffine(ctx, words, s, b), x, F.reference_f64(x, words, s, b, bits, 64, K))
            dw, x, ref = data[(bits, K)]
            ctx.force_variant(1, idx)
            acc = run_qmv(ctx, x, dw, M, K, N, 64, bits, True, "qmm")
            assert ctx.last_variant(1) == name
            check_accumulators(acc, ref, name)
            if staged:
                with pytest.raises(aq_mi355.AqError):      # a K the staging cannot take is refused, not mangled
                    run_qmv(ctx, x[:, :704].copy(), dw, M, 704, N, 64, bits, True, "qmm")
    finally:
        ctx.force_variant(1, -1)
    for dw, _, _ in data.values():
        dw.free()


@pytest.mark.parametrize("fn", ["qmv", "qmm"])
@pytest.mark.parametrize("M,K,N,bits", [(5, 256, 70, 4), (17, 1024, 130, 4), (32, 4096, 1000, 4), (33, 2048, 516, 8),
                                        (64, 4096, 257, 4), (48, 14336, 96, 4), (20, 768, 64, 8), (64, 512, 40, 4)])
def test_few_rows_k_shared_over_workgroups(ctx, orc, fn, M, K, N, bits):
    """5..64 activation rows: the tile kernels share K out over several workgroups per output tile and a
    second kernel adds the fp32 partial tiles in a fixed order.  Through both doors, fp32 and bf16 stores,
    widths 4 and 8, N that ends inside a tile, K whose group count allows 1, 2, 4 .. 16 splits; two calls
    give the same bytes (the order of the additions does not depend on which workgroup finishes first)."""
    say("few rows, split K", fn, M, K, N, bits)
    acc, ref, (words, s, b, x) = _qmv_case(ctx, orc, M, K, N, bits, 64, 4000 + M + K, fn=fn)
    say("  ran on", ctx.last_variant(0), ctx.last_variant(1))
    if M > 32 and fn == "qmv":
        assert ctx.last_variant(1).startswith("qmm"), ctx.last_variant(1)
    dw = DeviceAffine(ctx, words, s, b)
    again = run_qmv(ctx, x, dw, M, K, N, 64, bits, True, fn)
    assert np.array_equal(again.view(np.uint32), acc.view(np.uint32))
    dw.free()


def test_few_rows_call_in_a_graph_after_reserving_workspace(orc):
    """A matmul call with 32 rows keeps fp32 partial tiles in the context's workspace.  On a fresh context the workspace
    cannot grow while a capture is open: the call is refused with an error, not mangled; after
    aq_reserve_workspace_bytes the same call is captured and every replay equals the eager result."""
    import aq_mi355
    M, K, N = 32, 2048, 1000
    say("few rows in a graph", M, K, N)
    words, s, b = F.synthetic_affine(N, K, 4, 64, seed=931)
    x = F.synthetic_x(M, K, seed=932)
    ref = F.reference_f64(x, words, s, b, 4, 64, K)
    fresh = aq_mi355.Context(0)
    try:
        dw = DeviceAffine(fresh, words, s, b)
        dx, dy = fresh.to_device(x), fresh.alloc(M * N * 4)
        fresh.capture_begin()
        with pytest.raises(aq_mi355.AqError):
            fresh.qmm(dx, dw.w, dw.s, dw.b, dy, M, K, N, 64, 4, aq_mi355.AQ_OUT_F32)
        try:
            fresh.graph_destroy(fresh.capture_end())
        except aq_mi355.AqError:
            pass
        fresh.reserve_workspace_bytes(64 << 20)
        fresh.capture_begin()
        fresh.qmm(dx, dw.w, dw.s, dw.b, dy, M, K, N, 64, 4, aq_mi355.AQ_OUT_F32)
        graph = fresh.capture_end()
        first = None
        for i in range(3):
            fresh.fill_zero(dy)
            fresh.graph_launch(graph)
            fresh.sync()
            got = dy.download(np.float32, M * N).copy()
            check_accumulators(got, ref, "replay %d" % i)
            if first is None:
                first = got
            assert np.array_equal(got.view(np.uint32), first.view(np.uint32)), i
        fresh.graph_destroy(graph)
        fresh.qmm(dx, dw.w, dw.s, dw.b, dy, M, K, N, 64, 4, aq_mi355.AQ_OUT_F32)
        fresh.sync()
        assert np.array_equal(dy.download(np.float32, M * N).view(np.uint32), first.view(np.uint32))
        dw.free()
        dx.free()
        dy.free()
    finally:
        fresh.close()


def _half_variants():
    import aq_mi355
    return [(i, n) for i, n in enumerate(aq_mi355.variant_names(1)) if n.startswith("qmmh_")]


def test_qmm_fp16_operand_kernels_power_of_two_factors(ctx, orc):
    """The qmmh kernels multiply fp16 operands: rows of x and rows of the weights are brought into fp16 range by
    powers of two that the epilogue takes off again.  So scaling a row of x, or the scales and biases of a row of
    the weights, by a power of two must scale the fp32 outputs by exactly that power (bit for bit), wherever the
    row sits in bf16's range; an all-zero row gives zeros; and a row whose elements differ by many orders of
    magnitude still meets the reference to fp32 accumulation accuracy."""
    M, K, N = 130, 1024, 300
    words, s, b = F.synthetic_affine(N, K, 4, 64, seed=611)
    x = F.synthetic_x(M, K, seed=612)
    xf = F.bf16_bits_to_f32(x).reshape(M, K)
    row_pow = np.zeros(M, dtype=np.int64)
    row_pow[1:9] = [40, -40, 100, -100, 14, -14, 1, -1]
    x2 = (xf * np.exp2(row_pow)[:, None].astype(np.float32)).astype(np.float32)
    x2[9] = 0.0
    x2_bits = F.f32_to_bf16_bits(x2)
    col_pow = np.zeros(N, dtype=np.int64)
    col_pow[2:8] = [30, -30, 60, -60, 7, -7]
    sf, bf = F.bf16_bits_to_f32(s).reshape(N, -1), F.bf16_bits_to_f32(b).reshape(N, -1)
    s2 = F.f32_to_bf16_bits(sf * np.exp2(col_pow)[:, None].astype(np.float32)).reshape(s.shape)
    b2 = F.f32_to_bf16_bits(bf * np.exp2(col_pow)[:, None].astype(np.float32)).reshape(b.shape)
    # a row of x with a few very large elements among ordinary ones
    x3 = xf.copy()
    x3[11, ::97] *= 3000.0
    x3_bits = F.f32_to_bf16_bits(x3)
    dw, dw2 = DeviceAffine(ctx, words, s, b), DeviceAffine(ctx, words, s2, b2)
    try:
        for idx, name in _half_variants():
            say("qmmh scaling", name)
            ctx.force_variant(1, idx)
            base = run_qmv(ctx, x, dw, M, K, N, 64, 4, True, "qmm").reshape(M, N)
            assert ctx.last_variant(1) == name
            check_accumulators(base, F.reference_f64(x, words, s, b, 4, 64, K), name)
            rows = run_qmv(ctx, x2_bits, dw, M, K, N, 64, 4, True, "qmm").reshape(M, N)
            want = (base.astype(np.float64) * np.exp2(row_pow)[:, None]).astype(np.float32)
            want[9] = 0.0
            assert np.array_equal(rows.view(np.uint32), want.view(np.uint32)), name
            cols = run_qmv(ctx, x, dw2, M, K, N, 64, 4, True, "qmm").reshape(M, N)
            want = (base.astype(np.float64) * np.exp2(col_pow)[None, :]).astype(np.float32)
            assert np.array_equal(cols.view(np.uint32), want.view(np.uint32)), name
            wide = run_qmv(ctx, x3_bits, dw, M, K, N, 64, 4, True, "qmm").reshape(M, N)
            ref = F.reference_f64(x3_bits, words, s, b, 4, 64, K)
            wabs = np.abs(F.numpy_dequant(words, s, b, 4, 64, K).astype(np.float64))
            mass = np.abs(x3.astype(np.float64)) @ wabs.T
            assert (np.abs(wide - ref) <= 4e-6 * mass + 1e-6).all(), name
    finally:
        ctx.force_variant(1, -1)
    dw.free()
    dw2.free()


@pytest.mark.parametrize("M,K,N,gs", [(1, 64, 1, 64), (33, 192, 257, 64), (300, 2048, 520, 128), (70, 4096, 96, 64)])
def test_qmm_fp16_operand_kernels_shapes(ctx, orc, M, K, N, gs):
    """qmmh variants on shapes that end inside a tile, K of one block, K that ends inside a quad of blocks (192),
    and group size 128, fp32 and bf16 stores."""
    try:
        for idx, name in _half_variants():
            say("qmmh shape", name, M, K, N, gs)
            ctx.force_variant(1, idx)
            _qmv_case(ctx, orc, M, K, N, 4, gs, 7000 + M + K, fn="qmm")
            assert ctx.last_variant(1) == name
    finally:
        ctx.force_variant(1, -1)


def test_qmm_hardware_fixture_q4_g64_tokens16(ctx, orc):
    """17 x 704 x 16 batch fixture of go/engine/hip/hip_hardware_test.go:7822-7878 (reference tolerance 1e-3)."""
    say("qmm hw fixture")
    fx = F.hw_fixture_q4_g64_tokens16()
    want = orc.hip_reference_projection_batch(fx["x"], fx["tokens"], fx["packed"], fx["scales"], fx["biases"], fx["rows"], fx["cols"], 64, 4)
    dw = DeviceAffine(ctx, fx["packed"], fx["scales"], fx["biases"])
    # x = (integer/8) * (t+1)/16 has at most 6 significant bits: exact in bf16
    xb = F.f32_to_bf16_bits(fx["x"])
    assert np.array_equal(F.bf16_bits_to_f32(xb).reshape(fx["x"].shape), fx["x"])
    got = run_qmv(ctx, xb, dw, fx["tokens"], fx["cols"], fx["rows"], 64, 4, True, "qmm")
    assert np.abs(got - want).max() <= fx["tol"]
    dw.free()


def test_qmm_config3_full_size_sampled_columns(ctx, orc):
    """cfg 3 at full size (M=2048, K=4096, N=14336): every output of 192 sampled weight rows against the
    float64 reference, plus linearity in x over the whole output (size-independent)."""
    say("qmm cfg3 full")
    M, K, N = 2048, 4096, 14336
    words, s, b = F.synthetic_affine(N, K, 4, 64, seed=F.BASE_SEED + 3)
    x = F.synthetic_x(M, K, seed=F.BASE_SEED + 1003)
    dw = DeviceAffine(ctx, words, s, b)
    acc = run_qmv(ctx, x, dw, M, K, N, 64, 4, True, "qmm")
    rng = np.random.default_rng(3)
    cols = np.sort(rng.choice(N, 192, replace=False))
    ref = F.reference_f64(x, words[cols], s[cols], b[cols], 4, 64, K)
    check_accumulators(acc[:, cols], ref, "cfg3 sampled")
    # y(2x) == 2 y(x) exactly: doubling bf16 inputs doubles every exact product and every fp32 partial sum
    x2 = F.f32_to_bf16_bits(F.bf16_bits_to_f32(x) * np.float32(2))
    acc2 = run_qmv(ctx, x2, dw, M, K, N, 64, 4, True, "qmm")
    assert np.array_equal(acc2, acc * np.float32(2))
    dw.free()


def test_qmm_errors(ctx):
    import aq_mi355
    buf = ctx.alloc(4096)
    for args in [(0, 64, 4, 64, 4), (1, 64, 0, 64, 4), (1, 0, 4, 64, 4)]:
        with pytest.raises(aq_mi355.AqError) as e:
            ctx.qmm(buf, buf, buf, buf, buf, *args)
        assert e.value.code == aq_mi355.AQ_ERR_SHAPE
    buf.free()


def test_rows_through_the_gather_have_single_row_bytes(ctx, orc):
    """More than eight rows with the bytes of single-row calls: the reference's multi-row route rides its gather kernel
    with one expert and lhs = the identity (go/engine/metal/qmv_rows.go:14-24, up to 24 rows); the same call here."""
    say("rows through gather")
    import aq_mi355
    K, N, M = 4096, 528, 24
    words, s, b = F.synthetic_affine(N, K, 4, 64, seed=1401)
    x = F.synthetic_x(M, K, seed=1402)
    dw = DeviceAffine(ctx, words, s, b)
    dx, dl = ctx.to_device(x), ctx.to_device(np.arange(M, dtype=np.int32))
    dr, dy = ctx.to_device(np.zeros(M, dtype=np.int32)), ctx.alloc(M * N * 2)
    ctx.gather_qmv(dx, dw.w, dw.s, dw.b, dl, dr, dy, M, M, K, N, 1, N, 0, 64, 4, 0)
    ctx.sync()
    got = dy.download(np.uint16, M * N).reshape(M, N)
    for m in range(M):
        one = run_qmv(ctx, x[m:m + 1], dw, 1, K, N, 64, 4, False)
        assert np.array_equal(got[m], one[0]), m
    for t in (dx, dl, dr, dy):
        t.free()
    dw.free()
