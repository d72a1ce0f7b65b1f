// affine_qmv for 5..32 rows of x on gfx950 (batched / speculative-verify decode), 4-bit codes in groups of 64:
// one launch, the weights streamed exactly once, no pass over x beforehand and no partial tiles in memory.
//
// Same contract as the other matvec kernels: replaces rocm_mlx_q4_projection_batch*
// (go/engine/hip/kernels/quant/affine_projection_tuned.hipinc:292-472, 16 rows x 16 tokens in one launch) and the
// rows kernel of go/engine/metal/qmv_rows.go:14-60; semantics of MLX affine_qmv with M rows
// (go/engine/metal/kernels/quant/lthn_qmv_rows.metal:1-22).
//
// v_mfma_f32_32x32x16_bf16 with the TOKENS as the 32 rows of A and 32 weight rows as the columns of B:
//   * as B operand lane (n = lane % 32, h = lane / 32) holds 16 bytes of weight row n per quantisation group: codes
//     32 h .. 32 h + 31 of the group's 64, so a register set covers exactly one group of 32 rows, its four words are the
//     B operands of four MFMAs (8 codes per lane and MFMA, expanded to bf16 128 + code with one v_and_or_b32 per pair),
//     and D = sum over the group of (128 + code) * x for 32 tokens x 32 rows needs no separation of groups;
//   * the A operands come straight from x in global memory (L2): lane (t = lane % 32, h) holds the 16 bytes
//     x[t][64 g + 32 h + 8 i ..] for MFMA i, permuted into the order the expansion leaves the codes in
//     (c0 c4 c1 c5 c2 c6 c3 c7); tokens past M re-read the last one and are never stored;
//   * both are LOADED in another shape, 64 contiguous bytes of each of 16 rows per instruction, and brought into the
//     MFMA layout by v_permlane16_swap / v_permlane32_swap (two per register for the weights, one per register for x);
//   * per group and set of 32 rows: acc += scale * D, sixteen fp32 FMAs per lane (scale depends on the lane's row only);
//   * the affine term is MFMA work: the lane's share of a group's sum of x comes from four v_dot2 per A operand, the two
//     halves meet with one v_permlane32_swap, the sum is split into three bf16 terms (exact), and per four groups two
//     MFMAs per set of rows add (bias - 128 scale) * sum(x) with A = (X0 X1 X2 -128X0 -128X1 -128X2 0 0) and
//     B = (b b b s s s 0 0), one group per half of the lanes;
//   * the NW wavefronts of a workgroup share K (whole runs of four groups each) for the same R sets of 32 rows and meet
//     in LDS at the end; every wavefront keeps four groups of weights and of x in flight.
// A row's result depends on M only through which tokens exist: token t of an M-row call equals token t of any other
// call with the same (NW, R) split, bit for bit.
#include "aq_device.h"
#include "aq_kernels.h"

#include <type_traits>

namespace aq {

namespace {

typedef const __attribute__((address_space(1))) char* gptr_t;
__device__ __forceinline__ gptr_t uniform_ptr(const void* p) {
    const uint64_t u = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return reinterpret_cast<gptr_t>(((uint64_t)hi << 32) | lo);
}
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 load_u128_at(gptr_t base, uint32_t off) {
    const u32x4_t v = *reinterpret_cast<const __attribute__((address_space(1))) u32x4_t*>(base + off);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint2 load_u64_at(gptr_t base, uint32_t off) {
    const u32x2_t v = *reinterpret_cast<const __attribute__((address_space(1))) u32x2_t*>(base + off);
    return make_uint2(v[0], v[1]);
}
__device__ __forceinline__ bf16x8_t as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const uint4 v = make_uint4(a, b, c, d);
    return __builtin_bit_cast(bf16x8_t, v);
}

constexpr int kTokRows = 32;  // weight rows per set (the N side of the MFMA)
constexpr int kTokMax = 32;   // activation rows per launch (the M side)
// 8-byte pieces of scales (and of biases) a thread of the 16-token form stages at most: K up to 16384 with 16 wavefronts
__host__ __device__ constexpr int tok16_stage_pieces(int nw) { return nw >= 16 ? 4 : 8; }

}  // namespace

// NW wavefronts share K; each works on R sets of 32 weight rows.  (NW * kWave threads, NW * R * 4 KiB of LDS.)
template <int NW, int R>
__global__ __launch_bounds__(NW* kWave) void qmv_tok_kernel(const QmvArgs a) {
    static_assert((R * 16) % NW == 0, "the output registers are shared out over the wavefronts for the final sum");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31;
    const int h = lane >> 5;
    const int K = a.K, N = a.N, M = a.M;
    const int groups = K >> 6;
    const int quads = K >> 8;  // runs of four groups (K % 256 == 0)
    const int per = (quads + NW - 1) / NW;
    const int q_begin = wave * per;
    const int q_end = min(quads, q_begin + per);
    const int row0 = (int)blockIdx.x * (kTokRows * R);

    const gptr_t wg = uniform_ptr(a.w), sg = uniform_ptr(a.s), bg = uniform_ptr(a.b), xg = uniform_ptr(a.x);
    // Loads are shaped for the memory pipeline, not for the MFMA: lane (n16 = lane % 16, j = lane / 16) reads 16 bytes of
    // row (or token) n16 at 16 j, so that an instruction covers 64 contiguous bytes of each of 16 rows (with the MFMA's own
    // layout, two 16-byte pieces of each of 32 rows, the same kernel took 14 us with its arithmetic removed).  Two
    // such loads (rows 0..15 and 16..31) become two operands in the MFMA layout by two lane swaps per register.
    const int n16 = lane & 15, j16 = lane >> 4;
    uint32_t w_lane[R][2], sb_lane[R];
#pragma unroll
    for (int rs = 0; rs < R; rs++) {
#pragma unroll
        for (int ab = 0; ab < 2; ab++) {
            const int row = min(row0 + rs * kTokRows + ab * 16 + n16, N - 1);
            w_lane[rs][ab] = (uint32_t)row * (uint32_t)(K >> 1) + (uint32_t)j16 * 16u;
        }
        sb_lane[rs] = (uint32_t)min(row0 + rs * kTokRows + n, N - 1) * (uint32_t)groups * 2u;
    }
    uint32_t x_lane[2];
#pragma unroll
    for (int ab = 0; ab < 2; ab++) x_lane[ab] = (uint32_t)min(ab * 16 + n16, M - 1) * (uint32_t)K * 2u + (uint32_t)j16 * 16u;

    const uint32_t mask = opaque_s(kNibbleMask);
    const uint32_t magic = opaque_v(kMagic128);
    const uint32_t ones = 0x3f803f80u;
    // byte selectors for the affine-term B operand: the lane's group is the low (h = 0) or high (h = 1) half of a word
    const uint32_t sel_same = h ? 0x03020302u : 0x01000100u;
    const uint32_t sel_mix = h ? 0x07060302u : 0x05040100u;

    // In flight per wavefront: two quads of weights (whole quads, so that the four 32-byte pieces of a row's 128-byte line
    // are requested together: requested a group at a time, lines were evicted between their pieces and HBM fetched half
    // as much again), their scales and biases, and DA groups of x.
    constexpr int DA = 4;
    // wq[slot][L][ab]: bytes 64 L .. 64 L + 63 of the quad's 128 per row, rows 0..15 (ab = 0) / 16..31 (ab = 1); after the
    // swaps the same registers hold groups 2 L (ab = 0) and 2 L + 1 (ab = 1) in the MFMA layout.
    uint4 wq[2][2][2][R];
    uint2 sq[2][R], bq[2][R];
    // xq[slot][half h][ab]: x[token][64 g + 32 h + 8 j ..] of tokens 0..15 / 16..31; after the swaps [i / 2][i % 2] is the
    // A operand of MFMA i.
    uint4 xq[DA][2][2];
    auto issue_w = [&](auto slot_tag, int q) {
        constexpr int slot = decltype(slot_tag)::value;
        const uint32_t qc = (uint32_t)min(q, quads - 1);  // past the end of K: a valid address, the data is not used
#pragma unroll
        for (int rs = 0; rs < R; rs++) {
            sq[slot][rs] = load_u64_at(sg, sb_lane[rs] + qc * 8u);
            bq[slot][rs] = load_u64_at(bg, sb_lane[rs] + qc * 8u);
        }
#pragma unroll
        for (int L = 0; L < 2; L++)
#pragma unroll
            for (int rs = 0; rs < R; rs++)
#pragma unroll
                for (int ab = 0; ab < 2; ab++)
                    wq[slot][L][ab][rs] = load_u128_at(wg, w_lane[rs][ab] + qc * 128u + (uint32_t)L * 64u);
    };
    auto issue_x = [&](auto slot_tag, int g) {
        constexpr int slot = decltype(slot_tag)::value;
        const uint32_t gc = (uint32_t)min(g, groups - 1);
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int ab = 0; ab < 2; ab++) xq[slot][hh][ab] = load_u128_at(xg, x_lane[ab] + gc * 128u + (uint32_t)hh * 64u);
    };
    // 16-lane blocks [a0 a1 a2 a3], [b0 b1 b2 b3] -> [a0 b0 a1 b1], [a2 b2 a3 b3]
    auto weave = [](uint32_t& a, uint32_t& b) {
        const auto s1 = __builtin_amdgcn_permlane16_swap(a, b, false, false);      // [a0 b0 a2 b2], [a1 b1 a3 b3]
        const auto s2 = __builtin_amdgcn_permlane32_swap(s1[0], s1[1], false, false);  // [a0 b0 a1 b1], [a2 b2 a3 b3]
        a = s2[0];
        b = s2[1];
    };
    auto weave4 = [&](uint4& a, uint4& b) {
        weave(a.x, b.x);
        weave(a.y, b.y);
        weave(a.z, b.z);
        weave(a.w, b.w);
    };
    // four registers of 16-lane blocks s_k = [s_k.0 .. s_k.3] -> f_i = [s_0.i s_1.i s_2.i s_3.i]
    auto transpose = [](uint32_t& s0, uint32_t& s1, uint32_t& s2, uint32_t& s3) {
        const auto p = __builtin_amdgcn_permlane16_swap(s0, s1, false, false);  // [s0.0 s1.0 s0.2 s1.2], [s0.1 s1.1 s0.3 s1.3]
        const auto q = __builtin_amdgcn_permlane16_swap(s2, s3, false, false);
        const auto e = __builtin_amdgcn_permlane32_swap(p[0], q[0], false, false);  // f0, f2
        const auto o = __builtin_amdgcn_permlane32_swap(p[1], q[1], false, false);  // f1, f3
        s0 = e[0];
        s1 = o[0];
        s2 = e[1];
        s3 = o[1];
    };

    f32x16_t acc[R];
#pragma unroll
    for (int rs = 0; rs < R; rs++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[rs][r] = 0.0f;

    // Loads return in the order they were issued and the compiler waits by counting back from the newest: x first (it
    // comes from L2), then the quads in the order they are used; pinned, because the scheduler would reorder them.
#pragma unroll
    for (int d = 0; d < DA; d++) {
        if (d == 0) issue_x(std::integral_constant<int, 0>{}, 4 * q_begin + 0);
        if (d == 1) issue_x(std::integral_constant<int, 1 % DA>{}, 4 * q_begin + 1);
        if (d == 2) issue_x(std::integral_constant<int, 2 % DA>{}, 4 * q_begin + 2);
        if (d == 3) issue_x(std::integral_constant<int, 3 % DA>{}, 4 * q_begin + 3);
    }
    __builtin_amdgcn_sched_barrier(0);
    issue_w(std::integral_constant<int, 0>{}, q_begin);
    __builtin_amdgcn_sched_barrier(0);

    // One quad (four groups) from weight slot WS.  REFILL_X: after each group its x slot is reloaded with the group DA
    // further on (without it only with groups of the same quad); REFILL_W: after the quad its weight slot is reloaded with the quad after next.  Both are compile-time:
    // a conditional load inside the loop splits it into blocks across which the compiler moves the arithmetic to the end.
    auto quad = [&](int q, auto ws_tag, auto refill_x_tag, auto refill_w_tag) {
        constexpr int WS = decltype(ws_tag)::value;
        constexpr bool REFILL_X = decltype(refill_x_tag)::value;
        constexpr bool REFILL_W = decltype(refill_w_tag)::value;
        if constexpr (REFILL_W) {
            issue_w(std::integral_constant<int, 1 - WS>{}, q + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        float hsum[4];
        auto group = [&](auto d_tag) {
            constexpr int d = decltype(d_tag)::value;
            constexpr int XS = d % DA;
            // x: (half 0, tokens 0..15), (half 0, tokens 16..31), (half 1, ..), (half 1, ..) -> the A operands of MFMA 0 .. 3
            transpose(xq[XS][0][0].x, xq[XS][0][1].x, xq[XS][1][0].x, xq[XS][1][1].x);
            transpose(xq[XS][0][0].y, xq[XS][0][1].y, xq[XS][1][0].y, xq[XS][1][1].y);
            transpose(xq[XS][0][0].z, xq[XS][0][1].z, xq[XS][1][0].z, xq[XS][1][1].z);
            transpose(xq[XS][0][0].w, xq[XS][0][1].w, xq[XS][1][0].w, xq[XS][1][1].w);
            bf16x8_t af[4];
            float hs = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint4 v = xq[XS][i >> 1][i & 1];
                af[i] = as_bf16x8(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                                  __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
                hs = dot2_bf16(v.x, ones, hs);
                hs = dot2_bf16(v.y, ones, hs);
                hs = dot2_bf16(v.z, ones, hs);
                hs = dot2_bf16(v.w, ones, hs);
            }
            hsum[d] = hs;
#pragma unroll
            for (int rs = 0; rs < R; rs++) {
                if constexpr ((d & 1) == 0) weave4(wq[WS][d >> 1][0][rs], wq[WS][d >> 1][1][rs]);  // groups d and d + 1
                const uint4 wv = wq[WS][d >> 1][d & 1][rs];
                const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
                f32x16_t p;
#pragma unroll
                for (int r = 0; r < 16; r++) p[r] = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint32_t e[4];
                    unpack4_word(ww[i], mask, magic, e);
                    p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], as_bf16x8(e[0], e[1], e[2], e[3]), p, 0, 0, 0);
                }
                const uint32_t sw = d < 2 ? sq[WS][rs].x : sq[WS][rs].y;
                const float sc = (d & 1) ? __uint_as_float(sw & 0xffff0000u) : __uint_as_float(sw << 16);
#pragma unroll
                for (int r = 0; r < 16; r++) acc[rs][r] = __builtin_fmaf(sc, p[r], acc[rs][r]);
            }
            if constexpr (REFILL_X || d + DA < 4) issue_x(std::integral_constant<int, XS>{}, 4 * q + d + DA);
            // groups stay apart in the schedule: interleaved, their MFMA results and expanded codes need more
            // registers than two wavefronts per SIMD leave
            __builtin_amdgcn_sched_barrier(0);
        };
        group(std::integral_constant<int, 0>{});
        group(std::integral_constant<int, 1>{});
        group(std::integral_constant<int, 2>{});
        group(std::integral_constant<int, 3>{});
        // affine term of the quad: lanes h = 0 carry groups 0 and 2, lanes h = 1 groups 1 and 3
#pragma unroll
        for (int pq = 0; pq < 2; pq++) {
            const auto sw2 = __builtin_amdgcn_permlane32_swap(__float_as_uint(hsum[2 * pq]), __float_as_uint(hsum[2 * pq + 1]),
                                                              false, false);
            const float X = __uint_as_float(sw2[0]) + __uint_as_float(sw2[1]);
            const uint32_t u0 = __float_as_uint(X) & 0xffff0000u;
            const float r1 = X - __uint_as_float(u0);
            const uint32_t u1 = __float_as_uint(r1) & 0xffff0000u;
            const float r2 = r1 - __uint_as_float(u1);
            const uint32_t u2 = __float_as_uint(r2) & 0xffff0000u;
            const uint32_t n0 = __float_as_uint(-128.0f * __uint_as_float(u0));
            const uint32_t n1 = __float_as_uint(-128.0f * __uint_as_float(u1));
            const uint32_t n2 = __float_as_uint(-128.0f * __uint_as_float(u2));
            const bf16x8_t a2 = as_bf16x8((u0 >> 16) | u1, (u2 >> 16) | n0, (n1 >> 16) | n2, 0u);
#pragma unroll
            for (int rs = 0; rs < R; rs++) {
                const uint32_t sw = pq ? sq[WS][rs].y : sq[WS][rs].x;
                const uint32_t bw = pq ? bq[WS][rs].y : bq[WS][rs].x;
                const bf16x8_t b2 = as_bf16x8(__builtin_amdgcn_perm(bw, bw, sel_same), __builtin_amdgcn_perm(sw, bw, sel_mix),
                                              __builtin_amdgcn_perm(sw, sw, sel_same), 0u);
                acc[rs] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a2, b2, acc[rs], 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    {
        const std::integral_constant<int, 0> S0;
        const std::integral_constant<int, 1> S1;
        const std::true_type T;
        const std::false_type F;
        const int nq = q_end - q_begin;
        int q = q_begin;
        int full = nq > 1 ? nq - 1 : 0;  // quads with a next quad to request
        for (; full >= 2; full -= 2, q += 2) {
            quad(q, S0, T, T);
            quad(q + 1, S1, T, T);
        }
        if (full == 1) {
            quad(q, S0, T, T);
            quad(q + 1, S1, F, F);
        } else if (nq >= 1) {
            quad(q, S0, F, F);
        }
    }

    // ---- the wavefronts' partial sums meet in LDS; every wavefront adds and stores its share of the registers ----
    float* red = reinterpret_cast<float*>(lds_raw);
#pragma unroll
    for (int rs = 0; rs < R; rs++)
#pragma unroll
        for (int r = 0; r < 16; r++) red[((wave * R + rs) * 16 + r) * 64 + lane] = acc[rs][r];
    __syncthreads();
    constexpr int RPW = R * 16 / NW;
#pragma unroll
    for (int k = 0; k < RPW; k++) {
        const int idx = wave * RPW + k;  // (row set, register)
        const int rs = idx >> 4, r = idx & 15;
        float total = red[((0 * R + rs) * 16 + r) * 64 + lane];
#pragma unroll
        for (int p = 1; p < NW; p++) total += red[((p * R + rs) * 16 + r) * 64 + lane];
        // D layout of the 32x32 MFMA: lane (n, h), register r -> token 8 (r / 4) + 4 h + r % 4, weight row n
        const int t = 8 * (r >> 2) + 4 * h + (r & 3);
        const int row = row0 + rs * kTokRows + n;
        if (t < M && row < N) {
            const size_t o = (size_t)t * N + row;
            if (a.out_f32) {
                static_cast<float*>(a.y)[o] = total;
            } else {
                static_cast<uint16_t*>(a.y)[o] = f32_to_bf16_bits(total);
            }
        }
    }
}


// ---- up to 16 rows of x: 16x16x32 MFMAs, sixteen wavefronts that share K ---------------------------------------------
//
// v_mfma_f32_16x16x32_bf16 with the tokens as the 16 rows of A and 16 weight rows as the columns of B.  A workgroup of
// NW wavefronts owns RS sets of 16 weight rows; wavefront w takes the runs of 256 codes w, w + NW, ... of all of them.
//   * A load instruction covers whole 128-byte lines (a run of 256 codes) of 8 rows; two DPP moves per register pair
//     bring two such loads into the shape "lane (n = lane % 16, p = lane / 16) holds bytes 16 p .. 16 p + 15 of a
//     64-byte block of row n".  The MFMA wants from lane (n, q) the eight codes 8 q .. 8 q + 7 of a run of 32, i.e. word
//     q of four consecutive words: the four registers are transposed across the four 16-lane blocks (four lane swaps
//     per 16 bytes), after which register i of a block of 128 codes is the B operand of its step i (codes 32 i ..
//     32 i + 31), expanded with one v_and_or_b32 per pair of codes.
//   * x is read a whole 128-byte line of each of 8 tokens per instruction: lanes i = lane % 16 < 8 take the first 64
//     bytes of token i (an even step), lanes i >= 8 the second 64 bytes of token i - 8 (the odd step behind it); a
//     second instruction does the same for tokens 8..15, and two DPP moves per register pair put the halves where the
//     A operands want them.  Inside the 16 bytes the values are permuted into the order the expansion leaves the codes
//     in.  Every wavefront reads just the runs it multiplies.  (Requests are what this kernel pays for at the L1: with
//     64 bytes of 16 tokens per instruction, and every wavefront fetching its own 8 bytes of each row's scales and
//     biases, x and the scales each cost as much time as the weights.)
//   * scales and biases of the workgroup's rows are fetched once, whole rows by all threads together, and handed round
//     in LDS.
//   * two steps make a quantisation group: acc += scale * D, four FMAs per lane, group and set of rows.
//   * the affine term is one MFMA per run and set of rows: lane block q carries group q of the run, A = the three-way
//     bf16 split of the group's sum of x (and -128 times it), B = (b b b s s s 0 0); the sums of x come from v_dot2
//     per lane and a 4 x 4 transpose-add over the lane blocks, which leaves group q's total in block q.
//   * the wavefronts' partial sums meet in LDS; with sixteen wavefronts of at most 128 registers a SIMD holds four, whose
//     loads, lane swaps, expansions and MFMAs overlap.
// Token t of an M-row call equals token t of any other call on the same variant, bit for bit.
template <int NW, int RS, int QW, int RING>
__global__ __launch_bounds__(NW* kWave) void qmv_tok16_kernel(const QmvArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    constexpr int ROWS = RS * 16;   // weight rows per workgroup
    constexpr int TSTRIDE = ROWS;   // floats between tokens in the LDS partials
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15;
    const int q = lane >> 4;
    const int K = a.K, N = a.N, M = a.M;
    const int groups = K >> 6;
    const int quads = K >> 8;
    const int row0 = (int)blockIdx.x * ROWS;

    const gptr_t wg = uniform_ptr(a.w), sg = uniform_ptr(a.s), bg = uniform_ptr(a.b), xg = uniform_ptr(a.x);
    // weights: lane (i, q) of load `ab` reads row (i % 8) + 8 ab of a set, bytes 64 (i / 8) + 16 q of the run's 128: an
    // instruction covers whole 128-byte lines of 8 rows
    uint32_t w_lane[RS][2];
#pragma unroll
    for (int rs = 0; rs < RS; rs++)
#pragma unroll
        for (int ab = 0; ab < 2; ab++) {
            const int row = min(row0 + rs * 16 + (n & 7) + 8 * ab, N - 1);  // past N: a valid row, never stored
            w_lane[rs][ab] = (uint32_t)row * (uint32_t)(K >> 1) + (uint32_t)(n >> 3) * 64u + (uint32_t)q * 16u;
        }
    // x: lane (i, q) of load `ab` reads token (i % 8) + 8 ab, bytes 64 (i / 8) + 16 q of a 128-byte step pair
    uint32_t x_lane[2];
#pragma unroll
    for (int ab = 0; ab < 2; ab++)
        x_lane[ab] = (uint32_t)min((n & 7) + 8 * ab, M - 1) * (uint32_t)K * 2u + (uint32_t)(n >> 3) * 64u + (uint32_t)q * 16u;

    const uint32_t mask = opaque_s(kNibbleMask);
    const uint32_t magic = opaque_v(kMagic128);
    const uint32_t ones = 0x3f803f80u;
    // picks element q of four bf16 values in two registers, twice
    const uint32_t sel_q = 0x01000100u + 0x02020202u * (uint32_t)q;

    auto transpose = [](uint32_t& s0, uint32_t& s1, uint32_t& s2, uint32_t& s3) {
        const auto p = __builtin_amdgcn_permlane16_swap(s0, s1, false, false);
        const auto r = __builtin_amdgcn_permlane16_swap(s2, s3, false, false);
        const auto e = __builtin_amdgcn_permlane32_swap(p[0], r[0], false, false);
        const auto o = __builtin_amdgcn_permlane32_swap(p[1], r[1], false, false);
        s0 = e[0];
        s1 = o[0];
        s2 = e[1];
        s3 = o[1];
    };

    f32x4_t acc[RS];
#pragma unroll
    for (int rs = 0; rs < RS; rs++) acc[rs] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

    uint4* const sbq = reinterpret_cast<uint4*>(lds_raw);
    const int sb_pitch = quads + 1;

    // Scales and biases of the workgroup's rows: fetched once by all threads together, whole rows (every wavefront
    // fetching its own 8 bytes per row and run cost as much time as the weights), into LDS as (s0 s1, s2 s3, b0 b1,
    // b2 b3) per row and run; rows are a run apart plus 16 bytes, so that the 16 rows a wavefront reads at once fall into
    // different banks.  The loads go out first, the first pass's x and weights behind them, and only then are they stored.
    constexpr int NT = NW * kWave;
    constexpr int PRE = tok16_stage_pieces(NW);
    const int pieces = ROWS * quads;
    uint2 sv[PRE], bv[PRE];
#pragma unroll
    for (int i = 0; i < PRE; i++) {
        const int p = tid + i * NT;
        if (p < pieces) {
            const int r = p / quads, c = p - r * quads;
            const uint32_t at = (uint32_t)min(row0 + r, N - 1) * (uint32_t)groups * 2u + (uint32_t)c * 8u;
            sv[i] = load_u64_at(sg, at);
            bv[i] = load_u64_at(bg, at);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // A pass: QW runs of this wavefront (NW runs apart), their A operands in registers, and the RS sets of rows streamed
    // past them one set at a time through a ring of RING register slots.  Loads return in the order they were issued, and
    // requests that are out at the same time come back in the order the memory likes, not in the order they are needed:
    // a set is therefore requested only RING sets ahead of its use, which keeps HBM busy during the arithmetic without
    // making the first set wait for the last.
    uint4 ring[RING][QW][2];
    auto issue_set = [&](auto slot_tag, int rs_dyn, const int (&qds)[QW]) {
        constexpr int SL = decltype(slot_tag)::value;
#pragma unroll
        for (int j = 0; j < QW; j++)
#pragma unroll
            for (int ab = 0; ab < 2; ab++) {
                uint32_t base = 0;
#pragma unroll
                for (int rs = 0; rs < RS; rs++) base = rs == rs_dyn ? w_lane[rs][ab] : base;
                ring[SL][j][ab] = load_u128_at(wg, base + (uint32_t)qds[j] * 128u);
            }
    };
    bool staged = false;
    for (int qbase = wave; qbase < quads; qbase += NW * QW) {
        int qds[QW];   // clamped: a run past the end of K is loaded from the last run and not used
        bool live[QW];
#pragma unroll
        for (int j = 0; j < QW; j++) {
            live[j] = qbase + j * NW < quads;
            qds[j] = live[j] ? qbase + j * NW : qbase;
        }
        uint4 xa[QW][4], xb[QW][4];
#pragma unroll
        for (int j = 0; j < QW; j++)
#pragma unroll
            for (int sp = 0; sp < 4; sp++) {
                xa[j][sp] = load_u128_at(xg, x_lane[0] + (uint32_t)qds[j] * 512u + (uint32_t)sp * 128u);
                xb[j][sp] = load_u128_at(xg, x_lane[1] + (uint32_t)qds[j] * 512u + (uint32_t)sp * 128u);
            }
        __builtin_amdgcn_sched_barrier(0);
        issue_set(std::integral_constant<int, 0>{}, 0, qds);
        if constexpr (RING > 1 && RS > 1) issue_set(std::integral_constant<int, 1 % RING>{}, 1, qds);
        if constexpr (RING > 2 && RS > 2) issue_set(std::integral_constant<int, 2 % RING>{}, 2, qds);
        __builtin_amdgcn_sched_barrier(0);
        if (!staged) {
#pragma unroll
            for (int i = 0; i < PRE; i++) {
                const int p = tid + i * NT;
                if (p < pieces) {
                    const int r = p / quads, c = p - r * quads;
                    sbq[r * sb_pitch + c] = make_uint4(sv[i].x, sv[i].y, bv[i].x, bv[i].y);
                }
            }
            __syncthreads();
            staged = true;
        }

        // A operands of the pass's runs, and per run the three-way split of the lane block's group sum of x
        bf16x8_t af[QW][8], a2[QW];
#pragma unroll
        for (int j = 0; j < QW; j++) {
            float ps[4];
#pragma unroll
            for (int st = 0; st < 8; st++) {
                // even step: lanes i >= 8 take tokens 8..15 from the second load's lanes i - 8; odd step: lanes i < 8 take
                // tokens 0..7 from the first load's lanes i + 8
                const uint4 va = xa[j][st >> 1], vb = xb[j][st >> 1];
                uint4 v;
                if ((st & 1) == 0) {
                    v.x = __builtin_amdgcn_update_dpp(va.x, vb.x, 0x118, 0xf, 0xc, false);
                    v.y = __builtin_amdgcn_update_dpp(va.y, vb.y, 0x118, 0xf, 0xc, false);
                    v.z = __builtin_amdgcn_update_dpp(va.z, vb.z, 0x118, 0xf, 0xc, false);
                    v.w = __builtin_amdgcn_update_dpp(va.w, vb.w, 0x118, 0xf, 0xc, false);
                } else {
                    v.x = __builtin_amdgcn_update_dpp(vb.x, va.x, 0x108, 0xf, 0x3, false);
                    v.y = __builtin_amdgcn_update_dpp(vb.y, va.y, 0x108, 0xf, 0x3, false);
                    v.z = __builtin_amdgcn_update_dpp(vb.z, va.z, 0x108, 0xf, 0x3, false);
                    v.w = __builtin_amdgcn_update_dpp(vb.w, va.w, 0x108, 0xf, 0x3, false);
                }
                af[j][st] = as_bf16x8(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                                      __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
                float hs = (st & 1) ? ps[st >> 1] : 0.0f;
                hs = dot2_bf16(v.x, ones, hs);
                hs = dot2_bf16(v.y, ones, hs);
                hs = dot2_bf16(v.z, ones, hs);
                hs = dot2_bf16(v.w, ones, hs);
                ps[st >> 1] = hs;
            }
            // block q of register g holds lane block q's share of group g; transposed, the four registers of block q are
            // the four shares of group q
            uint32_t t0 = __float_as_uint(ps[0]), t1 = __float_as_uint(ps[1]), t2 = __float_as_uint(ps[2]), t3 = __float_as_uint(ps[3]);
            transpose(t0, t1, t2, t3);
            float X = (__uint_as_float(t0) + __uint_as_float(t1)) + (__uint_as_float(t2) + __uint_as_float(t3));
            if (!live[j]) X = 0.0f;
            const uint32_t u0 = __float_as_uint(X) & 0xffff0000u;
            const float r1 = X - __uint_as_float(u0);
            const uint32_t u1 = __float_as_uint(r1) & 0xffff0000u;
            const float r2 = r1 - __uint_as_float(u1);
            const uint32_t u2 = __float_as_uint(r2) & 0xffff0000u;
            const uint32_t m0 = __float_as_uint(-128.0f * __uint_as_float(u0));
            const uint32_t m1 = __float_as_uint(-128.0f * __uint_as_float(u1));
            const uint32_t m2 = __float_as_uint(-128.0f * __uint_as_float(u2));
            a2[j] = as_bf16x8((u0 >> 16) | u1, (u2 >> 16) | m0, (m1 >> 16) | m2, 0u);
        }

        auto run_set = [&](auto rs_tag) {
            constexpr int rs = decltype(rs_tag)::value;
            constexpr int SL = rs % RING;
#pragma unroll
            for (int j = 0; j < QW; j++) {
                // first 64 bytes of all 16 rows (lanes i >= 8 from the second load's lanes i - 8), second 64 bytes (lanes
                // i < 8 from the first load's lanes i + 8): as for x
                const uint4 la = ring[SL][j][0], lb = ring[SL][j][1];
                uint32_t f0 = __builtin_amdgcn_update_dpp(la.x, lb.x, 0x118, 0xf, 0xc, false);
                uint32_t f1 = __builtin_amdgcn_update_dpp(la.y, lb.y, 0x118, 0xf, 0xc, false);
                uint32_t f2 = __builtin_amdgcn_update_dpp(la.z, lb.z, 0x118, 0xf, 0xc, false);
                uint32_t f3 = __builtin_amdgcn_update_dpp(la.w, lb.w, 0x118, 0xf, 0xc, false);
                uint32_t g0 = __builtin_amdgcn_update_dpp(lb.x, la.x, 0x108, 0xf, 0x3, false);
                uint32_t g1 = __builtin_amdgcn_update_dpp(lb.y, la.y, 0x108, 0xf, 0x3, false);
                uint32_t g2 = __builtin_amdgcn_update_dpp(lb.z, la.z, 0x108, 0xf, 0x3, false);
                uint32_t g3 = __builtin_amdgcn_update_dpp(lb.w, la.w, 0x108, 0xf, 0x3, false);
                transpose(f0, f1, f2, f3);
                transpose(g0, g1, g2, g3);
                const uint32_t ww[8] = {f0, f1, f2, f3, g0, g1, g2, g3};
                const uint4 sbv = sbq[(rs * 16 + n) * sb_pitch + qds[j]];
                f32x4_t part = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    f32x4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int half = 0; half < 2; half++) {
                        uint32_t e[4];
                        unpack4_word(ww[2 * g + half], mask, magic, e);
                        d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[j][2 * g + half], as_bf16x8(e[0], e[1], e[2], e[3]), d, 0, 0, 0);
                    }
                    const uint32_t sw = g < 2 ? sbv.x : sbv.y;
                    const float sc = (g & 1) ? __uint_as_float(sw & 0xffff0000u) : __uint_as_float(sw << 16);
#pragma unroll
                    for (int r = 0; r < 4; r++) part[r] = __builtin_fmaf(sc, d[r], part[r]);
                }
                const uint32_t bb = __builtin_amdgcn_perm(sbv.w, sbv.z, sel_q);
                const uint32_t ss = __builtin_amdgcn_perm(sbv.y, sbv.x, sel_q);
                const bf16x8_t b2 = as_bf16x8(bb, __builtin_amdgcn_perm(ss, bb, 0x05040100u), ss, 0u);
                part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[j], b2, part, 0, 0, 0);
                // a run past the end of K (x and weights of the last run were loaded in its place) adds nothing
                if (live[j]) {
#pragma unroll
                    for (int r = 0; r < 4; r++) acc[rs][r] += part[r];
                }
            }
            if constexpr (rs + RING < RS) {
                __builtin_amdgcn_sched_barrier(0);
                issue_set(std::integral_constant<int, SL>{}, rs + RING, qds);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        run_set(std::integral_constant<int, 0>{});
        if constexpr (RS > 1) run_set(std::integral_constant<int, 1>{});
        if constexpr (RS > 2) run_set(std::integral_constant<int, 2>{});
        if constexpr (RS > 3) run_set(std::integral_constant<int, 3>{});
        static_assert(RS <= 4, "sets of rows per workgroup");
    }
    if (!staged) __syncthreads();  // a wavefront without a run of its own

    // ---- the wavefronts' partial sums meet in LDS: red[wave][token][row]; thread (token, row) adds them in wave order ----
    // (behind the staged scales and biases: a wavefront may get here while another still reads those)
    float* red = reinterpret_cast<float*>(lds_raw + (size_t)ROWS * sb_pitch * 16);
    // D layout of the 16x16 MFMA: lane (n, q), register r -> token 4 q + r, weight row n
#pragma unroll
    for (int rs = 0; rs < RS; rs++)
#pragma unroll
        for (int r = 0; r < 4; r++) red[(wave * 16 + 4 * q + r) * TSTRIDE + rs * 16 + n] = acc[rs][r];
    __syncthreads();
    for (int o = tid; o < 16 * ROWS; o += NW * kWave) {
        const int t = o / ROWS, rl = o - t * ROWS;
        float total = red[t * TSTRIDE + rl];
#pragma unroll
        for (int p = 1; p < NW; p++) total += red[(p * 16 + t) * TSTRIDE + rl];
        const int row = row0 + rl;
        if (t < M && row < N) {
            const size_t at = (size_t)t * N + row;
            if (a.out_f32) {
                static_cast<float*>(a.y)[at] = total;
            } else {
                static_cast<uint16_t*>(a.y)[at] = f32_to_bf16_bits(total);
            }
        }
    }
}

// ---- variant table --------------------------------------------------------

typedef void (*QmvTokKernel)(const QmvArgs);
struct QmvTokEntry {
    QmvVariant v;  // m = most activation rows, rows = sets of weight rows per wavefront, waves = wavefronts that share K
                   // (16-token form: depth = sets of rows in flight, xmode = runs of 256 codes a wavefront holds per pass)
    QmvTokKernel fn;
    int wg_rows;  // weight rows per workgroup
    int lds;      // bytes
};
#define AQ_QMVT(NW, R)                                                                               \
    {                                                                                                \
        {"qmvt_b4_m32_r" #R "_w" #NW, 4, kTokMax, R, NW, 4, 0, 0, 6}, qmv_tok_kernel<NW, R>,         \
            kTokRows * R, NW * R * 16 * 64 * 4                                                       \
    }
#define AQ_QMVT16(NW, RS, QW, RING)                                                                       \
    {                                                                                                     \
        {"qmvt_b4_m16_r" #RS "_w" #NW "_q" #QW "_d" #RING, 4, 16, RS, NW, RING, 0, QW, 6},                 \
            qmv_tok16_kernel<NW, RS, QW, RING>, 16 * RS, NW * 16 * (16 * RS) * 4                          \
    }
static const QmvTokEntry kQmvTokTable[] = {AQ_QMVT(8, 2), AQ_QMVT(8, 1), AQ_QMVT(4, 1), AQ_QMVT(4, 2),
                                           AQ_QMVT16(8, 4, 1, 2), AQ_QMVT16(8, 2, 1, 2), AQ_QMVT16(8, 1, 1, 1),
                                           AQ_QMVT16(16, 4, 1, 3), AQ_QMVT16(8, 4, 2, 2)};

int qmvt_variant_count() { return (int)(sizeof(kQmvTokTable) / sizeof(kQmvTokTable[0])); }
const QmvVariant* qmvt_variant(int idx) {
    if (idx < 0 || idx >= qmvt_variant_count()) return nullptr;
    return &kQmvTokTable[idx].v;
}

bool qmvt_fits(const QmvArgs& a, int bits, int group_size, int idx) {
    const QmvVariant* v = qmvt_variant(idx);
    if (!v || bits != 4 || group_size != 64) return false;
    if (a.M < 1 || a.M > v->m || a.N < 1 || a.K < 256 || a.K % 256 != 0) return false;
    const uintptr_t al16 = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.w);
    const uintptr_t al8 = reinterpret_cast<uintptr_t>(a.s) | reinterpret_cast<uintptr_t>(a.b);
    if ((al16 & 15) || (al8 & 7)) return false;
    // 32-bit byte offsets into the packed matrix and into x
    if ((uint64_t)a.N * (uint64_t)(a.K / 2) >= (1ull << 32)) return false;
    // the 16-token form keeps its rows' scales and biases in LDS next to the partial sums
    if (v->m == 16 && ((size_t)kQmvTokTable[idx].lds + (size_t)kQmvTokTable[idx].wg_rows * (a.K / 256 + 1) * 16 > 160 * 1024 ||
                       kQmvTokTable[idx].wg_rows * (a.K / 256) > tok16_stage_pieces(v->waves) * v->waves * kWave))
        return false;
    return true;
}

hipError_t qmvt_launch(int idx, const QmvArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmvt_variant_count()) return hipErrorInvalidValue;
    const QmvTokEntry& e = kQmvTokTable[idx];
    // the 16-token form also stages 16 bytes of scales and biases per row and run of 256 codes (rows a run apart plus 16 bytes)
    const size_t lds = (size_t)e.lds + (e.v.m == 16 ? (size_t)e.wg_rows * (a.K / 256 + 1) * 16 : 0);
    if (lds > 48 * 1024) {
        hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(e.fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)lds);
        if (rc != hipSuccess) return rc;
    }
    const int wg_rows = e.wg_rows;
    hipLaunchKernelGGL(e.fn, dim3((unsigned)((a.N + wg_rows - 1) / wg_rows)), dim3((unsigned)(e.v.waves * kWave)), lds, stream, a);
    return hipGetLastError();
}

// The variant for this shape, or -1: wavefronts so that each gets at least one run of four groups; two sets of rows per
// wavefront while that still leaves a workgroup for most CUs.
int qmvt_pick(int M, int K, int N, int cu_count) {
    if (M < 1 || M > kTokMax || K < 256 || K % 256 != 0) return -1;
    const int quads = K / 256;
    const int cus = cu_count > 0 ? cu_count : 256;
    if (M <= 16 && K <= 16384) {
        // the 16-token form: eight wavefronts, one run each per pass; as many sets of 16 rows per workgroup (fewer reads
        // of x) as still leave three quarters of the CUs a workgroup
        const int rs = (N + 63) / 64 >= (cus * 3) / 4 ? 4 : (N + 31) / 32 >= (cus * 3) / 4 ? 2 : 1;
        for (int i = 0; i < qmvt_variant_count(); i++) {
            const QmvVariant& v = kQmvTokTable[i].v;
            if (v.m == 16 && v.waves == 8 && v.rows == rs && v.xmode == 1) return i;
        }
    }
    const int nw = quads >= 8 ? 8 : 4;
    const int r = (N + 63) / 64 >= (cus * 3) / 4 ? 2 : 1;
    for (int i = 0; i < qmvt_variant_count(); i++) {
        const QmvVariant& v = kQmvTokTable[i].v;
        if (v.m == kTokMax && v.waves == nw && v.rows == r) return i;
    }
    return -1;
}

}  // namespace aq
