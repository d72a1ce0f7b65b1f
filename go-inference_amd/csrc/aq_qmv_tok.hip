// affine_qmv for 5..32 rows of x on gfx950 (batched / speculative-verify decode), 4- and 8-bit codes in
// groups of 64: one launch, the weights streamed exactly once, no pass over x beforehand and no partial tiles in memory.
//
// Same contract as the other matvec kernels: replaces rocm_mlx_q4_projection_batch*
// (go/engine/hip/kernels/quant/affine_projection_tuned.hipinc:292-472, 16 rows x 16 tokens in one launch) and the
// rows kernel of go/engine/metal/qmv_rows.go:14-60; semantics of MLX affine_qmv with M rows
// (go/engine/metal/kernels/quant/lthn_qmv_rows.metal:1-22).
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
// The same with the non-temporal hint, for the weights: they are read once, in whole 128-byte lines per instruction, and
// leave the L1 to x, scales and biases (4096 x 14336, 16 / 32 rows of x: 12.65 -> 12.28 / 17.14 -> 16.8 us).
__device__ __forceinline__ uint4 load_u128_stream_at(gptr_t base, uint32_t off) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x4_t*>(base + off));
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

constexpr int kTokMax = 32;   // activation rows per launch (the M side)
// 8-byte pieces of scales (and of biases) a thread of the 16-token form stages at most: K up to 16384 with 16 wavefronts
__host__ __device__ constexpr int tok16_stage_pieces(int nw) { return nw >= 16 ? 4 : 8; }

}  // namespace

// v_mfma_f32_16x16x32_bf16 with 16 tokens as the rows of A (TS such sets per expanded weight: up to 16 TS rows of x) and
// 16 weight rows as the columns of B.  A workgroup of NW wavefronts owns RS sets of 16 weight rows; wavefront w takes
// the runs of 256 codes w, w + NW, ... of all of them, QW runs per pass.
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
//   * a wavefront keeps the A operands of its runs in registers and streams the sets of rows past them, RING sets in
//     flight (see the loop); the wavefronts' partial sums meet in LDS.
// Token t of an M-row call equals token t of any other call on the same variant, bit for bit.
// 8-bit codes (BITS = 8): a run of 256 codes is two lines per row, four loads per set of rows; the 64 bytes a
// 16-lane-block row holds after the DPP moves are one quantisation group, lane (n, p) has its codes 16 p .. 16 p + 15, and
// the two halves of those are the B operands of the group's two steps as they lie (no transpose: which codes share a
// step is free as long as x follows, and x is loaded to follow: lane (t, p) takes x[64 g + 16 p + 8 i ..] for step i);
// codes become bf16 by v_cvt_f32_ubyte + v_perm (exact), in their natural order; the affine term is bias * sum(x) alone.
template <int BITS, int NW, int RS, int QW, int RING, int TS>
__global__ __launch_bounds__(NW* kWave) void qmv_tok16_kernel(const QmvArgs a) {
    static_assert(BITS == 4 || BITS == 8, "code width");
    constexpr int LINES = BITS / 4;  // 128-byte lines of a row per run of 256 codes
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
            w_lane[rs][ab] = (uint32_t)row * (uint32_t)(K * BITS / 8) + (uint32_t)(n >> 3) * 64u + (uint32_t)q * 16u;
        }
    // x: lane (i, q) of load `ab` of token set ts reads token 16 ts + (i % 8) + 8 ab, bytes 64 (i / 8) + 16 q of a
    // 128-byte step pair (TS sets of 16 tokens share every expanded weight)
    uint32_t x_lane[TS][2];
#pragma unroll
    for (int ts = 0; ts < TS; ts++)
#pragma unroll
        for (int ab = 0; ab < 2; ab++)
            x_lane[ts][ab] = (uint32_t)min(16 * ts + (n & 7) + 8 * ab, M - 1) * (uint32_t)K * 2u +
                             (BITS == 4 ? (uint32_t)(n >> 3) * 64u + (uint32_t)q * 16u   // step pair: first 64 bytes | second
                                        : (uint32_t)q * 32u + (uint32_t)(n >> 3) * 16u);  // group: first 16 of the lane's 32 | second

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

    f32x4_t acc[RS][TS];
#pragma unroll
    for (int rs = 0; rs < RS; rs++)
#pragma unroll
        for (int ts = 0; ts < TS; ts++) acc[rs][ts] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};

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
    uint4 ring[RING][QW][LINES][2];
    auto issue_set = [&](auto slot_tag, int rs_dyn, const int (&qds)[QW]) {
        constexpr int SL = decltype(slot_tag)::value;
#pragma unroll
        for (int j = 0; j < QW; j++)
#pragma unroll
            for (int ln = 0; ln < LINES; ln++)
#pragma unroll
                for (int ab = 0; ab < 2; ab++) {
                    uint32_t base = 0;
#pragma unroll
                    for (int rs = 0; rs < RS; rs++) base = rs == rs_dyn ? w_lane[rs][ab] : base;
                    ring[SL][j][ln][ab] = load_u128_stream_at(wg, base + (uint32_t)qds[j] * (uint32_t)(128 * LINES) + (uint32_t)ln * 128u);
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
        uint4 xa[TS][QW][4], xb[TS][QW][4];
#pragma unroll
        for (int ts = 0; ts < TS; ts++)
#pragma unroll
            for (int j = 0; j < QW; j++)
#pragma unroll
                for (int sp = 0; sp < 4; sp++) {
                    xa[ts][j][sp] = load_u128_at(xg, x_lane[ts][0] + (uint32_t)qds[j] * 512u + (uint32_t)sp * 128u);
                    xb[ts][j][sp] = load_u128_at(xg, x_lane[ts][1] + (uint32_t)qds[j] * 512u + (uint32_t)sp * 128u);
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
        bf16x8_t af[TS][QW][8], a2[TS][QW];
#pragma unroll
        for (int ts = 0; ts < TS; ts++)
#pragma unroll
        for (int j = 0; j < QW; j++) {
            float ps[4];
#pragma unroll
            for (int st = 0; st < 8; st++) {
                // even step: lanes i >= 8 take tokens 8..15 from the second load's lanes i - 8; odd step: lanes i < 8 take
                // tokens 0..7 from the first load's lanes i + 8
                const uint4 va = xa[ts][j][st >> 1], vb = xb[ts][j][st >> 1];
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
                if constexpr (BITS == 4) {  // the order the expansion leaves the codes of a word in: 0 4 1 5 2 6 3 7
                    af[ts][j][st] = as_bf16x8(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                                              __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
                } else {
                    af[ts][j][st] = as_bf16x8(v.x, v.y, v.z, v.w);
                }
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
            // 4 bit: the expanded codes are 128 + code
            const float off = BITS == 4 ? -128.0f : 0.0f;
            const uint32_t m0 = __float_as_uint(off * __uint_as_float(u0));
            const uint32_t m1 = __float_as_uint(off * __uint_as_float(u1));
            const uint32_t m2 = __float_as_uint(off * __uint_as_float(u2));
            a2[ts][j] = as_bf16x8((u0 >> 16) | u1, (u2 >> 16) | m0, (m1 >> 16) | m2, 0u);
        }

        auto run_set = [&](auto rs_tag) {
            constexpr int rs = decltype(rs_tag)::value;
            constexpr int SL = rs % RING;
#pragma unroll
            for (int j = 0; j < QW; j++) {
                // first 64 bytes of all 16 rows (lanes i >= 8 from the second load's lanes i - 8), second 64 bytes (lanes
                // i < 8 from the first load's lanes i + 8): as for x
                uint32_t ww[8 * LINES];  // 4 bit: the word of step st; 8 bit: the two words of step st at 2 st, 2 st + 1
#pragma unroll
                for (int ln = 0; ln < LINES; ln++) {
                    const uint4 la = ring[SL][j][ln][0], lb = ring[SL][j][ln][1];
                    uint32_t f0 = __builtin_amdgcn_update_dpp(la.x, lb.x, 0x118, 0xf, 0xc, false);
                    uint32_t f1 = __builtin_amdgcn_update_dpp(la.y, lb.y, 0x118, 0xf, 0xc, false);
                    uint32_t f2 = __builtin_amdgcn_update_dpp(la.z, lb.z, 0x118, 0xf, 0xc, false);
                    uint32_t f3 = __builtin_amdgcn_update_dpp(la.w, lb.w, 0x118, 0xf, 0xc, false);
                    uint32_t g0 = __builtin_amdgcn_update_dpp(lb.x, la.x, 0x108, 0xf, 0x3, false);
                    uint32_t g1 = __builtin_amdgcn_update_dpp(lb.y, la.y, 0x108, 0xf, 0x3, false);
                    uint32_t g2 = __builtin_amdgcn_update_dpp(lb.z, la.z, 0x108, 0xf, 0x3, false);
                    uint32_t g3 = __builtin_amdgcn_update_dpp(lb.w, la.w, 0x108, 0xf, 0x3, false);
                    if constexpr (BITS == 4) {
                        transpose(f0, f1, f2, f3);
                        transpose(g0, g1, g2, g3);
                    }
                    const uint32_t both[8] = {f0, f1, f2, f3, g0, g1, g2, g3};
#pragma unroll
                    for (int k = 0; k < 8; k++) ww[8 * ln + k] = both[k];
                }
                const uint4 sbv = sbq[(rs * 16 + n) * sb_pitch + qds[j]];
                f32x4_t part[TS];
#pragma unroll
                for (int ts = 0; ts < TS; ts++) part[ts] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    f32x4_t d[TS];
#pragma unroll
                    for (int ts = 0; ts < TS; ts++) d[ts] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int half = 0; half < 2; half++) {
                        uint32_t e[4];
                        if constexpr (BITS == 4) {
                            unpack4_word(ww[2 * g + half], mask, magic, e);
                        } else {
                            unpack8_word(ww[4 * g + 2 * half], e);
                            unpack8_word(ww[4 * g + 2 * half + 1], e + 2);
                        }
                        const bf16x8_t bop = as_bf16x8(e[0], e[1], e[2], e[3]);
#pragma unroll
                        for (int ts = 0; ts < TS; ts++)
                            d[ts] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[ts][j][2 * g + half], bop, d[ts], 0, 0, 0);
                    }
                    const uint32_t sw = g < 2 ? sbv.x : sbv.y;
                    const float sc = (g & 1) ? __uint_as_float(sw & 0xffff0000u) : __uint_as_float(sw << 16);
#pragma unroll
                    for (int ts = 0; ts < TS; ts++)
#pragma unroll
                        for (int r = 0; r < 4; r++) part[ts][r] = __builtin_fmaf(sc, d[ts][r], part[ts][r]);
                }
                const uint32_t bb = __builtin_amdgcn_perm(sbv.w, sbv.z, sel_q);
                const uint32_t ss = __builtin_amdgcn_perm(sbv.y, sbv.x, sel_q);
                const bf16x8_t b2 = as_bf16x8(bb, __builtin_amdgcn_perm(ss, bb, 0x05040100u), ss, 0u);
#pragma unroll
                for (int ts = 0; ts < TS; ts++) part[ts] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2[ts][j], b2, part[ts], 0, 0, 0);
                // a run past the end of K (x and weights of the last run were loaded in its place) adds nothing
                if (live[j]) {
#pragma unroll
                    for (int ts = 0; ts < TS; ts++)
#pragma unroll
                        for (int r = 0; r < 4; r++) acc[rs][ts][r] += part[ts][r];
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
    // D layout of the 16x16 MFMA: lane (n, q), register r -> token 4 q + r (of its set), weight row n
#pragma unroll
    for (int rs = 0; rs < RS; rs++)
#pragma unroll
        for (int ts = 0; ts < TS; ts++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[(wave * 16 * TS + 16 * ts + 4 * q + r) * TSTRIDE + rs * 16 + n] = acc[rs][ts][r];
    __syncthreads();
    for (int o = tid; o < 16 * TS * ROWS; o += NW * kWave) {
        const int t = o / ROWS, rl = o - t * ROWS;
        float total = red[t * TSTRIDE + rl];
#pragma unroll
        for (int p = 1; p < NW; p++) total += red[(p * 16 * TS + t) * TSTRIDE + rl];
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
#define AQ_QMVT16B(BITS, NW, RS, QW, RING)                                                                \
    {                                                                                                     \
        {"qmvt_b" #BITS "_m16_r" #RS "_w" #NW "_q" #QW "_d" #RING, BITS, 16, RS, NW, RING, 0, QW, 6},      \
            qmv_tok16_kernel<BITS, NW, RS, QW, RING, 1>, 16 * RS, NW * 16 * (16 * RS) * 4                 \
    }
#define AQ_QMVT16(NW, RS, QW, RING) AQ_QMVT16B(4, NW, RS, QW, RING)
// the same with two sets of 16 tokens per expanded weight: up to 32 rows of x
#define AQ_QMVT16X2B(BITS, NW, RS, QW, RING)                                                              \
    {                                                                                                     \
        {"qmvt_b" #BITS "_m32_s2_r" #RS "_w" #NW "_q" #QW "_d" #RING, BITS, 32, RS, NW, RING, 0, QW, 6},   \
            qmv_tok16_kernel<BITS, NW, RS, QW, RING, 2>, 16 * RS, NW * 32 * (16 * RS) * 4                 \
    }
#define AQ_QMVT16X2(NW, RS, QW, RING) AQ_QMVT16X2B(4, NW, RS, QW, RING)
static const QmvTokEntry kQmvTokTable[] = {AQ_QMVT16(8, 4, 1, 2), AQ_QMVT16(8, 2, 1, 2), AQ_QMVT16(8, 1, 1, 1),
                                           AQ_QMVT16X2(8, 4, 1, 2), AQ_QMVT16X2(8, 2, 1, 2), AQ_QMVT16X2(8, 1, 1, 1),
                                           AQ_QMVT16B(8, 8, 4, 1, 2), AQ_QMVT16B(8, 8, 2, 1, 2), AQ_QMVT16B(8, 8, 1, 1, 1),
                                           AQ_QMVT16X2B(8, 8, 4, 1, 2), AQ_QMVT16X2B(8, 8, 2, 1, 2), AQ_QMVT16X2B(8, 8, 1, 1, 1)};

int qmvt_variant_count() { return (int)(sizeof(kQmvTokTable) / sizeof(kQmvTokTable[0])); }
const QmvVariant* qmvt_variant(int idx) {
    if (idx < 0 || idx >= qmvt_variant_count()) return nullptr;
    return &kQmvTokTable[idx].v;
}

bool qmvt_fits(const QmvArgs& a, int bits, int group_size, int idx) {
    const QmvVariant* v = qmvt_variant(idx);
    if (!v || bits != v->bits || group_size != 64) return false;
    // (K up to 16384, as qmvt_pick has it: what the tests cover; longer rows go to the kernels that split K)
    if (a.M < 1 || a.M > v->m || a.N < 1 || a.K < 256 || a.K % 256 != 0 || a.K > 16384) return false;
    const uintptr_t al16 = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.w);
    const uintptr_t al8 = reinterpret_cast<uintptr_t>(a.s) | reinterpret_cast<uintptr_t>(a.b);
    if ((al16 & 15) || (al8 & 7)) return false;
    // 32-bit byte offsets into the packed matrix and into x
    if ((uint64_t)a.N * (uint64_t)(a.K * bits / 8) >= (1ull << 32)) return false;
    // the 16-token form keeps its rows' scales and biases in LDS next to the partial sums
    if (((size_t)kQmvTokTable[idx].lds + (size_t)kQmvTokTable[idx].wg_rows * (a.K / 256 + 1) * 16 > 160 * 1024 ||
                       kQmvTokTable[idx].wg_rows * (a.K / 256) > tok16_stage_pieces(v->waves) * v->waves * kWave))
        return false;
    return true;
}

hipError_t qmvt_launch(int idx, const QmvArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmvt_variant_count()) return hipErrorInvalidValue;
    const QmvTokEntry& e = kQmvTokTable[idx];
    // the 16-token form also stages 16 bytes of scales and biases per row and run of 256 codes (rows a run apart plus 16 bytes)
    const size_t lds = (size_t)e.lds + (size_t)e.wg_rows * (a.K / 256 + 1) * 16;
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e.fn), (size_t)lds)) return rc;
    const int wg_rows = e.wg_rows;
    hipLaunchKernelGGL(e.fn, dim3((unsigned)((a.N + wg_rows - 1) / wg_rows)), dim3((unsigned)(e.v.waves * kWave)), lds, stream, a);
    return hipGetLastError();
}

// The variant for this shape, or -1.
int qmvt_pick(int bits, int M, int K, int N, int cu_count) {
    if (M < 1 || M > kTokMax || K < 256 || K % 256 != 0) return -1;
    const int cus = cu_count > 0 ? cu_count : 256;
    if (K > 16384) return -1;
    // eight wavefronts, one run each per pass; one set of 16 tokens up to 16 rows of x, else two; as many sets of 16
    // weight rows per workgroup (fewer reads of x) as still leave three quarters of the CUs a workgroup
    const int most = M <= 16 ? 16 : 32;
    const int rs = (N + 63) / 64 >= (cus * 3) / 4 ? 4 : (N + 31) / 32 >= (cus * 3) / 4 ? 2 : 1;
    for (int i = 0; i < qmvt_variant_count(); i++) {
        const QmvVariant& v = kQmvTokTable[i].v;
        if (v.bits == bits && v.m == most && v.waves == 8 && v.rows == rs && v.xmode == 1) return i;
    }
    return -1;
}

}  // namespace aq
