// affine_qmm for gfx950, prefill sizes: both operands staged through LDS in MFMA-fragment order.
//
// Replaces rocm_mlx_q4_projection_batch* (go/engine/hip/kernels/quant/affine_projection_tuned.hipinc:166-1109)
// with the semantics of MLX affine_qmm_t (go/engine/metal/quant_seam_backend.go:77-109).  The
// arithmetic is that of aq_qmm.hip: the matrix cores multiply the activations with the exact codes
// (4 bit: 16 + c, 8 bit: c, as bf16), every 64-code block of K ends with out += scale * P in fp32,
// and one extra MFMA per four blocks adds (bias - off*scale) * sum(x) with the sums split into two
// bf16 values.  What changes is how the operands reach the matrix cores:
//   * a small pass over x (qmm_prep_kernel) writes the activations once in A-fragment order
//     (1 KiB per 32 rows x 16 K, lane-major, K already in the order the unpacker emits codes) and
//     the per-block sums as (hi, lo) bf16 pairs.  The main kernel then copies A tiles global -> LDS
//     with global_load_lds_dwordx4: no registers, no VALU work, no LDS write instructions;
//   * the packed weights of a tile are fetched once per workgroup (not once per wavefront) the same way
//     and stay PACKED in LDS (a quarter of the bytes of bf16 fragments: LDS read bandwidth, 128 B/clk/CU,
//     is what bounds 64 x 64 wavefront tiles); a lane reads the 16 bytes that hold its four MFMA steps
//     with one ds_read_b128 and expands them in registers;
//   * no LDS write instruction and no register staging in the main loop, so the only waits on global
//     memory are the explicit "at most this iteration's copies outstanding" before each barrier;
//   * wavefront tiles are 128 x 64 (or 64 x 64): LDS read bandwidth (128 B/clk/CU), not the matrix
//     pipe, bounds smaller ones;
//   * three LDS stages: the copies of block g+2 are issued at the top of iteration g and have two
//     blocks of MFMAs to arrive; one barrier per block;
//   * tiles are numbered so that the workgroups of one XCD (every 8th workgroup) walk one band of
//     rows of x across N: the band's A tile stays in that XCD's L2 while the weights stream by.
#include "aq_device.h"
#include "aq_kernels.h"
#include "aq_lds_copy.h"
#include "aq_qmm.h"

#include "../../include/aq_mi355.h"

#include <type_traits>

namespace aq {

namespace {

constexpr uint32_t kMask16 = 0x00780078u;   // a nibble moved to mantissa bits [6:3]
constexpr uint32_t kMagic16 = 0x41804180u;  // bf16 16.0 in both halves: 16 + code, exact

// 8 codes of one packed word -> 8 bf16 (16 + c) in slot order (c0,c4)(c1,c5)(c2,c6)(c3,c7)
__device__ __forceinline__ uint4 unpack_word4(uint32_t w, uint32_t mask_s, uint32_t magic_v) {
    uint4 v;
    v.x = and_or(w << 3, mask_s, magic_v);
    v.y = and_or(w >> 1, mask_s, magic_v);
    v.z = and_or(w >> 5, mask_s, magic_v);
    v.w = and_or(w >> 9, mask_s, magic_v);
    return v;
}

__device__ __forceinline__ uint4 unpack_words8(uint32_t w0, uint32_t w1) {
    uint32_t p[4];
    unpack8_word(w0, p);
    unpack8_word(w1, p + 2);
    return make_uint4(p[0], p[1], p[2], p[3]);
}

__device__ __forceinline__ uint32_t dup16(uint32_t h) { return (h & 0xffffu) | (h << 16); }

}  // namespace

// ---- pass over x ----------------------------------------------------------------------------
// xf: [mblks][K/16][64 lanes][8] bf16.  Lane (j, h) of fragment (mblk, 4g + t) holds
//     x[32 mblk + j][64 g + 32 h + 8 t + order(0..7)], order = 0,4,1,5,2,6,3,7 at 4 bit, natural at 8 bit:
//     MFMA step t pairs lane half h with the 8 codes number 4h + t of the block, so that the codes a
//     lane needs for its four steps are contiguous in the packed row.
// xs: [mblks * 32][ceil(G/4)][4 blocks][hi, lo] bf16: sum of x over each 64-code block, hi + lo.
// Rows past M are written as zeros.
template <int BITS>
__global__ __launch_bounds__(256) void qmm_prep_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ xf,
                                                        uint16_t* __restrict__ xs, int M, int K, int mblks) {
    const int G = K / 64;
    const int G4 = (G + 3) / 4;
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;  // ((row * G) + g) * 8 + c8
    const int64_t total = (int64_t)mblks * 32 * G * 8;
    if (p >= total) return;  // whole groups of 8 lanes leave together
    const int c8 = (int)(p & 7);
    const int64_t rg = p >> 3;
    const int g = (int)(rg % G);
    const int row = (int)(rg / G);
    uint4 v = {0u, 0u, 0u, 0u};
    if (row < M) v = *reinterpret_cast<const uint4*>(x + (int64_t)row * K + g * 64 + c8 * 8);
    float sx = 0.0f;
    sx = dot2_bf16(v.x, 0x3F803F80u, sx);
    sx = dot2_bf16(v.y, 0x3F803F80u, sx);
    sx = dot2_bf16(v.z, 0x3F803F80u, sx);
    sx = dot2_bf16(v.w, 0x3F803F80u, sx);
    // the 8 lanes that hold one row's block: xor 1, xor 2, mirror within 8
    sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0xB1, 0xF, 0xF, true));
    sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0x4E, 0xF, 0xF, true));
    sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0x141, 0xF, 0xF, true));
    if (c8 == 0) {
        const uint32_t hi = f32_to_bf16_bits(sx);
        const uint32_t lo = f32_to_bf16_bits(sx - bf16_bits_to_f32(hi));
        uint32_t* dst = reinterpret_cast<uint32_t*>(xs) + ((int64_t)row * G4 + (g >> 2)) * 4;
        dst[g & 3] = hi | (lo << 16);
        if (g == G - 1)
            for (int q = (g & 3) + 1; q < 4; q++) dst[q] = 0u;
    }
    if constexpr (BITS == 4) {
        uint4 o;
        o.x = (v.x & 0xffffu) | (v.z << 16);
        o.y = (v.x >> 16) | (v.z & 0xffff0000u);
        o.z = (v.y & 0xffffu) | (v.w << 16);
        o.w = (v.y >> 16) | (v.w & 0xffff0000u);
        v = o;
    }
    const int t = c8 & 3, h = c8 >> 2;
    const int64_t frag = (int64_t)(row >> 5) * (K / 16) + g * 4 + t;
    *reinterpret_cast<uint4*>(xf + (frag * 64 + h * 32 + (row & 31)) * 8) = v;
}

// ---- main kernel ----------------------------------------------------------------------------
// Wavefront tiles of at most 64 x 64 keep under 256 registers, so two wavefronts share a SIMD.
template <int BITS, int MB, int NB, int WM, int WN, int STAGES>
__global__ __launch_bounds__(WM* WN* kWave, 2) void qmm_tile_kernel(const QmmTileArgs a) {
    static_assert(STAGES == 3 || STAGES == 4, "LDS stages");
    constexpr int AHEAD = STAGES - 1;  // iteration g requests block g + AHEAD
    constexpr int BST = STAGES;  // LDS stages of packed codes
    constexpr int BM = WM * MB * 32;
    constexpr int BN = WN * NB * 32;
    constexpr int NWAVE = WM * WN;
    constexpr int NT = NWAVE * kWave;
    constexpr int A_STAGE = (BM / 32) * 4096;
    constexpr int B_STAGE = BN * (BITS == 4 ? 32 : 64);  // packed codes of one 64-code block
    constexpr int A_BLOCKS = (BM / 32) * 4;        // 1 KiB fragments of A per stage
    constexpr int WPB = BITS == 4 ? 8 : 16;        // packed words per row and 64-code block
    constexpr int W_PIECES = BN * WPB / 4;         // 16-byte pieces of packed weights per stage
    constexpr int WPT = W_PIECES / NT;             // per thread
    constexpr float OFFSET = BITS == 4 ? 16.0f : 0.0f;
    static_assert(A_BLOCKS % NWAVE == 0, "A fragments must divide among the wavefronts");
    static_assert(W_PIECES % NT == 0 && WPT >= 1, "weight pieces must divide among the threads");


    constexpr int NA = A_BLOCKS / NWAVE;  // A copies a wavefront issues per block
    constexpr int GROUP_OPS = NA + WPT;   // LDS copies a wavefront issues per block
    static_assert(W_PIECES % kWave == 0, "a copy instruction moves 64 pieces");

    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* const abuf = lds;                     // [STAGES][A_STAGE]
    uint8_t* const bbuf = lds + STAGES * A_STAGE;  // [BST][B_STAGE]
    // tile of this workgroup: workgroups are dealt to the 8 XCDs round-robin, so every 8th one
    // shares an L2; give each XCD a contiguous run of tiles in row-band-major order
    // With K split (a.ksplit > 1) every tile is computed by ksplit workgroups, each over a.gsplit blocks of K,
    // which store fp32 partial tiles; the grid is then ksplit times as large.
    const int tiles = a.tiles_m * a.tiles_n;
    const int T = tiles * a.ksplit;
    const int per_xcd = (T + 7) / 8;
    const int id = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (id >= T) return;
    const int split = id / tiles;
    const int tile = id - split * tiles;
    const int tm = tile / a.tiles_n;
    const int tn = tile - tm * a.tiles_n;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int wave_m = wave / WN;
    const int wave_n = wave % WN;
    const int j = lane & 31;
    const int h = lane >> 5;

    const int K = a.K, M = a.M, N = a.N;
    const int Gall = K / 64;
    const int G4 = (Gall + 3) / 4;
    const int gb = split * a.gsplit;                  // first block of K this workgroup multiplies (a multiple of 4)
    const int G = min(Gall, gb + a.gsplit);           // one past its last block
    const int ksteps = K / 16;
    const int sb_per_row = Gall / a.gs_blocks;
    const int64_t words_per_row = (int64_t)K * BITS / 32;
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    // A: this wavefront copies fragments wave, wave + NWAVE, ... of every stage
    auto issue_a = [&](int g, int stage) {
        uint8_t* dst = abuf + stage * A_STAGE;
#pragma unroll
        for (int q = 0; q < A_BLOCKS / NWAVE; q++) {
            const int blk = wave + q * NWAVE;
            int mblk = m0 / 32 + (blk >> 2);
            mblk = mblk < a.mblks ? mblk : a.mblks - 1;  // past the end: any valid rows, never stored
            const uint16_t* src = a.xf + ((int64_t)mblk * ksteps + g * 4 + (blk & 3)) * 512;
            copy16_to_lds(src, (uint32_t)lane * 16u, lds_offset(dst + blk * 1024));
        }
    };

    // B: the tile's packed rows, 16-byte pieces; copy instruction i of this wavefront moves pieces
    // (i * NWAVE + wave) * 64 + lane to consecutive LDS slots, which leaves row r at r * (WPB * 4) bytes
    // (rows past N repeat the last row; a tile spans well under 4 GiB, so the lane part fits 32 bits)
    const uint32_t* const wtile = a.w + (int64_t)min(n0, N - 1) * words_per_row;
    uint32_t woff[WPT];
#pragma unroll
    for (int i = 0; i < WPT; i++) {
        const int p = (i * NWAVE + wave) * kWave + lane;
        constexpr int PPR = WPB / 4;  // pieces per row
        const int r = p / PPR, q = p % PPR;
        const int n = min(n0 + r, N - 1);
        woff[i] = (uint32_t)(n - min(n0, N - 1)) * (uint32_t)(words_per_row * 4) + (uint32_t)q * 16u;
    }
    auto issue_b = [&](int g, int stage) {
        uint8_t* dst = bbuf + stage * B_STAGE;
#pragma unroll
        for (int i = 0; i < WPT; i++)
            copy16_to_lds(wtile + (int64_t)g * WPB, woff[i], lds_offset(dst + (i * NWAVE + wave) * 1024));
    };
    const uint32_t mask_s = opaque_s(kMask16);
    const uint32_t magic_v = opaque_v(kMagic16);

    // Scales, biases and block sums are fetched per QUAD of four 64-code blocks, one quad ahead: the bf16
    // bits of the quad's four blocks in two words per array and column tile (8-byte loads where the
    // rows allow it), and 16 bytes of (hi, lo) sums per row tile.
    const uint16_t* srow[NB];
    const uint16_t* brow[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int n = min(n0 + (wave_n * NB + nb) * 32 + j, N - 1);
        srow[nb] = a.s + (int64_t)n * sb_per_row;
        brow[nb] = a.b + (int64_t)n * sb_per_row;
    }
    const bool quad_loads = a.gs_blocks == 1 && (G & 3) == 0 && (((uintptr_t)a.s | (uintptr_t)a.b) & 7) == 0;
    uint2 s_cur[NB], b_cur[NB], s_nxt[NB], b_nxt[NB];
    auto load_quad = [&](int quad, uint2 (&sd)[NB], uint2 (&bd)[NB]) {
        if (quad_loads) {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                sd[nb] = *reinterpret_cast<const uint2*>(srow[nb] + quad * 4);
                bd[nb] = *reinterpret_cast<const uint2*>(brow[nb] + quad * 4);
            }
        } else {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                uint32_t sv[4], bv[4];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    int idx = (quad * 4 + k) / a.gs_blocks;
                    idx = idx < sb_per_row ? idx : sb_per_row - 1;  // blocks past K: never used
                    sv[k] = srow[nb][idx];
                    bv[k] = brow[nb][idx];
                }
                sd[nb] = make_uint2(sv[0] | (sv[1] << 16), sv[2] | (sv[3] << 16));
                bd[nb] = make_uint2(bv[0] | (bv[1] << 16), bv[2] | (bv[3] << 16));
            }
        }
    };
    // bf16 bits of block q (0..3) of a quad, as the high half of a word (= the fp32 value)
    auto quad_hi = [](const uint2& v, int q) {
        const uint32_t w = q < 2 ? v.x : v.y;
        return (q & 1) ? (w & 0xffff0000u) : (w << 16);
    };
    const uint4* xsrow[MB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        int row = m0 + (wave_m * MB + mb) * 32 + j;
        row = row < a.mblks * 32 ? row : a.mblks * 32 - 1;
        xsrow[mb] = reinterpret_cast<const uint4*>(a.xs) + (int64_t)row * G4;
    }
    uint4 xs_cur[MB], xs_nxt[MB];
    auto load_xs = [&](int quad, uint4 (&dst)[MB]) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++) dst[mb] = xsrow[mb][quad];
    };

    f32x16_t out[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) out[mb][nb][r] = 0.0f;

    // One 64-code block; Q = g & 3 is static so that everything indexed by it stays in fixed
    // registers.  The packed words alternate between two register sets, and nothing that is still in
    // flight is ever copied (a copy would wait for the newest load).  Iteration g requests the packed
    // words of block g+2 before its MFMAs (at Q = 1 also the next quad's scales, biases and sums), and
    // the A copies of block g+2 after its LDS writes: the compiler drains every outstanding copy into
    // LDS before an LDS write it cannot tell apart from the copy's target, so a copy issued earlier
    // would be waited for in the same iteration.  Each request has one block of MFMAs to arrive.  Past
    // the end of K the last block is requested again.
    const int glast = G - 1;
    int sa = 0;  // LDS stage of A that holds block g
    auto iteration = [&](auto q_tag, int g) {
        constexpr int Q = decltype(q_tag)::value;
        const bool more = g + 1 < G;
        if constexpr (Q == 0) {
            // the quad's scales, biases and sums were requested three blocks ago (the first quad: before
            // the loop).  Taken over here, before this iteration's copies are issued: the compiler waits
            // for every request it cannot count before the first use of a loaded register.
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                s_cur[nb] = s_nxt[nb];
                b_cur[nb] = b_nxt[nb];
            }
#pragma unroll
            for (int mb = 0; mb < MB; mb++) xs_cur[mb] = xs_nxt[mb];
        }
        if constexpr (Q == 1) {
            // ordinary loads first: the wait at the end of the iteration counts the copies behind them
            const int nq = (g >> 2) + 1 < G4 ? (g >> 2) + 1 : G4 - 1;
            load_quad(nq, s_nxt, b_nxt);
            load_xs(nq, xs_nxt);
        }
        {
            const int g2 = g + AHEAD < G ? g + AHEAD : glast;
            const int s2 = sa == 0 ? STAGES - 1 : sa - 1;  // stage (sa + AHEAD) % STAGES: read last in iteration g-1
            issue_a(g2, s2);
            issue_b(g2, s2);
        }

        const uint8_t* ab = abuf + sa * A_STAGE + (wave_m * MB) * 4096 + lane * 16;
        // this lane's codes: row (wave_n * NB + nb) * 32 + j, words 4h .. 4h+3 (8 bit: 8h .. 8h+7)
        const uint8_t* bb = bbuf + sa * B_STAGE + ((wave_n * NB) * 32 + j) * (WPB * 4) + h * (WPB * 2);
        bf16x8_t bfrag[NB][4];
        float sc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            if constexpr (BITS == 4) {
                const uint4 cw = *reinterpret_cast<const uint4*>(bb + nb * 32 * 32);
                bfrag[nb][0] = __builtin_bit_cast(bf16x8_t, unpack_word4(cw.x, mask_s, magic_v));
                bfrag[nb][1] = __builtin_bit_cast(bf16x8_t, unpack_word4(cw.y, mask_s, magic_v));
                bfrag[nb][2] = __builtin_bit_cast(bf16x8_t, unpack_word4(cw.z, mask_s, magic_v));
                bfrag[nb][3] = __builtin_bit_cast(bf16x8_t, unpack_word4(cw.w, mask_s, magic_v));
            } else {
                const uint4 c0 = *reinterpret_cast<const uint4*>(bb + nb * 32 * 64);
                const uint4 c1 = *reinterpret_cast<const uint4*>(bb + nb * 32 * 64 + 16);
                bfrag[nb][0] = __builtin_bit_cast(bf16x8_t, unpack_words8(c0.x, c0.y));
                bfrag[nb][1] = __builtin_bit_cast(bf16x8_t, unpack_words8(c0.z, c0.w));
                bfrag[nb][2] = __builtin_bit_cast(bf16x8_t, unpack_words8(c1.x, c1.y));
                bfrag[nb][3] = __builtin_bit_cast(bf16x8_t, unpack_words8(c1.z, c1.w));
            }
            sc[nb] = __uint_as_float(quad_hi(s_cur[nb], Q));
        }
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            bf16x8_t afrag[4];
#pragma unroll
            for (int t = 0; t < 4; t++) afrag[t] = *reinterpret_cast<const bf16x8_t*>(ab + (mb * 4 + t) * 1024);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                f32x16_t p = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; t++) p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afrag[t], bfrag[nb][t], p, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) out[mb][nb][r] = __fmaf_rn(sc[nb], p[r], out[mb][nb][r]);
            }
        }

        if (Q == 3 || !more) {
            // affine terms of the quad's blocks 0..Q in one MFMA: k-slots (2q, 2q+1) carry
            // (Sx_hi, Sx_lo) of block q on the A side; lanes h=0 pair them with bias, lanes h=1 with
            // -off*scale; blocks past Q (only at the end of K) contribute zeros
            bf16x8_t bbf[NB];
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                uint32_t v[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    if (q <= Q) {
                        const uint32_t neg = __float_as_uint(__uint_as_float(quad_hi(s_cur[nb], q)) * -OFFSET) >> 16;
                        const uint32_t bia = quad_hi(b_cur[nb], q) >> 16;
                        v[q] = dup16(h ? neg : bia);
                    } else {
                        v[q] = 0u;
                    }
                }
                const uint4 u = {v[0], v[1], v[2], v[3]};
                bbf[nb] = __builtin_bit_cast(bf16x8_t, u);
            }
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                const bf16x8_t aa = __builtin_bit_cast(bf16x8_t, xs_cur[mb]);
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    out[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aa, bbf[nb], out[mb][nb], 0, 0, 0);
            }
        }

        sa = sa == STAGES - 1 ? 0 : sa + 1;
        // Block g+1 has landed once at most the copies of the AHEAD-1 newest blocks are outstanding;
        // this iteration's LDS reads have returned.  A bare s_barrier on purpose: __syncthreads() carries
        // a workgroup fence, for which the compiler drains ALL outstanding copies into LDS.
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((AHEAD - 1) * GROUP_OPS) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    // the first quad and blocks 0 .. AHEAD-1 are requested up front
    load_quad(gb >> 2, s_nxt, b_nxt);
    load_xs(gb >> 2, xs_nxt);
#pragma unroll
    for (int d = 0; d < AHEAD; d++) {
        issue_a(gb + d < G ? gb + d : glast, d);
        issue_b(gb + d < G ? gb + d : glast, d);
    }
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((AHEAD - 1) * GROUP_OPS) : "memory");  // block 0 has landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    for (int g = gb; g < G; g += 4) {
        iteration(std::integral_constant<int, 0>{}, g);
        if (g + 1 < G) iteration(std::integral_constant<int, 1>{}, g + 1);
        if (g + 2 < G) iteration(std::integral_constant<int, 2>{}, g + 2);
        if (g + 3 < G) iteration(std::integral_constant<int, 3>{}, g + 3);
    }

    // the copies requested past the end of K must not outlive the wavefront's use of LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // D layout of v_mfma_f32_32x32x*: lane (j, h), register r -> row 8*(r/4) + 4*h + r%4, column j: a lane holds
    // single elements of 16 rows.  Stored as they lie that is one store instruction per element, to 64-byte
    // (bf16) or 128-byte (fp32) pieces of rows, which took a third of a big tile's time and most of a small one's.
    // So every 32-row block goes through a staging area in LDS that belongs to the wavefront (the stages are
    // free: every copy has landed, every read of the loop has returned, and the barrier says so for all
    // wavefronts) and leaves it row-major, eight consecutive columns per lane, as 16-byte stores.  The fp32
    // partial tile of a K split takes the same way into its slot of the workspace.
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    constexpr int CW = NB * 32;       // columns of the wavefront's tile
    constexpr int LPR = CW / 8;       // lanes that share a row, eight columns each
    constexpr int RPP = kWave / LPR;  // rows per pass
    static_assert(NWAVE * 32 * CW * 4 <= STAGES * A_STAGE + BST * B_STAGE, "staging area fits the stages");
    float* const stage = reinterpret_cast<float*>(lds) + wave * (32 * CW);
    void* const ybase = a.partial ? static_cast<void*>(a.partial + (int64_t)split * M * N) : a.y;
    const bool y_f32 = a.partial != nullptr || a.out_f32 != 0;
    const bool wide = (reinterpret_cast<uintptr_t>(ybase) & 15) == 0 && (y_f32 ? (N & 3) == 0 : (N & 7) == 0);
    const int row_in = lane / LPR, c8 = (lane % LPR) * 8;
    const int n = n0 + wave_n * CW + c8;
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        const int mtop = m0 + (wave_m * MB + mb) * 32;
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) stage[(8 * (r >> 2) + 4 * h + (r & 3)) * CW + nb * 32 + j] = out[mb][nb][r];
#pragma unroll
        for (int p = 0; p < 32 / RPP; p++) {
            const int row = p * RPP + row_in;
            const int m = mtop + row;
            float4 lo = *reinterpret_cast<const float4*>(stage + row * CW + c8);
            float4 hi = *reinterpret_cast<const float4*>(stage + row * CW + c8 + 4);
            if (m >= M || n >= N) continue;
            const int64_t o = (int64_t)m * N + n;
            if (a.gate && !a.partial) gate_mul8(a.gate, a.act, o, n, N, lo, hi);
            if (wide && n + 8 <= N) {
                if (y_f32) {
                    float4* dst = reinterpret_cast<float4*>(reinterpret_cast<float*>(ybase) + o);
                    dst[0] = lo;
                    dst[1] = hi;
                } else {
                    uint4 u;
                    u.x = pack_bf16x2(lo.x, lo.y);
                    u.y = pack_bf16x2(lo.z, lo.w);
                    u.z = pack_bf16x2(hi.x, hi.y);
                    u.w = pack_bf16x2(hi.z, hi.w);
                    *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(ybase) + o) = u;
                }
            } else {
                const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    if (n + e < N) {
                        if (y_f32) {
                            reinterpret_cast<float*>(ybase)[o + e] = v[e];
                        } else {
                            reinterpret_cast<uint16_t*>(ybase)[o + e] = f32_to_bf16_bits(v[e]);
                        }
                    }
                }
            }
        }
    }
}

// ---- variant table ----------------------------------------------------------------------------

typedef void (*QmmTileKernel)(const QmmTileArgs);
struct QmmTileEntry {
    QmmVariant v;
    QmmTileKernel fn;
    int lds_bytes;
};

#define AQ_QMMT(BITS, MB, NB, WM, WN, ST)                                                          \
    {                                                                                             \
        {"qmmt_b" #BITS "_mb" #MB "_nb" #NB "_wm" #WM "_wn" #WN, BITS, MB, NB, WM, WN},           \
            qmm_tile_kernel<BITS, MB, NB, WM, WN, ST>,                                            \
            ST * (WM * MB * 4096) + ST * (WN * NB * 32 * (BITS == 4 ? 32 : 64))                   \
    }
// 128 x 128 workgroup tiles for prefill sizes (8 bit, and 4-bit calls too small for the fp16-operand kernels);
// 32 x 256 and 64 x 256 for calls of fewer than 64 rows whose K the few-rows kernels do not take
#define AQ_QMMT_SET(BITS) AQ_QMMT(BITS, 2, 2, 2, 2, 3), AQ_QMMT(BITS, 1, 2, 1, 4, 3), AQ_QMMT(BITS, 2, 2, 1, 4, 3)

static const QmmTileEntry kQmmTileTable[] = {AQ_QMMT_SET(4), AQ_QMMT_SET(8)};

static int tile_variants() { return (int)(sizeof(kQmmTileTable) / sizeof(kQmmTileTable[0])); }
int qmmt_variant_count() { return tile_variants() + qmmh_variant_count() + qmmf_variant_count(); }
const QmmVariant* qmmt_variant(int idx) {
    if (idx < 0 || idx >= qmmt_variant_count()) return nullptr;
    if (idx < tile_variants()) return &kQmmTileTable[idx].v;
    idx -= tile_variants();
    return idx < qmmh_variant_count() ? qmmh_variant(idx) : qmmf_variant(idx - qmmh_variant_count());
}

// fragments of x, block sums, one fp32 factor per row (the fp16-operand kernels)
size_t qmmt_workspace_bytes(int M, int K) {
    const size_t mblks = ((size_t)M + 31) / 32;
    const size_t g4 = ((size_t)K / 64 + 3) / 4;
    return mblks * 32 * (size_t)K * 2 + mblks * 32 * g4 * 16 + mblks * 32 * 4;
}

// Adds the ksplit partial tiles [ksplit][M*N] in split order and stores bf16 or fp32.
__global__ __launch_bounds__(256) void qmm_splitk_reduce_kernel(const float* __restrict__ partial, int ksplit, int64_t mn,
                                                                 void* __restrict__ y, int out_f32, const float* __restrict__ gate,
                                                                 int act) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < mn; i += (int64_t)gridDim.x * 256) {
        float acc = partial[i];
        for (int s = 1; s < ksplit; s++) acc += partial[(int64_t)s * mn + i];
        if (gate) acc = fmul_unfused(act_value(act, gate[i]), acc);  // the gated-MLP epilogue (QmmArgs::gate)
        if (out_f32) {
            static_cast<float*>(y)[i] = acc;
        } else {
            static_cast<uint16_t*>(y)[i] = f32_to_bf16_bits(acc);
        }
    }
}

size_t qmmt_splitk_bytes(int M, int N, int ksplit) { return ksplit > 1 ? (size_t)ksplit * M * N * 4 : 0; }

hipError_t qmmt_launch(int idx, const QmmArgs& q, void* workspace, hipStream_t stream) {
    return qmmt_launch_splitk(idx, q, workspace, 1, stream);
}

int qmmt_x_kind(int idx) {
    const QmmVariant* v = qmmt_variant(idx);
    if (!v) return kXReadyNone;
    if (idx >= tile_variants() && idx < tile_variants() + qmmh_variant_count()) return kXReadyHalf;
    return v->bits == 4 ? kXReadyTile4 : kXReadyTile8;
}

// ksplit > 1: K/64 must be a multiple of 4 * ksplit; the fp32 partial tiles live in the workspace behind the
// rewritten activations (qmmt_workspace_bytes(M, K) rounded up to 256, then qmmt_splitk_bytes).
hipError_t qmmt_launch_splitk(int idx, const QmmArgs& q, void* workspace, int ksplit, hipStream_t stream) {
    if (idx < 0 || idx >= qmmt_variant_count()) return hipErrorInvalidValue;
    if (idx >= tile_variants() && idx < tile_variants() + qmmh_variant_count())
        return ksplit == 1 ? qmmh_launch(idx - tile_variants(), q, workspace, stream) : hipErrorInvalidValue;
    const int few = idx >= tile_variants() ? idx - tile_variants() - qmmh_variant_count() : -1;
    static const QmmTileEntry kNone{};
    const QmmTileEntry& e = few < 0 ? kQmmTileTable[idx] : kNone;
    const QmmVariant& v = few < 0 ? e.v : *qmmf_variant(few);
    if (ksplit < 1 || (ksplit > 1 && (q.K / 64) % (4 * ksplit) != 0)) return hipErrorInvalidValue;
    const int mblks = (q.M + 31) / 32;
    uint16_t* xf = static_cast<uint16_t*>(workspace);
    uint16_t* xs = xf + (size_t)mblks * 32 * q.K;
    const int64_t pieces = (int64_t)mblks * 32 * (q.K / 64) * 8;
    const unsigned prep_blocks = (unsigned)((pieces + 255) / 256);
    hipError_t rc = hipSuccess;
    if (q.x_ready != (v.bits == 4 ? kXReadyTile4 : kXReadyTile8)) {
        if (v.bits == 4)
            hipLaunchKernelGGL(qmm_prep_kernel<4>, dim3(prep_blocks), dim3(256), 0, stream, q.x, xf, xs, q.M, q.K, mblks);
        else
            hipLaunchKernelGGL(qmm_prep_kernel<8>, dim3(prep_blocks), dim3(256), 0, stream, q.x, xf, xs, q.M, q.K, mblks);
        rc = hipGetLastError();
        if (rc != hipSuccess) return rc;
    }

    QmmTileArgs a{};
    a.xf = xf;
    a.xs = xs;
    a.w = q.w;
    a.s = q.s;
    a.b = q.b;
    a.y = q.y;
    a.M = q.M;
    a.K = q.K;
    a.N = q.N;
    a.gs_blocks = q.gs_blocks;
    a.out_f32 = q.out_f32;
    a.gate = q.gate;
    a.act = q.act;
    a.mblks = mblks;
    const int bm = v.wm * v.mb * 32, bn = v.wn * v.nb * 32;
    a.tiles_m = (q.M + bm - 1) / bm;
    a.tiles_n = (q.N + bn - 1) / bn;
    a.ksplit = ksplit;
    a.gsplit = ksplit > 1 ? (q.K / 64) / ksplit : (q.K / 64 + 3) / 4 * 4;
    a.partial = nullptr;
    if (ksplit > 1) {
        const size_t off = (qmmt_workspace_bytes(q.M, q.K) + 255) & ~(size_t)255;
        a.partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + off);
    }
    const int T = a.tiles_m * a.tiles_n * ksplit;
    const unsigned grid = (unsigned)(((T + 7) / 8) * 8);
    if (few >= 0) {
        rc = qmmf_launch_kernel(few, a, stream);
    } else {
        rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e.fn), (size_t)e.lds_bytes);
        if (rc != hipSuccess) return rc;
        hipLaunchKernelGGL(e.fn, dim3(grid), dim3((unsigned)(e.v.wm * e.v.wn * kWave)), (size_t)e.lds_bytes, stream, a);
        rc = hipGetLastError();
    }
    if (rc != hipSuccess || ksplit == 1) return rc;
    const int64_t mn = (int64_t)q.M * q.N;
    int64_t blocks = (mn + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(qmm_splitk_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a.partial, ksplit, mn, q.y,
                       q.out_f32, q.gate, q.act);
    return hipGetLastError();
}

}  // namespace aq
