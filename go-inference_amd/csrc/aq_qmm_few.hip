// affine_qmm / affine_qmv for 5..64 rows of x on gfx950 (batched and speculative-verify decode): the weights are
// streamed once, K is shared out over workgroups, a small kernel adds the fp32 partial tiles.
//
// Contract and arithmetic are those of the tile kernels of aq_qmm_tile.hip (MLX affine_qmm_t,
// go/engine/metal/quant_seam_backend.go:77-109; the rows kernel of go/engine/metal/qmv_rows.go:14-140 for the row
// counts it names): the matrix cores multiply the activations with the exact codes (4 bit: 16 + c, 8 bit: c, as
// bf16), every 64-code block ends with out += scale * P in fp32, one extra MFMA per four blocks adds
// (bias - off * scale) * sum(x).  With so few rows a 64-code block is a handful of MFMAs, and a loop that waits
// and meets at a barrier once per block spends its time on exactly that (measured with in-kernel timestamps:
// 0.9 us per block, whatever the number of LDS stages).  Here an LDS stage holds a QUAD of four blocks: one wait
// and one barrier per 256 codes of K, the copies of the next quad issued at the top of the current one, and the
// next quad's scales, biases and block sums fetched with ordinary loads at the same point - by the end-of-quad
// wait everything outstanding has landed, so the compiler's own wait at the first use of those registers finds
// nothing to drain.  One workgroup per CU (two stages are 96 to 128 KiB of LDS); workgroup tiles are 32 or 64
// rows by 256 columns (4 bit, eight wavefronts side by side) or 128 columns (8 bit, four).
#include "aq_device.h"
#include "aq_kernels.h"
#include "aq_lds_copy.h"
#include "aq_qmm.h"

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

// Operands: QmmTileArgs as the tile kernels take them (x rewritten by their pass over x; ksplit workgroups per
// tile, each over gsplit blocks of K, a multiple of 4; partial tiles [ksplit][M][N] when ksplit > 1).
// WN wavefronts side by side: four with two column blocks each (4 bit) or eight with one, which puts two
// wavefronts on a SIMD (one's code expansion and scaling under the other's MFMAs) and halves both per wavefront.
template <int BITS, int MB, int WN>
__global__ __launch_bounds__(WN* kWave, 1) void qmm_few_kernel(const QmmTileArgs a) {
    constexpr int NB = BITS == 4 ? 8 / WN : 1;
    static_assert(WN == 4 || (WN == 8 && BITS == 4), "four wavefronts, or eight for 4-bit codes");
    constexpr int BM = MB * 32;
    constexpr int BN = WN * NB * 32;
    constexpr int WPB = BITS == 4 ? 8 : 16;       // packed words per row and 64-code block
    constexpr int A_BLK = MB * 4096;              // fragments of one block
    constexpr int B_BLK = BN * WPB * 4;           // packed codes of one block: 8 KiB either way
    constexpr int A_QUAD = 4 * A_BLK, B_QUAD = 4 * B_BLK;
    constexpr int NA = MB * 16 / WN;              // 1 KiB copies of A per wavefront and quad (MB * 16 fragments)
    constexpr int NBC = B_QUAD / 1024 / WN;       // 1 KiB copies of codes per wavefront and quad
    constexpr float OFFSET = BITS == 4 ? 16.0f : 0.0f;
    static_assert(B_BLK == 8192, "a block of codes is 8 KiB for both widths");

    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* const abuf = lds;               // [2][A_QUAD]
    uint8_t* const bbuf = lds + 2 * A_QUAD;  // [2][B_QUAD]
    const uint32_t abuf_at = __builtin_amdgcn_readfirstlane(lds_offset(lds));
    const uint32_t bbuf_at = abuf_at + 2 * A_QUAD;

    // workgroups are dealt to the 8 XCDs round-robin; every XCD gets a contiguous run of work items, split-major,
    // so that it reads its own range of K of every weight row
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
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // = its column group
    const int j = lane & 31;
    const int h = lane >> 5;

    const int K = a.K, M = a.M, N = a.N;
    const int Gall = K / 64;
    const int G4 = (Gall + 3) / 4;
    const int gb = split * a.gsplit;         // first block of K this workgroup multiplies (a multiple of 4)
    const int G = min(Gall, gb + a.gsplit);  // one past its last block
    const int ksteps = K / 16;
    const int sb_per_row = Gall / a.gs_blocks;
    const int64_t words_per_row = (int64_t)K * BITS / 32;
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    // copies of one quad (blocks 4 * quad .. 4 * quad + 3, clamped to the last block of K) into stage `st`:
    // this wavefront moves fragments wave, wave + 4, ... of the quad's MB * 16, and its share of the code pieces
    const uint32_t* const wtile = a.w + (int64_t)min(n0, N - 1) * words_per_row;
    constexpr int PPR = WPB / 4;  // 16-byte pieces per row and block
    uint32_t woff[NBC / 4];       // per block: NBC / 4 copies, the same rows in every block of the quad
#pragma unroll
    for (int i = 0; i < NBC / 4; i++) {
        const int p = (i * WN + wave) * kWave + lane;  // piece of the block this lane moves
        const int r = p / PPR, q = p % PPR;
        const int n = min(n0 + r, N - 1);
        woff[i] = (uint32_t)(n - min(n0, N - 1)) * (uint32_t)(words_per_row * 4) + (uint32_t)q * 16u;
    }
    auto issue_quad = [&](int quad, int st) {
#pragma unroll
        for (int c = 0; c < NA; c++) {
            const int f = wave + c * WN;     // fragment of the quad: [block q4][row block mb][step t]
            const int q4 = f / (MB * 4), rest = f % (MB * 4);
            const int g = min(quad * 4 + q4, Gall - 1);
            int mblk = m0 / 32 + (rest >> 2);
            mblk = mblk < a.mblks ? mblk : a.mblks - 1;  // past the end: any valid rows, never stored
            const uint16_t* src = a.xf + ((int64_t)mblk * ksteps + g * 4 + (rest & 3)) * 512;
            copy16_to_lds(src, (uint32_t)lane * 16u, abuf_at + (uint32_t)(st * A_QUAD + f * 1024));
        }
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const int g = min(quad * 4 + q4, Gall - 1);
#pragma unroll
            for (int i = 0; i < NBC / 4; i++)
                copy16_to_lds(wtile + (int64_t)g * WPB, woff[i],
                              bbuf_at + (uint32_t)(st * B_QUAD + q4 * B_BLK + (i * WN + wave) * 1024));
        }
    };
    const uint32_t mask_s = opaque_s(kMask16);
    const uint32_t magic_v = opaque_v(kMagic16);

    // scales and biases of a quad: the bf16 bits of its four blocks in two words per array and column block (8-byte
    // loads where the rows allow it); the (hi, lo) block sums of x: 16 bytes per row
    uint32_t sboff[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) sboff[nb] = (uint32_t)min(n0 + (wave * NB + nb) * 32 + j, N - 1) * (uint32_t)sb_per_row;
    const bool quad_loads = a.gs_blocks == 1 && (Gall & 3) == 0 && (((uintptr_t)a.s | (uintptr_t)a.b) & 7) == 0;
    auto load_quad = [&](const uint16_t* base, int quad, uint2 (&dst)[NB]) {
        if (quad_loads) {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) dst[nb] = *reinterpret_cast<const uint2*>(base + sboff[nb] + quad * 4);
        } else {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                uint32_t v[4];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    int idx = (quad * 4 + k) / a.gs_blocks;
                    idx = idx < sb_per_row ? idx : sb_per_row - 1;  // blocks past K: never used
                    v[k] = base[sboff[nb] + idx];
                }
                dst[nb] = make_uint2(v[0] | (v[1] << 16), v[2] | (v[3] << 16));
            }
        }
    };
    auto quad_hi = [](const uint2& v, int q) {
        const uint32_t w = q < 2 ? v.x : v.y;
        return (q & 1) ? (w & 0xffff0000u) : (w << 16);
    };
    uint32_t xsoff[MB];  // in 16-byte units
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        int row = m0 + mb * 32 + j;
        row = row < a.mblks * 32 ? row : a.mblks * 32 - 1;
        xsoff[mb] = (uint32_t)row * (uint32_t)G4;
    }
    uint2 s_cur[NB], b_cur[NB], s_nxt[NB], b_nxt[NB];
    uint4 xs_cur[MB], xs_nxt[MB];
    auto load_all = [&](int quad, uint2 (&s)[NB], uint2 (&b)[NB], uint4 (&xs)[MB]) {
        const int nq = quad < G4 ? quad : G4 - 1;
        load_quad(a.s, nq, s);
        load_quad(a.b, nq, b);
#pragma unroll
        for (int mb = 0; mb < MB; mb++) xs[mb] = reinterpret_cast<const uint4*>(a.xs)[xsoff[mb] + nq];
    };

    f32x16_t out[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) out[mb][nb][r] = 0.0f;

    // Order of the loop, chosen around one fact: the compiler cannot count the copy instructions (inline asm), so
    // wherever it waits for one of its own loads it waits until nothing at all is outstanding.  Scales, biases and
    // block sums of quad q+2 are therefore requested right behind the end-of-quad wait of quad q (nothing in
    // flight, the next copies not yet issued) and first used right behind the end-of-quad wait of quad q+1, which
    // has covered them anyway; the copies of quad q+1 are issued at the top of quad q.
    const int quad0 = gb >> 2, quad_end = (G + 3) >> 2;
    load_all(quad0, s_cur, b_cur, xs_cur);
    load_all(quad0 + 1, s_nxt, b_nxt, xs_nxt);
#pragma unroll
    for (int nb = 0; nb < NB; nb++) asm volatile("" : "+v"(s_cur[nb].x), "+v"(s_cur[nb].y), "+v"(b_cur[nb].x), "+v"(b_cur[nb].y));
#pragma unroll
    for (int mb = 0; mb < MB; mb++) asm volatile("" : "+v"(xs_cur[mb].x), "+v"(xs_cur[mb].y), "+v"(xs_cur[mb].z), "+v"(xs_cur[mb].w));
    __builtin_amdgcn_sched_barrier(0);
    issue_quad(quad0, 0);
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    int st = 0;
    for (int quad = quad0; quad < quad_end; quad++) {
        if (quad + 1 < quad_end) issue_quad(quad + 1, st ^ 1);  // uniform; that stage was read last in the quad before
        const int blocks = min(4, G - quad * 4);  // 4 except where K ends inside a quad
        // one block of the quad in stage st; q static.  A whole quad is written as straight-line code so that the
        // scheduler can run the blocks' independent MFMA chains back to back: with so few rows a block alone is two
        // chains of four dependent MFMAs, and a wavefront that is alone on its SIMD idles between them.
        auto block = [&](auto q_tag) {
            constexpr int q = decltype(q_tag)::value;
            const uint8_t* ab = abuf + st * A_QUAD + q * A_BLK + lane * 16;
            // this lane's codes: row (wave * NB + nb) * 32 + j, words 4h .. 4h+3 (8 bit: 8h .. 8h+7)
            const uint8_t* bb = bbuf + st * B_QUAD + q * B_BLK + ((wave * NB) * 32 + j) * (WPB * 4) + h * (WPB * 2);
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
                sc[nb] = __uint_as_float(quad_hi(s_cur[nb], q));
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
        };
        if (blocks == 4) {
            block(std::integral_constant<int, 0>{});
            block(std::integral_constant<int, 1>{});
            block(std::integral_constant<int, 2>{});
            block(std::integral_constant<int, 3>{});
        } else {
            block(std::integral_constant<int, 0>{});
            if (blocks > 1) block(std::integral_constant<int, 1>{});
            if (blocks > 2) block(std::integral_constant<int, 2>{});
        }
        {
            // affine terms of the quad's blocks in one MFMA: k-slots (2q, 2q+1) carry (Sx_hi, Sx_lo) of block q on
            // the A side; lanes h=0 pair them with the bias, lanes h=1 with -off * scale; blocks past the end of K
            // contribute zeros
            bf16x8_t bbf[NB];
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                uint32_t v[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t neg = __float_as_uint(__uint_as_float(quad_hi(s_cur[nb], q)) * -OFFSET) >> 16;
                    const uint32_t bia = quad_hi(b_cur[nb], q) >> 16;
                    v[q] = q < blocks ? dup16(h ? neg : bia) : 0u;
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
        // the next quad has landed, this quad's LDS reads have returned, and every wavefront knows.  A bare
        // s_barrier on purpose: __syncthreads() carries a fence for which the compiler drains what it knows of.
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        st ^= 1;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            asm volatile("" : "+v"(s_nxt[nb].x), "+v"(s_nxt[nb].y), "+v"(b_nxt[nb].x), "+v"(b_nxt[nb].y));
            s_cur[nb] = s_nxt[nb];
            b_cur[nb] = b_nxt[nb];
        }
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            asm volatile("" : "+v"(xs_nxt[mb].x), "+v"(xs_nxt[mb].y), "+v"(xs_nxt[mb].z), "+v"(xs_nxt[mb].w));
            xs_cur[mb] = xs_nxt[mb];
        }
        __builtin_amdgcn_sched_barrier(0);
        load_all(quad + 2, s_nxt, b_nxt, xs_nxt);  // clamped to the last quad of K
        __builtin_amdgcn_sched_barrier(0);
    }

    // D layout of v_mfma_f32_32x32x*: lane (j, h), register r -> row 8*(r/4) + 4*h + r%4, column j.  Every 32-row
    // block goes through a staging area in LDS that belongs to the wavefront (the stages are free after the last
    // barrier) and leaves it row-major, eight consecutive columns per lane, as 16-byte stores: into y, or as fp32
    // into this workgroup's slot of the partial tiles.
    constexpr int CW = NB * 32;
    constexpr int LPR = CW / 8;
    constexpr int RPP = kWave / LPR;
    float* const stage = reinterpret_cast<float*>(lds) + wave * (32 * CW);
    void* const ybase = a.partial ? static_cast<void*>(a.partial + (int64_t)split * M * N) : a.y;
    const bool y_f32 = a.partial != nullptr || a.out_f32 != 0;
    const bool wide = (reinterpret_cast<uintptr_t>(ybase) & 15) == 0 && (y_f32 ? (N & 3) == 0 : (N & 7) == 0);
    const int row_in = lane / LPR, c8 = (lane % LPR) * 8;
    const int n = n0 + wave * CW + c8;
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        const int mtop = m0 + mb * 32;
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

// ---- launch -----------------------------------------------------------------------------------

struct QmmFewEntry {
    QmmVariant v;
    void (*fn)(const QmmTileArgs);
    int lds_bytes;
};
#define AQ_QMMF(BITS, MB, NB, WN)                                                                                  \
    {                                                                                                              \
        {"qmmf_b" #BITS "_mb" #MB "_nb" #NB "_wm1_wn" #WN, BITS, MB, NB, 1, WN}, qmm_few_kernel<BITS, MB, WN>,     \
            2 * (4 * MB * 4096 + 4 * 8192)                                                                         \
    }
// 4 bit: eight wavefronts (64 x 14336 x 4096: 31.2 us against 34.1 us with four; 32 rows: 23.4 against 25.6 us)
static const QmmFewEntry kQmmFewTable[] = {AQ_QMMF(4, 1, 1, 8), AQ_QMMF(4, 2, 1, 8), AQ_QMMF(8, 1, 1, 4), AQ_QMMF(8, 2, 1, 4)};

int qmmf_variant_count() { return (int)(sizeof(kQmmFewTable) / sizeof(kQmmFewTable[0])); }
const QmmVariant* qmmf_variant(int idx) {
    if (idx < 0 || idx >= qmmf_variant_count()) return nullptr;
    return &kQmmFewTable[idx].v;
}

// `a` as qmmt_launch_splitk fills it for this variant's tile shape (x already rewritten); launches the kernel only
hipError_t qmmf_launch_kernel(int idx, const QmmTileArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmmf_variant_count()) return hipErrorInvalidValue;
    const QmmFewEntry& e = kQmmFewTable[idx];
    if (a.ksplit < 1 || a.gsplit % 4 != 0) return hipErrorInvalidValue;
    const int T = a.tiles_m * a.tiles_n * a.ksplit;
    const unsigned grid = (unsigned)(((T + 7) / 8) * 8);
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e.fn), (size_t)e.lds_bytes)) return rc;
    hipLaunchKernelGGL(e.fn, dim3(grid), dim3((unsigned)(e.v.wn * kWave)), (size_t)e.lds_bytes, stream, a);
    return hipGetLastError();
}

}  // namespace aq
