// affine_qmm for gfx950, 4-bit codes, prefill sizes: the scale rides inside the matrix-core operand.
//
// Same contract as the tile kernels of aq_qmm_tile.hip (MLX affine_qmm_t,
// go/engine/metal/quant_seam_backend.go:77-109; replaces rocm_mlx_q4_projection_batch*,
// go/engine/hip/kernels/quant/affine_projection_tuned.hipinc:166-1109).  Those multiply x with the bare codes
// and pay one fp32 FMA per output element and 64-code block to apply the scale, which keeps the accumulators
// in vector registers and the vector unit as busy as the matrix cores.  Here
//
//     w = scale * code + bias = scale * (code - 8) + (bias + 8 * scale)
//
// and scale * (code - 8) is formed EXACTLY as an fp16 value: a bf16 scale has 8 significant bits, |code - 8| <= 8
// has at most 3 below its leading one, so the product has at most 11 - what fp16 holds.  It is produced by one
// packed fp16 FMA per two codes, (16 + code) * s - 24 * s, with 16 + code built by OR-ing the nibble into the
// mantissa of fp16 16.0 and 24 * s exact (24 = 3 * 8).  The activations are bf16 and therefore exact in fp16 too,
// given the exponent range, which two power-of-two factors take care of: every row of x is scaled so that its
// largest magnitude lies in [2^14, 2^15) and every row of the weights so that its largest scale lies in
// [2^10, 2^11) (elements more than 2^28 below their row's largest lose low bits to fp16's subnormal range: far
// below the fp32 accumulation noise).  The matrix cores then accumulate x * w over all of K with no vector work
// on the accumulators at all, the epilogue multiplies by the two inverse powers of two, and the affine term
// (bias + 8 * scale) * sum(x) still costs one bf16 MFMA per four blocks as in the tile kernels.
// What is left for the vector unit is the expansion of the codes: 12 instructions per packed word, amortised
// over 128 rows of x per wavefront (wavefront tiles 128 x 64: 32 MFMAs per 64-code block, about three vector
// instructions each).
//
// Operand staging is that of the tile kernels: activations rewritten once in A-fragment order (here as fp16,
// one workgroup per row so that the row's largest magnitude is known), A tiles and PACKED weights copied
// global -> LDS by copy instructions three blocks deep, one barrier per block, XCD-aware tile order.
#include "aq_device.h"
#include "aq_kernels.h"
#include "aq_lds_copy.h"
#include "aq_qmm.h"

#include <type_traits>

namespace aq {

namespace {

typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));

constexpr uint32_t kMaskH = 0x03C003C0u;   // a nibble moved to fp16 mantissa bits [9:6]
constexpr uint32_t kMagicH = 0x4C004C00u;  // fp16 16.0 in both halves: 16 + code, exact

// 8 codes of one packed word -> 8 fp16 values s * (code - 8) in slot order (c0,c4)(c1,c5)(c2,c6)(c3,c7)
__device__ __forceinline__ uint4 expand_word(uint32_t w, uint32_t mask_s, uint32_t magic_v, f16x2_t s2, f16x2_t m24) {
    uint4 v;
    v.x = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(f16x2_t, and_or(w << 6, mask_s, magic_v)), s2, m24));
    v.y = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(f16x2_t, and_or(w << 2, mask_s, magic_v)), s2, m24));
    v.z = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(f16x2_t, and_or(w >> 2, mask_s, magic_v)), s2, m24));
    v.w = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(__builtin_bit_cast(f16x2_t, and_or(w >> 6, mask_s, magic_v)), s2, m24));
    return v;
}

__device__ __forceinline__ uint32_t dup16(uint32_t h) { return (h & 0xffffu) | (h << 16); }

// 2^e for the largest finite magnitude `mag` (bf16 bits without the sign) such that mag * 2^e has binary
// exponent `target`; 1 for an all-zero row.  e is kept inside what fp32 powers of two hold.
__device__ __forceinline__ int exponent_shift(uint32_t mag, int target) {
    if (mag == 0) return 0;
    int e = target + 127 - (int)(mag >> 7);
    e = e > 120 ? 120 : e;
    e = e < -120 ? -120 : e;
    return e;
}
__device__ __forceinline__ float pow2f(int e) { return __uint_as_float((uint32_t)(127 + e) << 23); }

}  // namespace

// ---- pass over x ----------------------------------------------------------------------------
// One workgroup per eight rows of x (rows padded to a multiple of 32 are written as zeros).  Thread (r = tid % 8,
// p = tid / 8) works on 16-byte pieces p, p + 64, ... of row r: a load instruction then covers whole 128-byte lines of
// eight rows, and the eight rows' slots of a fragment are 128 contiguous bytes of a store instruction (one row per
// workgroup wrote 16 bytes per kilobyte and took 18 us for 34 MB).
// xf: [mblks][K/16][64 lanes][8] fp16, the A-fragment order of the tile kernels (4-bit slot order), values
//     x * 2^e with e chosen per row;
// xs: [mblks * 32][ceil(G/4)][4 blocks][hi, lo] bf16: 2^e * sum of x over each 64-code block, hi + lo;
// rs: [mblks * 32] fp32: 2^-e.
constexpr int kPrepRows = 8;
constexpr int kPrepThreads = 512;                     // eight wavefronts: 64 pieces of each of the eight rows per pass
constexpr int kPrepStep = kPrepThreads / kPrepRows;   // pieces of a row between a thread's pieces
constexpr int kPrepHold = 8;
__global__ __launch_bounds__(kPrepThreads) void qmmh_prep_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ xf,
                                                         uint16_t* __restrict__ xs, float* __restrict__ rs, int M, int K) {
    const int tid = threadIdx.x;
    const int r = tid & 7, p0 = tid >> 3;
    const int row = (int)blockIdx.x * kPrepRows + r;
    const int G = K / 64;
    const int G4 = (G + 3) / 4;
    const int pieces = K / 8;
    const bool live = row < M;
    __shared__ uint32_t wave_mag[kPrepThreads / kWave][kPrepRows];
    uint32_t mag = 0;
    auto scan = [&](const uint4& v) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t lo = w[i] & 0x7fffu, hi = (w[i] >> 16) & 0x7fffu;
            if (lo < 0x7f80u) mag = max(mag, lo);  // inf and NaN do not set the scale
            if (hi < 0x7f80u) mag = max(mag, hi);
        }
    };
    // up to kPrepHold pieces per thread (K up to 4096) are requested together and stay in registers for the second pass
    const bool held = pieces <= kPrepStep * kPrepHold;
    uint4 hold[kPrepHold];
    if (held) {
#pragma unroll
        for (int i = 0; i < kPrepHold; i++) {
            const int p = p0 + kPrepStep * i;
            hold[i] = make_uint4(0u, 0u, 0u, 0u);
            if (live && p < pieces) hold[i] = *reinterpret_cast<const uint4*>(x + (int64_t)row * K + p * 8);
        }
#pragma unroll
        for (int i = 0; i < kPrepHold; i++) scan(hold[i]);
    } else if (live) {
        for (int p = p0; p < pieces; p += kPrepStep) scan(*reinterpret_cast<const uint4*>(x + (int64_t)row * K + p * 8));
    }
    // the eight threads of a wavefront that share a row are 8 lanes apart
#pragma unroll
    for (int o = 8; o < kWave; o <<= 1) mag = max(mag, (uint32_t)__shfl_xor((int)mag, o, kWave));
    if ((tid & (kWave - 1)) < kPrepRows) wave_mag[tid >> 6][r] = mag;
    __syncthreads();
    mag = 0;
#pragma unroll
    for (int w = 0; w < kPrepThreads / kWave; w++) mag = max(mag, wave_mag[w][r]);
    const int e = exponent_shift(mag, 14);
    const float up = pow2f(e);
    if (tid < kPrepRows) rs[row] = live ? pow2f(-e) : 0.0f;

    auto emit = [&](int p, const uint4& v) {
        const int g = p >> 3, c8 = p & 7;
        float sx = 0.0f;
        sx = dot2_bf16(v.x, 0x3F803F80u, sx);
        sx = dot2_bf16(v.y, 0x3F803F80u, sx);
        sx = dot2_bf16(v.z, 0x3F803F80u, sx);
        sx = dot2_bf16(v.w, 0x3F803F80u, sx);
        // the 8 pieces of a block of this row sit in the 8 lanes r, r + 8, ..., r + 56 of the wavefront
        sx += __shfl_xor(sx, 8, kWave);
        sx += __shfl_xor(sx, 16, kWave);
        sx += __shfl_xor(sx, 32, kWave);
        if (c8 == 0) {
            const float scaled = sx * up;
            const uint32_t hi = f32_to_bf16_bits(scaled);
            const uint32_t lo = f32_to_bf16_bits(scaled - bf16_bits_to_f32(hi));
            uint32_t* dst = reinterpret_cast<uint32_t*>(xs) + ((int64_t)row * G4 + (g >> 2)) * 4;
            dst[g & 3] = hi | (lo << 16);
            if (g == G - 1)
                for (int q = (g & 3) + 1; q < 4; q++) dst[q] = 0u;
        }
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        _Float16 hv[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            hv[2 * i] = (_Float16)(bf16_bits_to_f32(w[i] & 0xffffu) * up);
            hv[2 * i + 1] = (_Float16)(bf16_bits_to_f32(w[i] >> 16) * up);
        }
        // slot order (x0,x4)(x1,x5)(x2,x6)(x3,x7): the order in which expand_word emits the codes of a word
        const f16x8_t o = {hv[0], hv[4], hv[1], hv[5], hv[2], hv[6], hv[3], hv[7]};
        const int t = c8 & 3, h = c8 >> 2;
        const int64_t frag = (int64_t)(row >> 5) * (K / 16) + g * 4 + t;
        *reinterpret_cast<f16x8_t*>(xf + (frag * 64 + h * 32 + (row & 31)) * 8) = o;
    };
    if (held) {
#pragma unroll
        for (int i = 0; i < kPrepHold; i++)
            if (p0 + kPrepStep * i < pieces) emit(p0 + kPrepStep * i, hold[i]);
    } else {
        for (int p = p0; p < pieces; p += kPrepStep) {
            uint4 v = {0u, 0u, 0u, 0u};
            if (live) v = *reinterpret_cast<const uint4*>(x + (int64_t)row * K + p * 8);
            emit(p, v);
        }
    }
}

// ---- main kernel ----------------------------------------------------------------------------
// OCC: wavefronts per SIMD the register budget is cut for (2: 256 registers, 1: 512, the accumulators then live in
// the accumulation half of the register file).
// SPREAD: the copies of the block requested in an iteration are issued a few at a time in front of every row block's
// MFMAs instead of together at the top.
template <int MB, int NB, int WM, int WN, int STAGES, int OCC, bool SPREAD>
__global__ __launch_bounds__(WM* WN* kWave, OCC) void qmmh_kernel(const QmmTileArgs a) {
    static_assert(STAGES == 2 || STAGES == 3 || STAGES == 4, "LDS stages");
    constexpr int AHEAD = STAGES - 1;  // iteration g requests block g + AHEAD
    constexpr int BM = WM * MB * 32;
    constexpr int BN = WN * NB * 32;
    constexpr int NWAVE = WM * WN;
    constexpr int NT = NWAVE * kWave;
    constexpr int A_STAGE = (BM / 32) * 4096;
    constexpr int B_STAGE = BN * 32;         // packed codes of one 64-code block
    constexpr int A_BLOCKS = (BM / 32) * 4;  // 1 KiB fragments of A per stage
    constexpr int WPB = 8;                   // packed words per row and 64-code block
    constexpr int W_PIECES = BN * WPB / 4;   // 16-byte pieces of packed weights per stage
    constexpr int WPT = W_PIECES / NT;       // per thread
    static_assert(A_BLOCKS % NWAVE == 0, "A fragments must divide among the wavefronts");
    static_assert(W_PIECES % NT == 0 && WPT >= 1, "weight pieces must divide among the threads");
    constexpr int NA = A_BLOCKS / NWAVE;  // A copies a wavefront issues per block
    constexpr int GROUP_OPS = NA + WPT;   // LDS copies a wavefront issues per block

    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* const abuf = lds;                     // [STAGES][A_STAGE]
    uint8_t* const bbuf = lds + STAGES * A_STAGE;  // [STAGES][B_STAGE]
    // the same as LDS byte addresses: the copy instructions take theirs from a scalar register, and plain integer
    // arithmetic keeps it on the scalar unit (a pointer would be converted, null check included, per copy)
    const uint32_t abuf_at = __builtin_amdgcn_readfirstlane(lds_offset(lds));
    const uint32_t bbuf_at = abuf_at + STAGES * A_STAGE;

    // workgroups are dealt to the 8 XCDs round-robin, so every 8th one shares an L2; give each XCD a
    // contiguous run of tiles in row-band-major order
    const int T = a.tiles_m * a.tiles_n;
    const int per_xcd = (T + 7) / 8;
    const int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (tile >= T) return;
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
    const int G = K / 64;
    const int G4 = (G + 3) / 4;
    const int ksteps = K / 16;
    const int sb_per_row = G / a.gs_blocks;
    const int64_t words_per_row = (int64_t)K / 8;
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    auto issue_a = [&](int g, int stage) {
#pragma unroll
        for (int q = 0; q < NA; q++) {
            const int blk = wave + q * NWAVE;
            int mblk = m0 / 32 + (blk >> 2);
            mblk = mblk < a.mblks ? mblk : a.mblks - 1;  // past the end: any valid rows, never stored
            const uint16_t* src = a.xf + ((int64_t)mblk * ksteps + g * 4 + (blk & 3)) * 512;
            copy16_to_lds(src, (uint32_t)lane * 16u, abuf_at + (uint32_t)(stage * A_STAGE + blk * 1024));
        }
    };
    // the tile's packed rows in 16-byte pieces; copy instruction i of this wavefront moves pieces
    // (i * NWAVE + wave) * 64 + lane to consecutive LDS slots, which leaves row r at r * 32 bytes
    // (rows past N repeat the last row; a tile spans well under 4 GiB, so the lane part fits 32 bits)
    const uint32_t* const wtile = a.w + (int64_t)min(n0, N - 1) * words_per_row;
    uint32_t woff[WPT];
#pragma unroll
    for (int i = 0; i < WPT; i++) {
        const int p = (i * NWAVE + wave) * kWave + lane;
        const int r = p >> 1, q = p & 1;
        const int n = min(n0 + r, N - 1);
        woff[i] = (uint32_t)(n - min(n0, N - 1)) * (uint32_t)(words_per_row * 4) + (uint32_t)q * 16u;
    }
    auto issue_b = [&](int g, int stage) {
#pragma unroll
        for (int i = 0; i < WPT; i++)
            copy16_to_lds(wtile + (int64_t)g * WPB, woff[i], bbuf_at + (uint32_t)(stage * B_STAGE + (i * NWAVE + wave) * 1024));
    };
    // copy number c (0 .. GROUP_OPS-1) of a block: the A fragments first, then the codes
    auto issue_one = [&](int c, int g, int stage) {
        if (c < NA) {
            const int blk = wave + c * NWAVE;
            int mblk = m0 / 32 + (blk >> 2);
            mblk = mblk < a.mblks ? mblk : a.mblks - 1;
            const uint16_t* src = a.xf + ((int64_t)mblk * ksteps + g * 4 + (blk & 3)) * 512;
            copy16_to_lds(src, (uint32_t)lane * 16u, abuf_at + (uint32_t)(stage * A_STAGE + blk * 1024));
        } else {
            const int i = c - NA;
            copy16_to_lds(wtile + (int64_t)g * WPB, woff[i], bbuf_at + (uint32_t)(stage * B_STAGE + (i * NWAVE + wave) * 1024));
        }
    };
    const uint32_t mask_s = opaque_s(kMaskH);
    const uint32_t magic_v = opaque_v(kMagicH);
    // the first blocks are on their way while the prologue scans the scale rows
#pragma unroll
    for (int d = 0; d < AHEAD; d++) {
        issue_a(d < K / 64 ? d : K / 64 - 1, d);
        issue_b(d < K / 64 ? d : K / 64 - 1, d);
    }

    // this lane's weight rows (one per column block), and the power of two that brings the row's largest scale
    // into [2^10, 2^11): lane half h scans its half of the row's scales
    uint32_t sboff[NB];  // element offset of the row's scales (and biases): a 32-bit lane part next to a uniform base
    float col_up[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int n = min(n0 + (wave_n * NB + nb) * 32 + j, N - 1);
        sboff[nb] = (uint32_t)n * (uint32_t)sb_per_row;
        const uint16_t* srow = a.s + sboff[nb];
        uint32_t mag = 0;
        if ((sb_per_row & 15) == 0 && ((uintptr_t)a.s & 15) == 0) {
            const uint4* p = reinterpret_cast<const uint4*>(srow) + h * (sb_per_row >> 4);
            for (int i = 0; i < (sb_per_row >> 4); i++) {
                const uint4 v = p[i];
                const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const uint32_t lo = w[c] & 0x7fffu, hi = (w[c] >> 16) & 0x7fffu;
                    if (lo < 0x7f80u) mag = max(mag, lo);
                    if (hi < 0x7f80u) mag = max(mag, hi);
                }
            }
        } else {
            for (int i = h; i < sb_per_row; i += 2) {
                const uint32_t v = srow[i] & 0x7fffu;
                if (v < 0x7f80u) mag = max(mag, v);
            }
        }
        mag = max(mag, (uint32_t)__shfl_xor((int)mag, 32, kWave));
        col_up[nb] = pow2f(exponent_shift(mag, 10));
    }

    // Scales are fetched per QUAD of four 64-code blocks, one quad ahead: the bf16 bits of the quad's four blocks
    // in two words per column block (8-byte loads where the rows allow it).  Biases and the (hi, lo) block sums
    // of x are needed once per quad, by the affine MFMA behind its last block, and are fetched for the quad under
    // way.
    const bool quad_loads = a.gs_blocks == 1 && (G & 3) == 0 && (((uintptr_t)a.s | (uintptr_t)a.b) & 7) == 0;
    uint2 s_cur[NB], s_nxt[NB], b_cur[NB];
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
    // bf16 bits of block q (0..3) of a quad, as the high half of a word (= the fp32 value)
    auto quad_hi = [](const uint2& v, int q) {
        const uint32_t w = q < 2 ? v.x : v.y;
        return (q & 1) ? (w & 0xffff0000u) : (w << 16);
    };
    uint32_t xsoff[MB];  // in 16-byte units
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        int row = m0 + (wave_m * MB + mb) * 32 + j;
        row = row < a.mblks * 32 ? row : a.mblks * 32 - 1;
        xsoff[mb] = (uint32_t)row * (uint32_t)G4;
    }
    uint4 xs_cur[MB];
    auto load_xs = [&](int quad) {
#pragma unroll
        for (int mb = 0; mb < MB; mb++) xs_cur[mb] = reinterpret_cast<const uint4*>(a.xs)[xsoff[mb] + quad];
    };

    f32x16_t out[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) out[mb][nb][r] = 0.0f;

    // Affine terms of a quad's blocks 0..Q in one bf16 MFMA per output tile: k-slots (2q, 2q+1) carry
    // (Sx_hi, Sx_lo) of block q on the A side; lanes h=0 pair them with the bias, lanes h=1 with 8 * scale
    // (both times the row's power of two: exact); blocks past Q (only at the end of K) contribute zeros.
    auto affine = [&](auto q_tag) {
        constexpr int Q = decltype(q_tag)::value;
        bf16x8_t bbf[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            uint32_t v[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                if (q <= Q) {
                    const uint32_t eight = __float_as_uint(__uint_as_float(quad_hi(s_cur[nb], q)) * (8.0f * col_up[nb])) >> 16;
                    const uint32_t bia = __float_as_uint(__uint_as_float(quad_hi(b_cur[nb], q)) * col_up[nb]) >> 16;
                    v[q] = dup16(h ? eight : bia);
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
    };

    // One 64-code block per iteration; Q = g & 3 is static so that everything indexed by it stays in fixed
    // registers.  Iteration g requests block g + AHEAD.  Past the end of K the last block is requested again.
    //
    // The next quad's scales and the current quad's biases and sums are fetched at Q = 1 with ordinary loads.
    // The compiler cannot count the copy instructions, so wherever it first uses a loaded register it waits
    // until NOTHING is outstanding, copies included.  Iteration Q = 1 is therefore ordered: loads, MFMAs, first
    // use of the loaded registers (forced), and only then this iteration's copies - the forced wait then covers
    // the loads, a block of MFMAs old, and the copies of block g+1, which the end of the iteration needs anyway.
    // With two or four stages the stage of block g is g & 3 modulo the stages, static like Q, and every LDS address
    // of the loop is a constant; with three it is carried along.
    const int glast = G - 1;
    constexpr bool STATIC_STAGE = STAGES == 2 || STAGES == 4;
    int sa_carried = 0;  // LDS stage that holds block g
    auto iteration = [&](auto q_tag, int g) {
        constexpr int Q = decltype(q_tag)::value;
        constexpr bool LATE = Q == 1;  // copies behind the MFMAs
        const bool more = g + 1 < G;
        const int sa = STATIC_STAGE ? Q % STAGES : sa_carried;
        if constexpr (Q == 0) {
#pragma unroll
            for (int nb = 0; nb < NB; nb++) s_cur[nb] = s_nxt[nb];
        }
        if constexpr (Q == 1) {
            const int nq = (g >> 2) + 1 < G4 ? (g >> 2) + 1 : G4 - 1;
            load_quad(a.s, nq, s_nxt);
            load_quad(a.b, g >> 2, b_cur);
            load_xs(g >> 2);
        }
        // the copies of block g + AHEAD: together at the top, or (SPREAD) a few in front of every row block's
        // MFMAs, so that they do not queue up behind those of the other wavefronts
        const int g2 = g + AHEAD < G ? g + AHEAD : glast;
        const int st2 = sa == 0 ? STAGES - 1 : sa - 1;  // stage (sa + AHEAD) % STAGES: read last in iteration g-1
        if constexpr (!SPREAD && !LATE) {
            issue_a(g2, st2);
            issue_b(g2, st2);
        }
        const uint8_t* ab = abuf + sa * A_STAGE + (wave_m * MB) * 4096 + lane * 16;
        // this lane's codes: row (wave_n * NB + nb) * 32 + j, words 4h .. 4h+3
        const uint8_t* bb = bbuf + sa * B_STAGE + ((wave_n * NB) * 32 + j) * 32 + h * 16;
        f16x8_t bfrag[NB][4];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const uint4 cw = *reinterpret_cast<const uint4*>(bb + nb * 32 * 32);
            // the block's scale, brought into fp16 range (8 significant bits: exact), and -24 times it (10 bits)
            const float sv = __uint_as_float(quad_hi(s_cur[nb], Q)) * col_up[nb];
            const f16x2_t s2 = {(_Float16)sv, (_Float16)sv};
            const float mv = sv * -24.0f;
            const f16x2_t m24 = {(_Float16)mv, (_Float16)mv};
            bfrag[nb][0] = __builtin_bit_cast(f16x8_t, expand_word(cw.x, mask_s, magic_v, s2, m24));
            bfrag[nb][1] = __builtin_bit_cast(f16x8_t, expand_word(cw.y, mask_s, magic_v, s2, m24));
            bfrag[nb][2] = __builtin_bit_cast(f16x8_t, expand_word(cw.z, mask_s, magic_v, s2, m24));
            bfrag[nb][3] = __builtin_bit_cast(f16x8_t, expand_word(cw.w, mask_s, magic_v, s2, m24));
        }
        // the A fragments of row block mb+1 are read while row block mb is multiplied
        f16x8_t afrag[2][4];
#pragma unroll
        for (int t = 0; t < 4; t++) afrag[0][t] = *reinterpret_cast<const f16x8_t*>(ab + t * 1024);
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            if (mb + 1 < MB) {
#pragma unroll
                for (int t = 0; t < 4; t++)
                    afrag[(mb + 1) & 1][t] = *reinterpret_cast<const f16x8_t*>(ab + ((mb + 1) * 4 + t) * 1024);
                __builtin_amdgcn_sched_barrier(0);  // or the scheduler sinks the reads back to their first use
            }
            if constexpr (SPREAD && !LATE) {
#pragma unroll
                for (int c = mb * GROUP_OPS / MB; c < (mb + 1) * GROUP_OPS / MB; c++) issue_one(c, g2, st2);
            }
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    out[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(afrag[mb & 1][t], bfrag[nb][t], out[mb][nb], 0, 0, 0);
        }
        if constexpr (LATE) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
                asm volatile("" : "+v"(s_nxt[nb].x), "+v"(s_nxt[nb].y), "+v"(b_cur[nb].x), "+v"(b_cur[nb].y));
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
                asm volatile("" : "+v"(xs_cur[mb].x), "+v"(xs_cur[mb].y), "+v"(xs_cur[mb].z), "+v"(xs_cur[mb].w));
            __builtin_amdgcn_sched_barrier(0);
            issue_a(g2, st2);
            issue_b(g2, st2);
        }
        if (Q == 3 || !more) {
            if (Q < 1) {  // K ends inside a quad before its biases and sums were asked for
                load_quad(a.b, g >> 2, b_cur);
                load_xs(g >> 2);
            }
            affine(q_tag);
        }
        sa_carried = sa == STAGES - 1 ? 0 : sa + 1;
        // Block g+1 has landed once at most the copies of the AHEAD-1 newest blocks are outstanding; this
        // iteration's LDS reads have returned.  A bare s_barrier on purpose: __syncthreads() carries a workgroup
        // fence, for which the compiler drains ALL outstanding copies into LDS.
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((AHEAD - 1) * GROUP_OPS) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    // the first quad's scales; blocks 0 .. AHEAD-1 were requested before the scan of the scale rows (any wait of
    // the compiler's for the loads since then has drained those copies too: all the better)
    load_quad(a.s, 0, s_nxt);
#pragma unroll
    for (int nb = 0; nb < NB; nb++) asm volatile("" : "+v"(s_nxt[nb].x), "+v"(s_nxt[nb].y));
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((AHEAD - 1) * GROUP_OPS) : "memory");  // block 0 has landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    for (int g = 0; g < G; g += 4) {
        iteration(std::integral_constant<int, 0>{}, g);
        if (g + 1 < G) iteration(std::integral_constant<int, 1>{}, g + 1);
        if (g + 2 < G) iteration(std::integral_constant<int, 2>{}, g + 2);
        if (g + 3 < G) iteration(std::integral_constant<int, 3>{}, g + 3);
    }
    // the copies requested past the end of K must not outlive the wavefront's use of LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // D layout of v_mfma_f32_32x32x*: lane (j, h), register r -> row 8*(r/4) + 4*h + r%4, column j: a lane holds
    // single elements of 16 rows, and storing them as they lie means 2-byte stores to 64-byte pieces of rows
    // (measured: a third of a tile's time).  Each 32-row block of the wavefront's tile therefore goes through a
    // staging area in LDS that belongs to the wavefront (the stages are free: every copy has landed, every read of
    // the loop has returned, and the barrier says so for all wavefronts), scaled by the two inverse powers of two
    // (exact, whatever the order), and leaves it row-major, eight consecutive columns per lane: 16-byte bf16
    // stores, whole 128-byte lines per eight lanes.
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    constexpr int CW = NB * 32;       // columns of the wavefront's tile
    constexpr int LPR = CW / 8;       // lanes that share a row, eight columns each
    constexpr int RPP = kWave / LPR;  // rows per pass
    static_assert(NWAVE * 32 * CW * 4 <= STAGES * (A_STAGE + B_STAGE), "staging area fits the stages");
    float* const stage = reinterpret_cast<float*>(lds) + wave * (32 * CW);
    const bool wide = (reinterpret_cast<uintptr_t>(a.y) & 15) == 0 && (a.out_f32 ? (N & 3) == 0 : (N & 7) == 0);
    const int row_in = lane / LPR, c8 = (lane % LPR) * 8;
    const int n = n0 + wave_n * CW + c8;
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
        const int mtop = m0 + (wave_m * MB + mb) * 32;  // < mblks * 32 unless the whole block lies past M
        float4 down[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const int m = mtop + 4 * h + 8 * q;
            down[q] = m < a.mblks * 32 ? *reinterpret_cast<const float4*>(a.rs + m) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const float col_down = 1.0f / col_up[nb];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float4 d4 = down[r >> 2];
                const float dm = (r & 3) == 0 ? d4.x : (r & 3) == 1 ? d4.y : (r & 3) == 2 ? d4.z : d4.w;
                stage[(8 * (r >> 2) + 4 * h + (r & 3)) * CW + nb * 32 + j] = out[mb][nb][r] * dm * col_down;
            }
        }
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
                if (a.out_f32) {
                    float4* dst = reinterpret_cast<float4*>(reinterpret_cast<float*>(a.y) + o);
                    dst[0] = lo;
                    dst[1] = hi;
                } else {
                    uint4 u;
                    u.x = pack_bf16x2(lo.x, lo.y);
                    u.y = pack_bf16x2(lo.z, lo.w);
                    u.z = pack_bf16x2(hi.x, hi.y);
                    u.w = pack_bf16x2(hi.z, hi.w);
                    *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(a.y) + o) = u;
                }
            } else {
                const float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    if (n + e < N) {
                        if (a.out_f32) {
                            reinterpret_cast<float*>(a.y)[o + e] = v[e];
                        } else {
                            reinterpret_cast<uint16_t*>(a.y)[o + e] = f32_to_bf16_bits(v[e]);
                        }
                    }
                }
            }
        }
    }
}

// ---- variant table ----------------------------------------------------------------------------

typedef void (*QmmHalfKernel)(const QmmTileArgs);
struct QmmHalfEntry {
    QmmVariant v;
    QmmHalfKernel fn;
    int lds_bytes;
};

#define AQ_QMMH(MB, NB, WM, WN, ST, OCC, SPREAD, SUFFIX)                                               \
    {                                                                                                 \
        {"qmmh_b4_mb" #MB "_nb" #NB "_wm" #WM "_wn" #WN SUFFIX, 4, MB, NB, WM, WN},                   \
            qmmh_kernel<MB, NB, WM, WN, ST, OCC, SPREAD>, ST*((WM * MB * 4096) + (WN * NB * 32 * 32)) \
    }

static const QmmHalfEntry kQmmHalfTable[] = {
    AQ_QMMH(4, 2, 2, 2, 2, 2, true, "_s2c"),  // 256 x 128, four wavefronts, two stages (every LDS address a constant)
    AQ_QMMH(4, 2, 2, 4, 3, 2, false, ""),     // 256 x 256, eight wavefronts, three stages (120 KiB): an A tile feeds twice the MFMAs
    AQ_QMMH(3, 2, 2, 4, 3, 2, false, ""),     // 192 x 256: a round of these takes 0.82 of a round of those; for row counts
                                              // that fill their rounds better (1536 rows: 8 bands instead of 6 of 256)
};

int qmmh_variant_count() { return (int)(sizeof(kQmmHalfTable) / sizeof(kQmmHalfTable[0])); }
const QmmVariant* qmmh_variant(int idx) {
    if (idx < 0 || idx >= qmmh_variant_count()) return nullptr;
    return &kQmmHalfTable[idx].v;
}

// workspace: fragments, block sums, then the row factors (the layout qmmt_workspace_bytes sizes)
hipError_t qmmh_launch(int idx, const QmmArgs& q, void* workspace, hipStream_t stream) {
    if (idx < 0 || idx >= qmmh_variant_count()) return hipErrorInvalidValue;
    const QmmHalfEntry& e = kQmmHalfTable[idx];
    const int mblks = (q.M + 31) / 32;
    const size_t g4 = ((size_t)q.K / 64 + 3) / 4;
    uint16_t* xf = static_cast<uint16_t*>(workspace);
    uint16_t* xs = xf + (size_t)mblks * 32 * q.K;
    float* rs = reinterpret_cast<float*>(xs + (size_t)mblks * 32 * g4 * 8);
    hipError_t rc = hipSuccess;
    if (q.x_ready != kXReadyHalf) {
        hipLaunchKernelGGL(qmmh_prep_kernel, dim3((unsigned)(mblks * 32 / kPrepRows)), dim3(kPrepThreads), 0, stream, q.x, xf, xs, rs, q.M, q.K);
        rc = hipGetLastError();
        if (rc != hipSuccess) return rc;
    }

    QmmTileArgs a{};
    a.xf = xf;
    a.xs = xs;
    a.rs = rs;
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
    const int bm = e.v.wm * e.v.mb * 32, bn = e.v.wn * e.v.nb * 32;
    a.tiles_m = (q.M + bm - 1) / bm;
    a.tiles_n = (q.N + bn - 1) / bn;
    a.ksplit = 1;
    a.gsplit = (q.K / 64 + 3) / 4 * 4;
    a.partial = nullptr;
    const int T = a.tiles_m * a.tiles_n;
    const unsigned grid = (unsigned)(((T + 7) / 8) * 8);
    rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e.fn), (size_t)e.lds_bytes);
    if (rc != hipSuccess) return rc;
    hipLaunchKernelGGL(e.fn, dim3(grid), dim3((unsigned)(e.v.wm * e.v.wn * kWave)), (size_t)e.lds_bytes, stream, a);
    return hipGetLastError();
}

}  // namespace aq
