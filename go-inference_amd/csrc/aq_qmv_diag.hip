// affine_qmv / gather_qmv for gfx950, 4-bit codes in groups of 64 (1..8 activation rows) or 32 (1..2): the
// diagonal-MFMA kernels, with their multi-matrix, gate|up pair, gathered and lm_head forms; and a dense form for
// 8-bit codes in groups of 64 (1..4 rows; the reference's q8 decode kernels, affine_projection.hipinc:105-149).
//
// Same contract as the dot2 kernel (aq_qmv.hip): replaces rocm_mlx_q4_projection*
// (go/engine/hip/kernels/quant/affine_projection.hipinc:3-266), semantics of MLX affine_qmv
// (go/engine/metal/qmv.go:354-421).
//
// The dot2 kernel pays, per packed word of a lane, 7 vector instructions to expand the codes and 4 more
// to multiply them, then a cross-lane reduction per row; it is bound by those issue slots.  Here only the
// expansion stays on the vector unit:
//   * v_mfma_f32_16x16x32_bf16 contracts over (lane group, element): lane (n = lane % 16, j = lane / 16)
//     supplies as B eight codes of weight row n, so the sum over the 64 lanes that the dot2 kernel does
//     with DPP adds happens inside the instruction;
//   * the 16 rows of A are (token t, group slot g): row (t, g) carries the activations of token t in the
//     lane groups whose codes belong to 64-group g of the current chunk and zeros elsewhere, so
//     D[(t, g)][n] is the code . activation sum of exactly one quantisation group, for up to four tokens
//     at the cost of one.  D lands as lane (t, n), register g;
//   * per 256-code chunk of 16 rows: two 16-byte loads per lane (64 contiguous bytes per row and
//     instruction), 8 MFMAs, and per lane `acc += scale[g] * D[g]` (four FMAs);
//   * a wavefront works in steps of 1024 codes (four chunks; the last step of a row may hold fewer) and requests
//     everything it will read up front.
//     The scales and biases of a step are ONE 8-byte load each per lane: lane group j takes the four groups of
//     chunk j (16 rows x 32 contiguous bytes per instruction; a load per chunk touched as many cache lines as
//     the weights themselves and cost 2 us on the headline shape).  The lanes that need the scales of chunk c
//     for the FMAs fetch them from lane group c with ds_bpermute (no vector instruction);
//   * the affine term needs no vector work either: the group sums X of the activations are split into
//     three bf16 terms when x is staged (exact: 3 x 8 bits), and three more MFMAs per step accumulate
//     bias * X - 128 * scale * X over its 16 groups from B = (b, b, b, s, s, s) and A = (X0, X1, X2, -128 X0,
//     -128 X1, -128 X2) per group, every product exact (the codes travel as 128 + code, see aq_device.h);
//   * the NW wavefronts of a set take the steps of the same 16 rows in turn and meet in LDS; a workgroup
//     holds NR sets (more rows per workgroup when more activation rows have to be staged).
//   * one activation row: every wavefront stages the activations of its own step (no workgroup barrier before
//     the arithmetic: with many wavefronts per workgroup the barrier made all wait for the one whose loads got out
//     last); more rows: the workgroup stages x together.
// Every variant of one (NW, steps per wavefront) pair computes the same bytes for a row, whatever NR and
// whatever the number of activation rows, and so does the multi-matrix launch.
#include "aq_device.h"
#include "aq_kernels.h"
#include "aq_tile.h"

#include <cstdlib>
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
// The same with the non-temporal hint: the line leaves the L1 once it has been read.  Only for loads that take whole
// 128-byte lines per instruction (a line requested in two halves would be fetched twice).
__device__ __forceinline__ uint4 load_u128_stream_at(gptr_t base, uint32_t off) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x4_t*>(base + off));
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint32_t load_u32_at(gptr_t base, uint32_t off) {
    return *reinterpret_cast<const __attribute__((address_space(1))) uint32_t*>(base + off);
}
__device__ __forceinline__ uint2 load_u64_at(gptr_t base, uint32_t off) {
    const u32x2_t v = *reinterpret_cast<const __attribute__((address_space(1))) u32x2_t*>(base + off);
    return make_uint2(v[0], v[1]);
}

__device__ __forceinline__ bf16x8_t as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const uint4 v = make_uint4(a, b, c, d);
    return __builtin_bit_cast(bf16x8_t, v);
}

}  // namespace

constexpr int kDiagRows = 16;      // weight rows per workgroup
constexpr int kDiagChunk = 256;    // codes of a row per MFMA chain (four groups of 64)
// A wavefront step is CPS chunks (a template parameter: 4, or 3 where that shares K out more evenly, e.g. the 11
// chunks of K = 2816 as 3 + 3 + 3 + 2 over four wavefronts instead of 4 + 4 + 3 + none).
constexpr int kDiagZeroBytes = 128;
#ifndef AQ_DIAG_AHEAD
#define AQ_DIAG_AHEAD 2  // chunks of a step requested before its arithmetic starts; chunk c + 2 when chunk c is about to be multiplied
#endif
#ifndef AQ_DIAG_WROWS
#define AQ_DIAG_WROWS 1  // most activation rows a wavefront stages for itself (4 measured slower for every row count)
#endif

// LDS: activations in expansion order [M][K] bf16, the split group sums [M][chunks of 256 codes] x 48 B, 64 zero bytes,
// the partial sums of the wavefronts [NW][sets of four activation rows][64] fp32.
// (8-bit codes: chunks of 128 codes and 32 bytes of sums each.)
__host__ __device__ inline size_t qmvd_lds_bytes_for(int M, int K, int nw, int mt = 1, bool g32 = false, bool b8 = false) {
    const int chunk = b8 ? kDiagChunk / 2 : kDiagChunk;
    return (size_t)M * K * 2 + (size_t)M * ((K + chunk - 1) / chunk) * (g32 ? 96 : b8 ? 32 : 48) + kDiagZeroBytes +
           (size_t)nw * mt * 64 * 4;
}

// NR sets of NW wavefronts (a set per 16 rows); each wavefront takes SUP steps of 1024 codes (steps wave,
// wave + NW, ...) of its set's rows.
// PAIR (NR = 2): set 0 works on the `gate` matrix (a.w, a.s, a.b), set 1 on the `up` matrix (a.w2, a.s2, a.b2), both
// on the same 16 rows, and the store is act(gate . x) * (up . x).
// MT: sets of four activation rows (the 16 rows of A hold four tokens; a second set reuses the expanded codes with
// eight more MFMAs per chunk).
// GATHER: blockIdx.y is a route; the expert id and the activation row are read from a.rhs / a.lhs on the device
// (kernels/moe/lthn_gather_qmv.metal:54-66 semantics), one activation row per route.
// G32: quantisation groups of 32 codes.  A lane group's 32 codes are then one whole group: the 16 rows of A are
// (token, group slot) for TWO tokens and the eight groups of a chunk, row (t, g) is non-zero in load L for lane
// group j iff g == 4 L + j, D lands as lane (2 t + g / 4, n), register g % 4, and the two halves of a token's sum
// meet at the end.  Scales and biases are 16 bytes per chunk and lane.  K is then a multiple of 256.
// EVEN (the caller has checked): 2 (or `true`) K is a whole number of steps of CPS chunks: no step is short and no chunk a single half;
// 1 K is a whole number of chunks (the last step may be short, no chunk is a single half);
// and what deals with those is not compiled in.
// HEAD (lm_head, one activation row): 4 stores every row's packed (score, row) instead of the score, 3 keeps the
// best packed value of the 16 rows in a.partial[set] for fold_best_kernel (aq_qmv_head.hip).
// B8: 8-bit codes.  The bytes of a row keep the geometry of the 4-bit kernel (64-byte halves, 128-byte chunks, 16 bytes
// per lane and half), so the loads are the same instructions; a half is then ONE group of 64 codes and a chunk two:
// row (t, g) of A is non-zero in half L iff g == L, whatever the lane group, a lane's 16 codes of a half are two MFMAs
// (cvt_f32_ubyte + v_perm give bf16 pairs in the order of the codes, every code 0..255 exact), D registers 0 and 1 of
// the two halves are the two group sums, and the affine term is bias * X alone (the codes travel as themselves).
// K is then a multiple of 128, so no chunk is a single half.
template <int NW, int SUP, int NR, bool PAIR, int MT = 1, bool GATHER = false, int CPS = 4, bool G32 = false, int HEAD = 0,
          bool LINES = true, bool STREAM = false, bool TILED = false, int EVEN = 0, bool B8 = false>
__device__ __forceinline__ void qmv_diag_body(const QmvArgs& a, const int block) {
    static_assert(!B8 || (!G32 && !TILED && !GATHER && !PAIR && HEAD == 0), "8-bit codes: dense group-64 projections");
    static_assert(!STREAM || LINES || TILED, "streaming loads take whole lines");
    static_assert(!TILED || (!G32 && !GATHER && HEAD == 0), "the tile-major layout: dense group-64 projections");
    static_assert(HEAD == 0 || (!PAIR && !GATHER && MT == 1), "the head epilogues take one plain activation row");
    static_assert(!G32 || MT == 1, "group 32: one set of two activation rows");
    constexpr int TPS = G32 ? 2 : 4;      // activation rows per set
    constexpr int A2B = G32 ? 96 : B8 ? 32 : 48;  // bytes of split group sums per chunk and activation row (8 bit: 24 + 8 of zeros)
    constexpr int SBB = G32 ? 16 : B8 ? 4 : 8;    // bytes of scales (or biases) per chunk and weight row
    constexpr int HSH = B8 ? 6 : 7;               // log2 of the codes in a 64-byte half of a row
    constexpr int XH = B8 ? 128 : 256;            // bytes of activations per half
    constexpr int PPC = B8 ? 16 : 32;             // 16-byte pieces of activations per chunk
    constexpr int NI = B8 ? 2 : 4;                // MFMAs per half
    static_assert(!PAIR || NR == 2, "the pair kernel runs one set per matrix");
    static_assert(!GATHER || MT == 1, "a route has one activation row");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave_wg = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = wave_wg % NW;  // which steps of K
    const int rg = wave_wg / NW;    // which 16 rows of the workgroup's NR x 16
    const int K = a.K, N = a.N, M = GATHER ? 1 : a.M;
    const int groups = K >> (G32 ? 5 : 6);
    const int halves = K >> HSH;           // 64-byte halves of a row (K % 128 == 0)
    const int chunks = (halves + 1) >> 1;  // the last chunk may be a single half
    static_assert(CPS >= 2 && CPS <= 4, "a step holds 2..4 chunks (one lane group per chunk for the scales)");
    const int supers = (chunks + CPS - 1) / CPS;  // the last step may hold fewer chunks
    const uint32_t xs_off = 0;
    const uint32_t a2_off = (uint32_t)M * K * 2;
    const uint32_t zero_off = a2_off + (uint32_t)M * chunks * A2B;
    const uint32_t red_off = zero_off + kDiagZeroBytes;

    // gather: the route's expert slab and activation row
    int64_t slab_row = 0, slab_row2 = 0, x_row = 0, y_row = 0;
    bool route_ok = true;
    if constexpr (GATHER) {
        const int z = blockIdx.y;
        const int e = a.rhs[z];
        int xr = a.lhs ? a.lhs[z] : 0;
        route_ok = (unsigned)e < (unsigned)a.num_experts && (unsigned)xr < (unsigned)a.x_rows;
        if (!route_ok) xr = 0;
        slab_row = route_ok ? (int64_t)e * a.expert_rows + a.row_base : 0;
        slab_row2 = route_ok ? (int64_t)e * a.expert_rows + a.row_base2 : 0;
        x_row = xr;
        y_row = z;
    }

    // ---- stage x: expansion order within every 8 values, group sums split into three bf16 terms ----
    const gptr_t xg = uniform_ptr(reinterpret_cast<const char*>(a.x) + x_row * K * 2);
    const int ppt = K >> 3;        // 16-byte pieces of a token (K % 128 == 0: whole groups of eight)
    const int pieces = M * ppt;
    auto stage = [&](int p, uint32_t t, const uint4 v) {  // piece p of x, which belongs to activation row t
        uint4 o = v;  // (8-bit codes expand in their own order)
        if constexpr (!B8) {
            o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (x0, x4)
            o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (x1, x5)
            o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (x2, x6)
            o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (x3, x7)
        }
        *reinterpret_cast<uint4*>(lds_raw + xs_off + (uint32_t)p * 16) = o;
        const uint32_t ones = 0x3f803f80u;
        float sum = dot2_bf16(v.x, ones, 0.0f);
        sum = dot2_bf16(v.y, ones, sum);
        sum = dot2_bf16(v.z, ones, sum);
        sum = dot2_bf16(v.w, ones, sum);
        // the eight pieces of a group sit in eight consecutive, aligned lanes: two quad swaps, then the mirror of the
        // half row adds the other quad (DPP, no LDS round trips)
        sum += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0xB1, 0xF, 0xF, true));
        sum += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0x4E, 0xF, 0xF, true));
        if constexpr (!G32)
            sum += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0x141, 0xF, 0xF, true));
        if ((p & (G32 ? 3 : 7)) == 0) {
            const uint32_t u0 = __float_as_uint(sum) & 0xffff0000u;
            const float r1 = sum - __uint_as_float(u0);
            const uint32_t u1 = __float_as_uint(r1) & 0xffff0000u;
            const float r2 = r1 - __uint_as_float(u1);
            const uint32_t u2 = __float_as_uint(r2) & 0xffff0000u;
            // (8-bit codes carry no offset: the scale slots of the affine term multiply zeros)
            const uint32_t n0 = B8 ? 0u : __float_as_uint(-128.0f * __uint_as_float(u0));
            const uint32_t n1 = B8 ? 0u : __float_as_uint(-128.0f * __uint_as_float(u1));
            const uint32_t n2 = B8 ? 0u : __float_as_uint(-128.0f * __uint_as_float(u2));
            // group g of token t: 12 bytes at [t][chunk g / 4][g % 4]
            const uint32_t g = ((uint32_t)p - t * (uint32_t)ppt) >> (G32 ? 2 : 3);
            uint32_t* e = G32  ? reinterpret_cast<uint32_t*>(lds_raw + a2_off + (t * chunks + (g >> 3)) * 96 + (g & 7) * 12)
                          : B8 ? reinterpret_cast<uint32_t*>(lds_raw + a2_off + (t * chunks + (g >> 1)) * 32 + (g & 1) * 12)
                               : reinterpret_cast<uint32_t*>(lds_raw + a2_off + (t * chunks + (g >> 2)) * 48 + (g & 3) * 12);
            e[0] = (u0 >> 16) | u1;  // (X0, X1)
            e[1] = (u2 >> 16) | n0;  // (X2, -128 X0)
            e[2] = (n1 >> 16) | n2;  // (-128 X1, -128 X2)
            if (B8 && (g & 1)) e[3] = e[4] = 0;  // the last 8 of a chunk's 32 bytes
            if (EVEN == 0 && !G32 && !B8 && (halves & 1) && (int)g == groups - 1) {
                // a last chunk of one half: its two missing groups must add nothing to the affine term
#pragma unroll
                for (int q = 3; q < 9; q++) e[q] = 0;
            }
        }
    };
    // One step per wavefront and up to WROWS activation rows: every wavefront stages the 1024 activations per row of
    // its own step (128 pieces per row, two per lane) and nobody waits for anybody before the arithmetic.  Otherwise
    // the workgroup stages all of x together and meets at a barrier.
    constexpr int WROWS = (SUP == 1 && MT == 1) ? AQ_DIAG_WROWS : 0;
    const bool wstage = M <= WROWS;
    // the first pieces of a thread are requested before the weights, so that they arrive first
    constexpr int PRE = WROWS > 1 ? 2 * WROWS : 2;
    uint4 pre[PRE];
    int pre_p[PRE];
#pragma unroll
    for (int q = 0; q < PRE; q++) {
        if (wstage) {
            const int pl = wave * (CPS * PPC) + (q & 1) * 64 + lane;  // piece of row q / 2
            pre_p[q] = (q >> 1) < M && pl < ppt && (q & 1) * 64 + lane < CPS * PPC ? (q >> 1) * ppt + pl : pieces;
        } else {
            pre_p[q] = q < 2 ? tid + q * NR * NW * kWave : pieces;
        }
        if (q < 2 || (wstage && (q >> 1) < M)) pre[q] = load_u128_at(xg, (uint32_t)min(pre_p[q], pieces - 1) * 16);
    }
    if (lane < kDiagZeroBytes / 16 && (wstage || wave_wg == 0))
        *reinterpret_cast<uint4*>(lds_raw + zero_off + lane * 16) = make_uint4(0, 0, 0, 0);

    // ---- per-lane constants ----
    const int n = lane & 15;   // weight row of the lane (B operand, D column)
    const int j = lane >> 4;   // lane group: which 16 bytes of a 64-byte row piece (B), token (D)
    const int at = G32 ? (lane & 15) >> 3 : (lane & 15) >> 2;  // A operand: token of the lane's A row
    const int ag = G32 ? lane & 7 : lane & 3;                  // A operand: group slot of the lane's A row
    const int row0 = (PAIR ? block : block * NR + rg) * kDiagRows;
    int row = row0 + n;
    if (row >= N) row = N - 1;
    const bool second = PAIR && rg == 1;
    const bool other = second && !GATHER;  // gathered pairs: two row bases inside one expert slab
    const int64_t srow = second ? slab_row2 : slab_row;
    const gptr_t wg = uniform_ptr(reinterpret_cast<const char*>(other ? a.w2 : a.w) + srow * (K >> 1));
    const gptr_t sg = uniform_ptr(reinterpret_cast<const char*>(other ? a.s2 : a.s) + srow * groups * 2);
    const gptr_t bg = uniform_ptr(reinterpret_cast<const char*>(other ? a.b2 : a.b) + srow * groups * 2);
    // LINES: weights are requested as whole 128-byte lines of 8 rows per instruction (half as many requests at the L1 as
    // 64 bytes of each of 16 rows): lane (i = lane % 16, j) of load `ab` reads row 8 ab + i % 8 of the set, bytes
    // 64 (i / 8) + 16 j of a chunk; two DPP moves per register pair then leave "lane (n, j): bytes 16 j .. 16 j + 15 of
    // the first (second) 64 bytes of row n", the shape the B operands have.  Otherwise load L of a chunk is that shape
    // as it comes.  (Measured on one box, old shape -> lines: the four-launch layer 33.0 -> 32.3 us, 14336 -> 4096
    // 9.0 -> 8.8 us, the MoE block 84.2 -> 82.4 us, but 4096 -> 14336 as a launch of its own 8.5 -> 8.6 us: the plain
    // kernel of up to four wavefronts keeps the old shape.)
    uint32_t w_lane[2];
#pragma unroll
    for (int ab = 0; ab < 2; ab++) {
        int r8 = LINES ? row0 + (n & 7) + 8 * ab : row0 + n;
        if (r8 >= N) r8 = N - 1;
        w_lane[ab] = (uint32_t)r8 * (uint32_t)(B8 ? K : K >> 1) + (uint32_t)j * 16;  // bytes
    }
    const uint32_t w_half = LINES ? (uint32_t)(n >> 3) * 64 : 0;  // which 64 bytes of the chunk this lane requests
    // TILED (aq_tile.h): a step of a set of 16 rows is one contiguous tile, 1 KiB of scales and biases and then 1 KiB
    // per 128-code half, each KiB in lane order, so every load instruction of a wavefront takes 1 KiB of consecutive
    // bytes and the registers arrive in operand order
    // (a workgroup of several sets may reach past the last set of the tensor: it reads the last one again and stores nothing)
    const uint32_t t_lane = TILED ? (uint32_t)min(row0 / kDiagRows, (N + kDiagRows - 1) / kDiagRows - 1) * tile_set_bytes(K, CPS) + (uint32_t)lane * 16 : 0;
    // scales and biases: lane group j holds the four groups of chunk j of the step
    const uint32_t sb_lane = (uint32_t)row * (uint32_t)groups * 2 + (uint32_t)j * SBB;  // bytes

    // the lane that holds the scales of chunk 0 of the step for this lane's row (ds_bpermute byte address)
    const int sc_addr = n * 4;

    const uint32_t mask = opaque_s(kNibbleMask);
    const uint32_t magic = opaque_v(kMagic128);

    uint4 wq[SUP][CPS][2];
    uint4 sq[SUP], bq[SUP];  // (group 64: x and y only)
    // Scales and biases are requested before the codes: loads come back in the order they went out, and every chunk's
    // arithmetic needs them, so the first chunk can be worked on while the later ones are still on the way.
    auto step_of = [&](int u) {
        const int sp = wave + u * NW;
        return sp >= supers ? supers - 1 : sp;  // past the end: a valid address, the result is not used
    };
    auto issue_scales = [&](int u) {
        const int sp = step_of(u);
        const int valid = EVEN == 2 ? CPS : min(CPS, chunks - CPS * sp);  // chunks of this step
        if constexpr (TILED) {
            const uint32_t to = t_lane + (uint32_t)sp * tile_step_bytes(CPS);
            const uint4 sb = STREAM ? load_u128_stream_at(wg, to) : load_u128_at(wg, to);
            sq[u] = make_uint4(sb.x, sb.y, 0, 0);
            bq[u] = make_uint4(sb.z, sb.w, 0, 0);
        } else {
            // A last chunk of one half has two groups: its 8 bytes are read 4 bytes early (inside the row) and the
            // upper word, which holds the two groups, moves down.
            const bool halfl = EVEN == 0 && !B8 && (halves & 1) && j < CPS && CPS * sp + j == chunks - 1;
            const uint32_t so = sb_lane + (uint32_t)sp * (CPS * SBB) - (j < valid ? 0u : (uint32_t)j * SBB) - (halfl ? 4u : 0u);
            if constexpr (G32) {
                sq[u] = load_u128_at(sg, so);
                bq[u] = load_u128_at(bg, so);
            } else if constexpr (B8) {
                sq[u] = make_uint4(load_u32_at(sg, so), 0, 0, 0);
                bq[u] = make_uint4(load_u32_at(bg, so), 0, 0, 0);
            } else {
                const uint2 s2 = load_u64_at(sg, so), b2 = load_u64_at(bg, so);
                sq[u] = make_uint4(s2.x, s2.y, 0, 0);
                bq[u] = make_uint4(b2.x, b2.y, 0, 0);
            }
            if (EVEN == 0 && !G32 && !B8 && (halves & 1)) {
                sq[u].x = halfl ? sq[u].y : sq[u].x;
                bq[u].x = halfl ? bq[u].y : bq[u].x;
            }
        }
    };
    auto issue_chunk = [&](int u, int cc) {
        const int sp = step_of(u);
        const int valid = EVEN == 2 ? CPS : min(CPS, chunks - CPS * sp);  // chunks of this step; the others re-read chunk 0 and are not used
        if constexpr (TILED) {
            const uint32_t to = t_lane + (uint32_t)sp * tile_step_bytes(CPS);
#pragma unroll
            for (int L = 0; L < 2; L++) {
                // (a half past the end of the row: re-reads the tile's first, not used)
                const uint32_t ho = EVEN == 2 || (cc < valid && (EVEN == 1 || 2 * (CPS * sp + cc) + L < halves)) ? (uint32_t)(2 * cc + L) * 1024 : 0;
                wq[u][cc][L] = STREAM ? load_u128_stream_at(wg, to + 1024 + ho) : load_u128_at(wg, to + 1024 + ho);
            }
        } else {
            const uint32_t wo = (uint32_t)sp * (CPS * 128);
            const uint32_t co = cc < valid ? cc * 128 : 0;
            // (the second half of a last chunk that is a single half: re-reads the first, not used)
            const bool whole = EVEN == 2 || (cc < valid && (EVEN == 1 || 2 * (CPS * sp + cc) + 1 < halves));
            const uint32_t ho = whole ? w_half : 0;
            if constexpr (STREAM) {
                wq[u][cc][0] = load_u128_stream_at(wg, w_lane[0] + wo + co + ho);
                wq[u][cc][1] = load_u128_stream_at(wg, w_lane[1] + wo + co + ho);
            } else {
                wq[u][cc][0] = load_u128_at(wg, w_lane[0] + wo + co + ho);
                wq[u][cc][1] = load_u128_at(wg, w_lane[1] + wo + co + (LINES ? ho : whole ? 64u : 0u));
            }
        }
    };
    auto stage_x = [&]() {
#pragma unroll
        for (int q = 0; q < PRE; q++)
            if (pre_p[q] < pieces) stage(pre_p[q], wstage ? (uint32_t)(q >> 1) : (uint32_t)pre_p[q] / (uint32_t)ppt, pre[q]);
        if (wstage) {
            // LDS operations of one wavefront complete in order: what its lanes wrote is there for its later reads
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        } else {
            for (int p = tid + 2 * NR * NW * kWave; p < pieces; p += NR * NW * kWave)
                stage(p, (uint32_t)p / (uint32_t)ppt, load_u128_at(xg, (uint32_t)p * 16));
            __syncthreads();  // x, sums and zeros are in LDS
        }
    };
    // A CU takes the loads of its workgroups roughly in the order the workgroups arrived: the first workgroup of a CU
    // gets its requests out at once, the later ones wait for up to microseconds before theirs are accepted.  Those
    // stage x BEFORE they request their weights (they would wait anyway), so that nothing but the arithmetic on the
    // weights is left to do once their loads, the last of the launch, have come back; the first a.early_wgs
    // workgroups request first and stage while the memory system is starting up.
    // (Several activation rows are staged by the workgroup together, behind a barrier: always first; measured at eight
    // rows of 4096 x 14336: 13.4 -> 11.1 us.)
    // (a.early_wgs is read with the first kernel arguments, whether or not it is used: a scalar load behind a branch
    // would be a second wait in front of the first request.  Only the gathered grids have a second dimension.)
    const int early_wgs = a.early_wgs;
    const int linear_block = GATHER ? (int)(blockIdx.x + blockIdx.y * gridDim.x) : (int)blockIdx.x;
    const bool late = linear_block >= early_wgs || !wstage;
    if (late) stage_x();
    // AHEAD chunks are requested before the arithmetic starts; chunk cc + AHEAD when chunk cc is about to be worked on
    // (The group-32 and lm_head kernels request the whole step at once: their launches are grids of many rounds of
    // workgroups, in which a wavefront's requests do not queue behind a whole launch's; 262144 x 1536, group 32:
    // 40.0-42.6 us against 43.2-46.5 us with the ring.)
    constexpr int AHEAD = SUP == 1 && AQ_DIAG_AHEAD < CPS && !G32 && HEAD == 0 ? AQ_DIAG_AHEAD : CPS;
#pragma unroll
    for (int u = 0; u < SUP; u++) {
        issue_scales(u);
#pragma unroll
        for (int cc = 0; cc < AHEAD; cc++) issue_chunk(u, cc);
    }
    // (nothing below is needed to request the weights: it must not delay the requests of the workgroups that start first)
    __builtin_amdgcn_sched_barrier(0);
    // A fragments: load L (0, 1) of a chunk holds groups 2L and 2L + 1; lane group j holds codes of group
    // 2L + (j >> 1).  The lane's A row (at, ag) is non-zero in load L iff ag == 2L + (j >> 1).
    // affine-term A: rows (t, 0) carry the split sums of the four groups of chunk j of the step, 48 bytes
    uint32_t a_base0[MT], a_base1[MT], a_mul0[MT], a_mul1[MT], a_chunk0[MT], a_chunk1[MT], a2_base[MT], a2_mul[MT];
#pragma unroll
    for (int tg = 0; tg < MT; tg++) {
        const int token = tg * TPS + at;
        const bool tok = token < M;
        const bool d0 = tok && ag == (G32 ? j : B8 ? 0 : j >> 1);
        const bool d1 = tok && ag == (G32 ? 4 + j : B8 ? 1 : 2 + (j >> 1));
        const uint32_t x_lane = xs_off + (uint32_t)token * K * 2 + (uint32_t)j * (XH / 4);  // the lane group's quarter of a half
        a_base0[tg] = d0 ? x_lane : zero_off;
        a_base1[tg] = d1 ? x_lane + XH : zero_off;
        a_mul0[tg] = d0 ? CPS * 2 * XH : 0;
        a_mul1[tg] = d1 ? CPS * 2 * XH : 0;
        a_chunk0[tg] = d0 ? 2 * XH : 0;
        a_chunk1[tg] = d1 ? 2 * XH : 0;
        const bool d2 = tok && ag == 0;
        a2_base[tg] = d2 ? a2_off + ((uint32_t)token * chunks + j) * A2B : zero_off;
        a2_mul[tg] = d2 ? CPS * A2B : 0;
    }
    if (!late) stage_x();

    float acc[MT];
    f32x4_t dsum[MT];  // affine term, register 0 is the one that is used
#pragma unroll
    for (int tg = 0; tg < MT; tg++) {
        acc[tg] = 0.0f;
        dsum[tg] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    }
#pragma unroll
    for (int u = 0; u < SUP; u++) {
        const int sp = wave + u * NW;
        if (sp < supers) {
            const int valid = EVEN == 2 ? CPS : min(CPS, chunks - CPS * sp);
            const uint4 sv = sq[u], bv = bq[u];
            // affine term of the groups of the step: six k-slots per group (b b b s s s), 24 (group 32: 48) per lane
            {
                const uint32_t lo2 = 0x01000100u, hi2 = 0x03020302u, lolo = 0x05040100u, hihi = 0x07060302u;
                constexpr int NWORD = G32 ? 4 : B8 ? 1 : 2;  // words of two groups each
                const uint32_t sw[4] = {sv.x, sv.y, sv.z, sv.w}, bw[4] = {bv.x, bv.y, bv.z, bv.w};
                uint32_t e[B8 ? 8 : 6 * NWORD];
                if constexpr (B8) e[6] = e[7] = 0;
#pragma unroll
                for (int w = 0; w < NWORD; w++) {
                    // (b0 b0 | b0 s0 | s0 s0 | b1 b1 | b1 s1 | s1 s1) of the word's two groups
                    e[6 * w + 0] = __builtin_amdgcn_perm(bw[w], bw[w], lo2);
                    e[6 * w + 1] = __builtin_amdgcn_perm(sw[w], bw[w], lolo);
                    e[6 * w + 2] = __builtin_amdgcn_perm(sw[w], sw[w], lo2);
                    e[6 * w + 3] = __builtin_amdgcn_perm(bw[w], bw[w], hi2);
                    e[6 * w + 4] = __builtin_amdgcn_perm(sw[w], bw[w], hihi);
                    e[6 * w + 5] = __builtin_amdgcn_perm(sw[w], sw[w], hi2);
                }
#pragma unroll
                for (int tg = 0; tg < MT; tg++) {
                    // (lane groups past the last chunk of the row contribute zeros)
                    const uint32_t a2_addr = j < valid ? a2_base[tg] + (uint32_t)sp * a2_mul[tg] : zero_off;
#pragma unroll
                    for (int q = 0; q < (B8 ? 2 : 6 * NWORD / 4); q++) {
                        const bf16x8_t a2 = *reinterpret_cast<const bf16x8_t*>(lds_raw + a2_addr + q * 16);
                        dsum[tg] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            a2, as_bf16x8(e[4 * q], e[4 * q + 1], e[4 * q + 2], e[4 * q + 3]), dsum[tg], 0, 0, 0);
                    }
                }
            }
            uint32_t a_addr0[MT], a_addr1[MT];
#pragma unroll
            for (int tg = 0; tg < MT; tg++) {
                a_addr0[tg] = a_base0[tg] + (uint32_t)sp * a_mul0[tg];
                a_addr1[tg] = a_base1[tg] + (uint32_t)sp * a_mul1[tg];
            }
            // The A fragments of chunk cc + 1 are read from LDS while chunk cc is multiplied: every register of `af` is
            // loaded again as soon as the MFMA that read it has been issued, so the wavefront never waits for LDS.
            bf16x8_t af[MT][2][NI];
            // (A last chunk of one half: the A rows of its missing second half are read from the zero block, so that the
            // MFMAs of that half add exact zeros and every chunk runs the same code.)
            auto read_af = [&](int tg, int L, int i, int cc) {
                const bool there = EVEN != 0 || L == 0 || 2 * (CPS * sp + cc) + 1 < halves;
                const uint32_t at1 = there ? a_addr1[tg] + cc * a_chunk1[tg] : zero_off;
                af[tg][L][i] = *reinterpret_cast<const bf16x8_t*>(lds_raw + (L == 0 ? a_addr0[tg] + cc * a_chunk0[tg] : at1) + i * 16);
            };
            // (Two sets of activation rows: the registers do not allow it; a chunk's fragments are read when it starts.)
            constexpr bool PF = MT == 1 && SUP == 1;
            auto read_chunk_af = [&](int cc) {
#pragma unroll
                for (int tg = 0; tg < MT; tg++)
#pragma unroll
                    for (int i = 0; i < NI; i++) {
                        read_af(tg, 0, i, cc);
                        read_af(tg, 1, i, cc);
                    }
            };
            if constexpr (PF) read_chunk_af(0);
#pragma unroll
            for (int cc = 0; cc < CPS; cc++) {
                if (cc + AHEAD < CPS) {
                    issue_chunk(u, cc + AHEAD);
                    __builtin_amdgcn_sched_barrier(0);  // (the request goes out before chunk cc is waited for, not behind its arithmetic)
                }
                if (cc >= valid) break;
                if constexpr (!PF) read_chunk_af(cc);
                const int cnext = min(cc + 1, valid - 1);  // (the last chunk reads its own fragments again: not used)
                // the four scales of chunk cc of this lane's row sit in lane group cc
                uint32_t sx = (uint32_t)__builtin_amdgcn_ds_bpermute(sc_addr + cc * 64, (int)sv.x);
                uint32_t sy = (uint32_t)__builtin_amdgcn_ds_bpermute(sc_addr + cc * 64, (int)sv.y);
                if constexpr (G32) {
                    // this lane's D registers are groups 4 (j & 1) .. + 3 of the chunk's eight
                    const uint32_t sz = (uint32_t)__builtin_amdgcn_ds_bpermute(sc_addr + cc * 64, (int)sv.z);
                    const uint32_t sw2 = (uint32_t)__builtin_amdgcn_ds_bpermute(sc_addr + cc * 64, (int)sv.w);
                    sx = (j & 1) ? sz : sx;
                    sy = (j & 1) ? sw2 : sy;
                }
                // Two chains of MFMAs, one per 128-code half, that take turns: the rows of A that are not zero in
                // half L are those of groups 2 L and 2 L + 1 (group 32: 4 L .. 4 L + 3), so chain L is the whole of
                // those groups' sums and adds exact zeros to the others; the sums are the bits one chain over both
                // halves would give, at half the dependent length.
                f32x4_t dq[MT][2];
#pragma unroll
                for (int tg = 0; tg < MT; tg++) dq[tg][0] = dq[tg][1] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                const uint4 la = wq[u][cc][0], lb = wq[u][cc][1];
                auto multiply = [&](auto both_halves) {  // straight-line code in either case
                    constexpr int NL = decltype(both_halves)::value ? 2 : 1;
#pragma unroll
                    for (int i = 0; i < NI; i++) {
#pragma unroll
                        for (int L = 0; L < NL; L++) {
                            // LINES, first 64 bytes: lanes i >= 8 take rows 8..15 from the second load's lanes i - 8;
                            // second 64 bytes: lanes i < 8 take rows 0..7 from the first load's lanes i + 8
                            auto word = [&](int q) {
                                const uint32_t wa = q == 0 ? la.x : q == 1 ? la.y : q == 2 ? la.z : la.w;
                                const uint32_t wb = q == 0 ? lb.x : q == 1 ? lb.y : q == 2 ? lb.z : lb.w;
                                if constexpr (!LINES || TILED)
                                    return L == 0 ? wa : wb;
                                else if (L == 0)
                                    return (uint32_t)__builtin_amdgcn_update_dpp(wa, wb, 0x118, 0xf, 0xc, false);
                                else
                                    return (uint32_t)__builtin_amdgcn_update_dpp(wb, wa, 0x108, 0xf, 0x3, false);
                            };
                            uint32_t p[4];
                            if constexpr (B8) {
                                unpack8_word(word(2 * i), p);
                                unpack8_word(word(2 * i + 1), p + 2);
                            } else {
                                unpack4_word(word(i), mask, magic, p);
                            }
                            const bf16x8_t bfrag = as_bf16x8(p[0], p[1], p[2], p[3]);
#pragma unroll
                            for (int tg = 0; tg < MT; tg++) {
                                dq[tg][L] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[tg][L][i], bfrag, dq[tg][L], 0, 0, 0);
                                if (PF && cc + 1 < CPS) read_af(tg, L, i, cnext);
                            }
                        }
                    }
                };
                multiply(std::true_type{});
                const float s0 = bf16_bits_to_f32(sx & 0xffffu), s1 = __uint_as_float(sx & 0xffff0000u);
                const float s2 = bf16_bits_to_f32(sy & 0xffffu), s3 = __uint_as_float(sy & 0xffff0000u);
#pragma unroll
                for (int tg = 0; tg < MT; tg++) {
                    // group 64: registers 0, 1 come from the first half, 2, 3 from the second; group 32: all four from
                    // the half of this lane's token slot
                    const f32x4_t d0 = dq[tg][0], d1 = dq[tg][1];
                    const bool odd = G32 && (j & 1);
                    if constexpr (B8) {
                        // two groups a chunk: register 0 of the first half's sums, register 1 of the second's
                        acc[tg] = __builtin_fmaf(s0, d0[0], acc[tg]);
                        acc[tg] = __builtin_fmaf(s1, d1[1], acc[tg]);
                    } else {
                        acc[tg] = __builtin_fmaf(s0, odd ? d1[0] : d0[0], acc[tg]);
                        acc[tg] = __builtin_fmaf(s1, odd ? d1[1] : d0[1], acc[tg]);
                        acc[tg] = __builtin_fmaf(s2, (G32 && !odd) ? d0[2] : d1[2], acc[tg]);
                        acc[tg] = __builtin_fmaf(s3, (G32 && !odd) ? d0[3] : d1[3], acc[tg]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int tg = 0; tg < MT; tg++) acc[tg] += dsum[tg][0];

    // ---- the wavefronts' partial sums meet in LDS; lane (t, n) of the first wavefront of a set stores ----
    float* red = reinterpret_cast<float*>(lds_raw + red_off);
#pragma unroll
    for (int tg = 0; tg < MT; tg++) red[(wave_wg * MT + tg) * 64 + lane] = acc[tg];
    __syncthreads();
    if (wave == 0 && !second) {
#pragma unroll
        for (int tg = 0; tg < MT; tg++) {
            float total = red[(wave_wg * MT + tg) * 64 + lane];
#pragma unroll
            for (int w2 = 1; w2 < NW; w2++) total += red[((wave_wg + w2) * MT + tg) * 64 + lane];
            if constexpr (PAIR) {
                float up = red[(NW * MT + tg) * 64 + lane];
#pragma unroll
                for (int w2 = 1; w2 < NW; w2++) up += red[((NW + w2) * MT + tg) * 64 + lane];
                static_assert(!G32, "the pair kernels are built for group 64");
                total = fmul_unfused(act_value(a.act, total), up);
            }
            if constexpr (GATHER) {
                if (!route_ok) total = 0.0f;
            }
            if constexpr (G32) total += __shfl_xor(total, 16);  // the two halves of a token's groups
            const int t = G32 ? (j >> 1) : tg * 4 + j, r = row0 + n;
            if constexpr (HEAD != 0) {
                // lanes 0..15 hold the scores of rows row0 .. row0 + 15 for the one activation row
                unsigned long long packed = 0;
                if (lane < 16 && r < N && isfinite(total) && !token_suppressed((uint32_t)r, a.suppress, a.suppress_count))
                    packed = pack_score_index(total, (uint32_t)r);
                if constexpr (HEAD == 4) {
                    if (lane < 16 && r < N) reinterpret_cast<unsigned long long*>(a.y)[r] = packed;
                } else {
                    // maximum over the 16 lanes, 32 bits at a time (the halves travel together)
                    uint32_t hi = (uint32_t)(packed >> 32), lo = (uint32_t)packed;
#pragma unroll
                    for (int d = 8; d >= 1; d >>= 1) {
                        const uint32_t ohi = (uint32_t)__shfl_xor((int)hi, d), olo = (uint32_t)__shfl_xor((int)lo, d);
                        const bool take = ohi > hi || (ohi == hi && olo > lo);
                        hi = take ? ohi : hi;
                        lo = take ? olo : lo;
                    }
                    if (lane == 0) a.partial[(size_t)block * NR + rg] = ((unsigned long long)hi << 32) | lo;
                }
                continue;
            }
            if (t < M && r < N && (!G32 || (j & 1) == 0)) {
                const size_t o = (size_t)(GATHER ? y_row : t) * N + r;
                if (a.out_f32) {
                    static_cast<float*>(a.y)[o] = total;
                } else {
                    static_cast<uint16_t*>(a.y)[o] = f32_to_bf16_bits(total);
                }
            }
        }
    }
}

// MODE of the dense kernels, chosen per launch on the host (one kernel per mode, so that a launch carries only the code
// it runs): bit 0 = the weights are loaded with the non-temporal hint, as whole lines (large matrices; same box:
// 4096 x 14336 8.70 -> 8.31 us, the four-launch layer 32.3 -> 30.9 us, but 4096 x 4096 4.05 -> 4.17 us; a read of the
// same bytes with no arithmetic: 6.73 -> 6.17 us in contiguous pieces, but 7.47 -> 8.35 us in 64-byte pieces of rows,
// whose lines are then fetched twice); bit 1 = a.w (and a.w2) hold the tile-major layout of aq_tile.h and a.s, a.b
// are not read; bit 2 = K is a whole number of steps (no code for short steps and half chunks).  The arithmetic and
// its bytes are the same in every mode.
template <int NW, int SUP, int NR, bool PAIR, int MT, int CPS, bool G32, int MODE>
__device__ __forceinline__ void qmv_diag_dense(const QmvArgs& a, const int block) {
    constexpr bool STREAM = (MODE & 1) != 0, TILED = (MODE & 2) != 0;
    constexpr int EVEN = (MODE & 4) != 0 ? 2 : 0;
    constexpr bool LINES = !TILED;
    qmv_diag_body<NW, SUP, NR, PAIR, MT, false, CPS, G32, 0, LINES, STREAM, TILED, EVEN>(a, block);
}

template <int NW, int SUP, int NR, int MT, int CPS, int MODE>
__global__ __launch_bounds__(NR* NW* kWave, 4) void qmv_diag_kernel(const QmvArgs a) {
    if constexpr ((MODE & 3) == 0)  // (the plain kernel of up to four wavefronts keeps 64-byte pieces of 16 rows, see the body)
        qmv_diag_body<NW, SUP, NR, false, MT, false, CPS, false, 0, (NW > 4), false, false, ((MODE & 4) != 0 ? 2 : 0)>(a, (int)blockIdx.x);
    else
        qmv_diag_dense<NW, SUP, NR, false, MT, CPS, false, MODE>(a, (int)blockIdx.x);
}

template <int NW, int SUP, int CPS, int MODE>
__global__ __launch_bounds__(2 * NW* kWave, 4) void qmv_diag_pair_kernel(const QmvArgs a) {
    qmv_diag_dense<NW, SUP, 2, true, 1, CPS, false, MODE>(a, (int)blockIdx.x);
}

// Quantisation groups of 32 codes, up to two activation rows.
template <int NW, int SUP, int NR, int CPS, int MODE>
__global__ __launch_bounds__(NR* NW* kWave, 4) void qmv_diag_g32_kernel(const QmvArgs a) {
    static_assert((MODE & 2) == 0, "groups of 32 have no tile-major form");
    qmv_diag_dense<NW, SUP, NR, false, 1, CPS, true, MODE>(a, (int)blockIdx.x);
}

// 8-bit codes in groups of 64, up to four activation rows (whole lines of 8 rows per load instruction, as the 4-bit
// kernels of more than four wavefronts have them).
template <int NW, int SUP, int NR, int CPS, int MODE>
__global__ __launch_bounds__(NR* NW* kWave, 4) void qmv_diag_b8_kernel(const QmvArgs a) {
    static_assert((MODE & 2) == 0, "8-bit codes have no tile-major form");
    qmv_diag_body<NW, SUP, NR, false, 1, false, CPS, false, 0, true, (MODE & 1) != 0, false, ((MODE & 4) != 0 ? 2 : 1), true>(a, (int)blockIdx.x);
}

// lm_head forms (one activation row): packed scores (4) or the best packed value per 16 rows (3).
// EVEN: K a whole number of steps (the launch checks): without the code for short steps and half chunks the group-32
// form needs 61-75 registers instead of 100-108, i.e. eight wavefronts per SIMD instead of four.
template <int NW, int SUP, int NR, int CPS, bool G32, int HEAD, bool EVEN>
__global__ __launch_bounds__(NR* NW* kWave, 4) void qmv_diag_head_kernel(const QmvArgs a) {
    // always with the non-temporal hint: an lm_head is hundreds of megabytes (262144 x 1536, group 32: 42.0 -> 37.4-38.6 us)
    qmv_diag_body<NW, SUP, NR, false, 1, false, CPS, G32, HEAD, true, true, false, EVEN ? 2 : 0>(a, (int)blockIdx.x);
}

// Gathered forms: grid.y = routes.
// WHOLE: K is a whole number of chunks of 256 codes (the launch checks): the code for a last chunk of one half is left out.
template <int NW, int SUP, int NR, int CPS, bool WHOLE = false>
__global__ __launch_bounds__(NR* NW* kWave, 4) void qmv_diag_gather_kernel(const QmvArgs a) {
    qmv_diag_body<NW, SUP, NR, false, 1, true, CPS, false, 0, true, false, false, (WHOLE ? 1 : 0)>(a, (int)blockIdx.x);
}
template <int NW, int SUP, int CPS, bool WHOLE = false>
__global__ __launch_bounds__(2 * NW* kWave, 4) void qmv_diag_gather_pair_kernel(const QmvArgs a) {
    qmv_diag_body<NW, SUP, 2, true, 1, true, CPS, false, 0, true, false, false, (WHOLE ? 1 : 0)>(a, (int)blockIdx.x);
}

// Several weight matrices against the same activations in one launch (q|k|v, gate|up): the workgroups of all
// matrices form one grid, and each looks up which matrix it belongs to.
template <int NW, int SUP, int NR, int CPS, int MODE>
__global__ __launch_bounds__(NR* NW* kWave, 4) void qmv_diag_multi_kernel(const QmvMultiArgs ma) {
    int set = 0;
#pragma unroll
    for (int i = 1; i < kQmvMultiMax; i++)
        if (i < ma.count && (int)blockIdx.x >= ma.block_end[i - 1]) set = i;
    QmvArgs a = ma.common;
    a.w = ma.w[set];
    a.s = ma.s[set];
    a.b = ma.b[set];
    a.y = ma.y[set];
    a.N = ma.N[set];
    const int block = (int)blockIdx.x - (set ? ma.block_end[set - 1] : 0);
    qmv_diag_dense<NW, SUP, NR, false, 1, CPS, false, MODE>(a, block);
}

// ---- variant table --------------------------------------------------------

// Packed bytes of a dense launch (all its matrices) from which the weights are loaded with the non-temporal hint; the
// gathered kernels keep plain loads (the MoE block measured 80.7 against 83.1 us with the hint: routes share experts).
constexpr int64_t kDiagStreamBytes = (int64_t)16 << 20;

// Workgroups that request their weights before staging x: as many as the device has CUs (the first workgroup each CU
// receives; later ones find the CU's memory queue busy).
static int diag_cu_count() {
    static int cached = -1;
    if (cached < 0) {
        const char* e = getenv("AQ_DIAG_EARLY");
        int dev = 0, cus = 0;
        if (e)
            cached = atoi(e);
        else if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && cus > 0)
            cached = cus;
        else
            cached = 256;
    }
    return cached;
}
// For a grid of `blocks` workgroups.  The rule is for launches whose workgroups are all resident at once (up to four
// per CU): there the later arrivals wait for the CU's memory queue anyway.  In a larger grid (an lm_head, the MoE
// gathers) a workgroup starts when another has finished and should request its weights at once: with every workgroup
// but the first staging x first, the 262144 x 1536 head measured 44.6-45.7 us against 38.8 us.
static int diag_early_wgs(int64_t blocks) {
    const int cus = diag_cu_count();
    return blocks <= (int64_t)4 * cus ? cus : INT32_MAX;
}

typedef void (*QmvDiagKernel)(const QmvArgs);
// Index into a variant's kernels for this launch.
// (K: in codes of 4 bits; a row of 8-bit codes counts as one of twice the length, which has the same bytes)
static int diag_mode(int K, int cps, bool tiled, bool stream) {
    return (K % (cps * kDiagChunk) == 0 ? 4 : 0) + (tiled ? 2 : 0) + (stream ? 1 : 0);
}
struct QmvDiagEntry {
    QmvVariant v;
    QmvDiagKernel fn[8];  // by mode (bit 0: non-temporal weight loads, bit 1: tile-major weights, bit 2: whole steps); gathered: [0], and [1] where K is whole chunks
};
#define AQ_DIAG_MODES(K, ...) {K<__VA_ARGS__, 0>, K<__VA_ARGS__, 1>, K<__VA_ARGS__, 2>, K<__VA_ARGS__, 3>, K<__VA_ARGS__, 4>, K<__VA_ARGS__, 5>, K<__VA_ARGS__, 6>, K<__VA_ARGS__, 7>}
// name, bits, m (most rows), sets of 16 rows per workgroup, wavefronts per set, steps per wavefront, gather,
// xmode = chunks per step when not 4, kind.  waves x depth steps cover K.
#define AQ_QMVD(NW, SUP, NR)                                                                                    \
    {                                                                                                           \
        {"qmvd_b4_m4_r" #NR "_w" #NW "_d" #SUP "_g0", 4, 4, NR, NW, SUP, 0, 0, 4}, AQ_DIAG_MODES(qmv_diag_kernel, NW, SUP, NR, 1, 4) \
    }
#define AQ_QMVD3(NW, SUP, NR)                                                                                      \
    {                                                                                                              \
        {"qmvd_b4_m4_r" #NR "_w" #NW "_d" #SUP "_g0_c3", 4, 4, NR, NW, SUP, 0, 3, 4}, AQ_DIAG_MODES(qmv_diag_kernel, NW, SUP, NR, 1, 3) \
    }
#define AQ_QMVDG(NW, SUP, NR)                                                                                          \
    {                                                                                                                  \
        {"qmvd_b4_m1_r" #NR "_w" #NW "_d" #SUP "_g1", 4, 1, NR, NW, SUP, 1, 0, 4}, {qmv_diag_gather_kernel<NW, SUP, NR, 4, false>, qmv_diag_gather_kernel<NW, SUP, NR, 4, true>, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr} \
    }
#define AQ_QMVDG3(NW, SUP, NR)                                                                                            \
    {                                                                                                                     \
        {"qmvd_b4_m1_r" #NR "_w" #NW "_d" #SUP "_g1_c3", 4, 1, NR, NW, SUP, 1, 3, 4}, {qmv_diag_gather_kernel<NW, SUP, NR, 3, false>, qmv_diag_gather_kernel<NW, SUP, NR, 3, true>, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr} \
    }
#define AQ_QMVD8(NW, SUP, NR)                                                                                   \
    {                                                                                                           \
        {"qmvd_b4_m8_r" #NR "_w" #NW "_d" #SUP "_g0", 4, 8, NR, NW, SUP, 0, 0, 4}, AQ_DIAG_MODES(qmv_diag_kernel, NW, SUP, NR, 2, 4) \
    }
#define AQ_QMVD83(NW, SUP, NR)                                                                                     \
    {                                                                                                              \
        {"qmvd_b4_m8_r" #NR "_w" #NW "_d" #SUP "_g0_c3", 4, 8, NR, NW, SUP, 0, 3, 4}, AQ_DIAG_MODES(qmv_diag_kernel, NW, SUP, NR, 2, 3) \
    }
// kind 5: quantisation groups of 32 codes
#define AQ_QMVDS(NW, SUP, NR)                                                                                          \
    {                                                                                                                  \
        {"qmvd_b4_m2_r" #NR "_w" #NW "_d" #SUP "_g0_s32", 4, 2, NR, NW, SUP, 0, 0, 5}, {qmv_diag_g32_kernel<NW, SUP, NR, 4, 0>, qmv_diag_g32_kernel<NW, SUP, NR, 4, 1>, nullptr, nullptr, qmv_diag_g32_kernel<NW, SUP, NR, 4, 4>, qmv_diag_g32_kernel<NW, SUP, NR, 4, 5>, nullptr, nullptr} \
    }
#define AQ_QMVDS3(NW, SUP, NR)                                                                                            \
    {                                                                                                                     \
        {"qmvd_b4_m2_r" #NR "_w" #NW "_d" #SUP "_g0_s32_c3", 4, 2, NR, NW, SUP, 0, 3, 5}, {qmv_diag_g32_kernel<NW, SUP, NR, 3, 0>, qmv_diag_g32_kernel<NW, SUP, NR, 3, 1>, nullptr, nullptr, qmv_diag_g32_kernel<NW, SUP, NR, 3, 4>, qmv_diag_g32_kernel<NW, SUP, NR, 3, 5>, nullptr, nullptr} \
    }
// 8-bit codes (bits = 8; the split of K is that of a 4-bit row of the same bytes)
#define AQ_QMVDB(NW, SUP, NR)                                                                                          \
    {                                                                                                                  \
        {"qmvd_b8_m4_r" #NR "_w" #NW "_d" #SUP "_g0", 8, 4, NR, NW, SUP, 0, 0, 4}, {qmv_diag_b8_kernel<NW, SUP, NR, 4, 0>, qmv_diag_b8_kernel<NW, SUP, NR, 4, 1>, nullptr, nullptr, qmv_diag_b8_kernel<NW, SUP, NR, 4, 4>, qmv_diag_b8_kernel<NW, SUP, NR, 4, 5>, nullptr, nullptr} \
    }
#define AQ_QMVDB3(NW, SUP, NR)                                                                                            \
    {                                                                                                                     \
        {"qmvd_b8_m4_r" #NR "_w" #NW "_d" #SUP "_g0_c3", 8, 4, NR, NW, SUP, 0, 3, 4}, {qmv_diag_b8_kernel<NW, SUP, NR, 3, 0>, qmv_diag_b8_kernel<NW, SUP, NR, 3, 1>, nullptr, nullptr, qmv_diag_b8_kernel<NW, SUP, NR, 3, 4>, qmv_diag_b8_kernel<NW, SUP, NR, 3, 5>, nullptr, nullptr} \
    }
static const QmvDiagEntry kQmvDiagTable[] = {
    AQ_QMVD(4, 1, 1), AQ_QMVD(4, 1, 2), AQ_QMVD(4, 1, 4), AQ_QMVD(2, 2, 2), AQ_QMVD(2, 1, 2), AQ_QMVD(8, 1, 1),
    AQ_QMVD(4, 2, 1), AQ_QMVD(2, 1, 4), AQ_QMVD(6, 1, 1), AQ_QMVD(10, 1, 1), AQ_QMVD(12, 1, 1),
    AQ_QMVD(14, 1, 1), AQ_QMVD(16, 1, 1), AQ_QMVD8(4, 1, 4), AQ_QMVD8(4, 1, 2), AQ_QMVD8(2, 1, 4),
    AQ_QMVDG(2, 1, 1), AQ_QMVDG(2, 1, 2), AQ_QMVDG(4, 1, 1), AQ_QMVDG(4, 1, 2), AQ_QMVDG(6, 1, 1), AQ_QMVDG(8, 1, 1),
    AQ_QMVD3(4, 1, 1), AQ_QMVD3(4, 1, 2), AQ_QMVD3(4, 1, 4), AQ_QMVD3(2, 1, 2), AQ_QMVD3(2, 1, 4),
    AQ_QMVD83(4, 1, 4), AQ_QMVD83(4, 1, 2), AQ_QMVD83(2, 1, 4), AQ_QMVDG3(2, 1, 2), AQ_QMVDG3(4, 1, 1),
    AQ_QMVDS(2, 1, 2), AQ_QMVDS(4, 1, 1), AQ_QMVDS(4, 1, 2), AQ_QMVDS(8, 1, 1), AQ_QMVDS3(2, 1, 2), AQ_QMVDS3(4, 1, 1),
    AQ_QMVDB(2, 1, 2), AQ_QMVDB(2, 1, 4), AQ_QMVDB(4, 1, 1), AQ_QMVDB(4, 1, 2), AQ_QMVDB(4, 1, 4), AQ_QMVDB(6, 1, 1),
    AQ_QMVDB(8, 1, 1), AQ_QMVDB(10, 1, 1), AQ_QMVDB(12, 1, 1), AQ_QMVDB(14, 1, 1), AQ_QMVDB(16, 1, 1),
    AQ_QMVDB3(4, 1, 1), AQ_QMVDB3(4, 1, 2), AQ_QMVDB3(4, 1, 4), AQ_QMVDB3(2, 1, 2), AQ_QMVDB3(2, 1, 4),
};

static int cps_of(const QmvVariant& v) { return v.xmode ? v.xmode : 4; }
static bool g32_of(const QmvVariant& v) { return v.kind == 5; }
static bool b8_of(const QmvVariant& v) { return v.bits == 8; }
// The length of the 4-bit row that has the bytes of this row: what the split of K goes by.
static int k4_of(int K, int bits) { return bits == 8 ? 2 * K : K; }
// Steps of cps chunks of 256 codes that cover K (its last chunk may be a single half of 128 codes).
static int steps_for(int K, int cps) { return ((K + kDiagChunk - 1) / kDiagChunk + cps - 1) / cps; }
static int cps_for(int K) { return tile_cps_for(K); }

int qmvd_variant_count() { return (int)(sizeof(kQmvDiagTable) / sizeof(kQmvDiagTable[0])); }
const QmvVariant* qmvd_variant(int idx) {
    if (idx < 0 || idx >= qmvd_variant_count()) return nullptr;
    return &kQmvDiagTable[idx].v;
}

bool qmvd_fits(const QmvArgs& a, int bits, int group_size, bool gather, int idx) {
    const QmvVariant* v = qmvd_variant(idx);
    if (!v || bits != v->bits || group_size != (g32_of(*v) ? 32 : 64) || gather != (v->gather != 0)) return false;
    const int K4 = k4_of(a.K, bits);
    if (g32_of(*v) && (a.K % kDiagChunk != 0 || ((reinterpret_cast<uintptr_t>(a.s) | reinterpret_cast<uintptr_t>(a.b)) & 15)))
        return false;
    if (gather && (a.M != 1 || a.routes < 1 || a.routes > 65535)) return false;
    if (a.M < 1 || a.M > v->m || a.K <= 0 || a.K % 128 != 0 || a.N < 1) return false;
    if (steps_for(K4, cps_of(*v)) > v->waves * v->depth) return false;
    const uintptr_t al16 = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.w);
    const uintptr_t al8 = reinterpret_cast<uintptr_t>(a.s) | reinterpret_cast<uintptr_t>(a.b);
    if ((al16 & 15) || (al8 & 7)) return false;
    // 32-bit byte offsets into the packed matrix
    if ((uint64_t)a.N * (uint64_t)(K4 / 2) >= (1ull << 32)) return false;
    if (a.tiled) {
        // the layout is cut for one split of K; 32-bit byte offsets into it
        if (gather || g32_of(*v) || b8_of(*v) || cps_of(*v) != tile_cps_for(a.K)) return false;
        const int64_t total = tile_total_bytes(a.N, a.K, group_size, bits);
        if (total < 0 || total >= ((int64_t)1 << 32)) return false;
    }
    // (up to four steps: two workgroups per CU; longer K: whatever one workgroup may use)
    return qmvd_lds_bytes_for(a.M, a.K, v->waves * v->rows, (v->m + 3) / 4, g32_of(*v), b8_of(*v)) <=
           (size_t)(steps_for(K4, cps_of(*v)) <= 4 ? 96 : 156) * 1024;
}

hipError_t qmvd_launch(int idx, const QmvArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmvd_variant_count()) return hipErrorInvalidValue;
    const QmvDiagEntry& e = kQmvDiagTable[idx];
    const size_t lds = qmvd_lds_bytes_for(a.M, a.K, e.v.waves * e.v.rows, (e.v.m + 3) / 4, g32_of(e.v), b8_of(e.v));
    const int K4 = k4_of(a.K, e.v.bits);
    const int stream_w = !e.v.gather && (int64_t)a.N * (K4 / 2) >= kDiagStreamBytes ? 1 : 0;
    const QmvDiagKernel fn = e.fn[e.v.gather ? (K4 % kDiagChunk == 0 ? 1 : 0) : diag_mode(K4, cps_of(e.v), a.tiled != 0, stream_w != 0)];
    if (!fn) return hipErrorInvalidValue;
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fn), lds)) return rc;
    const int wg_rows = kDiagRows * e.v.rows;
    dim3 grid((unsigned)((a.N + wg_rows - 1) / wg_rows), e.v.gather ? (unsigned)a.routes : 1u, 1u);
    QmvArgs b = a;
    b.stream_w = stream_w;
    b.early_wgs = diag_early_wgs((int64_t)grid.x * grid.y);
    hipLaunchKernelGGL(fn, grid, dim3((unsigned)(e.v.rows * e.v.waves * kWave)), lds, stream, b);
    return hipGetLastError();
}

// The variant the library picks for M rows and this K, or -1: one step of 1024 codes per wavefront; up to 4 steps,
// more rows per workgroup the more activation rows there are to stage.
int qmvd_pick(int M, int K, int N, int bits) {
    if (bits != 4 && bits != 8) return -1;
    if (M < 1 || M > (bits == 8 ? 4 : 8) || K % 128 != 0) return -1;
    const int64_t codes = (int64_t)N * K;
    K = k4_of(K, bits);
    if (K <= 1024) return -1;  // (up to 1024 codes of 4 bits: one wavefront per row set, not built)
    const int cps = cps_for(K);
    const int steps = steps_for(K, cps);
    if (bits == 8) {
        // Where these kernels were measured ahead of the dot2 kernel (one row) and the token-tile kernel (2..4 rows):
        // K of 2048, 4096 or 8192 (4, 8 or 16 whole steps) and up to 40 MiB of codes, e.g. 4096 x 4096 5.5 against
        // 5.7 us (one row) and 6.8 against 8.8 us (four), 8192 x 4096 8.6 against 10.0 us; not 4096 x 14336, 14.7 against
        // 12.7 us, nor 3072 x 6144, 7.1 against 6.0 us, nor four rows of 2048 x 8192, 7.5 against 6.5 us.
        if (cps != 4 || (steps != 4 && steps != 8 && steps != 16) || K % (4 * kDiagChunk) != 0) return -1;
        if (codes > ((int64_t)40 << 20) || (steps == 4 && M > 2)) return -1;
    }
    const int cap = M <= 4 ? 4 : 8;
    int nw, nr;
    if (steps == 2) {
        nw = 2;
        nr = M == 1 ? 2 : 4;
    } else if (steps == 3 || steps == 4) {
        nw = 4;
        nr = M == 1 ? 1 : M == 2 ? 2 : 4;
    } else if (steps <= 16 && M <= 4) {
        // one step per wavefront (an idle one when the count is odd) and one set of rows per workgroup: up to four
        // activation rows of this length fit the LDS (more go in further launches, see run_diag)
        nw = (steps + 1) & ~1;
        nr = 1;
    } else {
        return -1;
    }
    // fewer rows per workgroup while that leaves under 128 workgroups (the 8-row kernels exist for 2 and 4 sets)
    const int min_nr = (cap == 8 || nw == 2) ? 2 : 1;
    while (nr > min_nr && (N + kDiagRows * nr - 1) / (kDiagRows * nr) < 128) nr >>= 1;
    if (cap == 8 && nw == 2) nr = 4;
    // More sets per workgroup where that makes the launch one workgroup per CU (between three quarters of the CUs and
    // all of them): every workgroup then starts at once and none queues behind another on its CU.  4096 x 14336: 224
    // workgroups of 64 rows 7.43 us against 7.66 us for 896 of 16; 4096 x 6144: 192 of 32 rows 4.85 against 5.0 us;
    // 2048 x 16384: 256 of 64 rows 5.30 against 5.45 us.  Not where it leaves more workgroups than CUs (4096 x 28672:
    // 448 of 64 rows 13.6 us against 12.0 us for 1792 of 16).  The bytes of a row do not depend on it.
    if (cap == 4 && bits == 4 && nw <= 4) {
        const int cus = diag_cu_count();
        for (int cand = 4; cand > nr; cand >>= 1) {
            const int wgs = (N + kDiagRows * cand - 1) / (kDiagRows * cand);
            if (wgs <= cus && wgs * 4 >= cus * 3) {
                nr = cand;
                break;
            }
        }
    }
    for (int i = 0; i < qmvd_variant_count(); i++) {
        const QmvVariant& v = kQmvDiagTable[i].v;
        if (v.bits == bits && v.waves == nw && v.depth == 1 && v.rows == nr && v.m == cap && !v.gather && cps_of(v) == cps && !g32_of(v)) return i;
    }
    return -1;
}

// The group-32 variant for up to two rows and this K (a multiple of 256), or -1.
int qmvd_pick_g32(int M, int K, int N) {
    if (M < 1 || M > 2 || K <= 1024 || K % kDiagChunk != 0) return -1;
    const int cps = cps_for(K);
    const int steps = steps_for(K, cps);
    if (steps > 8) return -1;
    const int nw = (steps + 1) & ~1;
    int nr = nw == 2 ? 2 : (nw == 4 && M == 2 && N >= 4096) ? 2 : 1;
    for (int pass = 0; pass < 2; pass++) {
        for (int i = 0; i < qmvd_variant_count(); i++) {
            const QmvVariant& v = kQmvDiagTable[i].v;
            if (g32_of(v) && v.waves == nw && v.depth == 1 && v.rows == nr && cps_of(v) == cps) return i;
        }
        nr = 1;
    }
    return -1;
}

// act(gate . x) * (up . x) with the variant's (wavefronts, steps) split of K; a.w2 / a.s2 / a.b2 are the `up` matrix.
struct QmvDiagPairEntry {
    int nw, sup, cps;
    QmvDiagKernel fn[8], gather_fn[2];  // gather_fn[1]: K a whole number of chunks
};
#define AQ_QMVD_PAIR(NW, SUP, CPS) {NW, SUP, CPS, AQ_DIAG_MODES(qmv_diag_pair_kernel, NW, SUP, CPS), {qmv_diag_gather_pair_kernel<NW, SUP, CPS, false>, qmv_diag_gather_pair_kernel<NW, SUP, CPS, true>}}
static const QmvDiagPairEntry kQmvDiagPairTable[] = {
    AQ_QMVD_PAIR(2, 1, 4), AQ_QMVD_PAIR(4, 1, 4), AQ_QMVD_PAIR(6, 1, 4), AQ_QMVD_PAIR(8, 1, 4),
    AQ_QMVD_PAIR(2, 1, 3), AQ_QMVD_PAIR(4, 1, 3),
};
static const QmvDiagPairEntry* find_pair(int idx) {
    const QmvVariant* v = qmvd_variant(idx);
    if (v)
        for (const QmvDiagPairEntry& e : kQmvDiagPairTable)
            if (e.nw == v->waves && e.sup == v->depth && e.cps == cps_of(*v) && !g32_of(*v) && !b8_of(*v)) return &e;
    return nullptr;
}
bool qmvd_pair_supported(int idx) { return find_pair(idx) != nullptr; }

hipError_t qmvd_pair_launch(int idx, const QmvArgs& a, bool gather, hipStream_t stream) {
    const QmvDiagPairEntry* e = find_pair(idx);
    if (!e) return hipErrorInvalidValue;
    const int stream_w = !gather && (int64_t)2 * a.N * (a.K / 2) >= kDiagStreamBytes ? 1 : 0;
    const QmvDiagKernel fn = gather ? e->gather_fn[a.K % kDiagChunk == 0 ? 1 : 0] : e->fn[diag_mode(a.K, e->cps, a.tiled != 0, stream_w != 0)];
    const size_t lds = qmvd_lds_bytes_for(gather ? 1 : a.M, a.K, 2 * e->nw);
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fn), lds)) return rc;
    dim3 grid((unsigned)((a.N + kDiagRows - 1) / kDiagRows), gather ? (unsigned)a.routes : 1u, 1u);
    QmvArgs b = a;
    b.stream_w = stream_w;
    b.early_wgs = diag_early_wgs((int64_t)grid.x * grid.y);
    hipLaunchKernelGGL(fn, grid, dim3((unsigned)(2 * e->nw * kWave)), lds, stream, b);
    return hipGetLastError();
}

// The gathered variant for this K (one activation row per route), or -1.
int qmvd_pick_gather(int K) {
    if (K <= 1024 || K % 128 != 0) return -1;
    const int cps = cps_for(K);
    const int steps = steps_for(K, cps);
    if (steps < 2 || steps > 8) return -1;
    const int nw = (steps + 1) & ~1;
    const int nr = nw == 2 ? 2 : 1;
    for (int i = 0; i < qmvd_variant_count(); i++) {
        const QmvVariant& v = kQmvDiagTable[i].v;
        if (v.gather && v.waves == nw && v.depth == 1 && v.rows == nr && cps_of(v) == cps && !g32_of(v)) return i;
    }
    return -1;
}

// lm_head epilogues on variant idx's split of K: fuse 4 writes packed scores to a.y, fuse 3 one partial maximum per
// set of 16 rows into a.partial (qmvd_head_partials slots), which the caller folds.
struct QmvDiagHeadEntry {
    int nw, sup, nr, cps, g32, fuse;
    QmvDiagKernel fn, fn_even;  // any K the split covers; K a whole number of steps
};
#define AQ_QMVD_HEAD(NW, NR, CPS, G32)                                                                                              \
    {NW, 1, NR, CPS, G32, 3, qmv_diag_head_kernel<NW, 1, NR, CPS, (G32 != 0), 3, false>, qmv_diag_head_kernel<NW, 1, NR, CPS, (G32 != 0), 3, true>}, \
    {NW, 1, NR, CPS, G32, 4, qmv_diag_head_kernel<NW, 1, NR, CPS, (G32 != 0), 4, false>, qmv_diag_head_kernel<NW, 1, NR, CPS, (G32 != 0), 4, true>}
static const QmvDiagHeadEntry kQmvDiagHeadTable[] = {
    AQ_QMVD_HEAD(2, 2, 3, 1), AQ_QMVD_HEAD(2, 2, 4, 1), AQ_QMVD_HEAD(4, 1, 4, 1), AQ_QMVD_HEAD(4, 1, 3, 1),
    AQ_QMVD_HEAD(2, 2, 3, 0), AQ_QMVD_HEAD(2, 2, 4, 0), AQ_QMVD_HEAD(4, 1, 4, 0), AQ_QMVD_HEAD(4, 1, 3, 0),
};
static const QmvDiagHeadEntry* find_head(int idx, int fuse) {
    const QmvVariant* v = qmvd_variant(idx);
    if (v && !v->gather && !b8_of(*v))
        for (const QmvDiagHeadEntry& e : kQmvDiagHeadTable)
            if (e.nw == v->waves && e.sup == v->depth && e.nr == v->rows && e.cps == cps_of(*v) &&
                (e.g32 != 0) == g32_of(*v) && e.fuse == fuse)
                return &e;
    return nullptr;
}
bool qmvd_head_supported(int idx, int fuse) { return find_head(idx, fuse) != nullptr; }
size_t qmvd_head_partials(int idx, int N) {
    const QmvVariant* v = qmvd_variant(idx);
    const int wg_rows = kDiagRows * (v ? v->rows : 1);
    return (size_t)((N + wg_rows - 1) / wg_rows) * (v ? v->rows : 1);
}
hipError_t qmvd_head_launch(int idx, int fuse, const QmvArgs& a, hipStream_t stream) {
    const QmvDiagHeadEntry* e = find_head(idx, fuse);
    if (!e || a.M != 1 || (fuse == 3 && !a.partial)) return hipErrorInvalidValue;
    const size_t lds = qmvd_lds_bytes_for(1, a.K, e->nw * e->nr, 1, e->g32 != 0);
    const QmvDiagKernel fn = a.K % (e->cps * kDiagChunk) == 0 ? e->fn_even : e->fn;
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fn), lds)) return rc;
    const int wg_rows = kDiagRows * e->nr;
    QmvArgs b = a;
    b.early_wgs = diag_early_wgs((a.N + wg_rows - 1) / wg_rows);
    hipLaunchKernelGGL(fn, dim3((unsigned)((a.N + wg_rows - 1) / wg_rows)), dim3((unsigned)(e->nw * e->nr * kWave)), lds,
                       stream, b);
    return hipGetLastError();
}

typedef void (*QmvDiagMultiKernel)(const QmvMultiArgs);
struct QmvDiagMultiEntry {
    int nw, sup, nr, cps;
    QmvDiagMultiKernel fn[8];
};
#define AQ_QMVD_MULTI(NW, SUP, NR) {NW, SUP, NR, 4, AQ_DIAG_MODES(qmv_diag_multi_kernel, NW, SUP, NR, 4)}
#define AQ_QMVD_MULTI3(NW, SUP, NR) {NW, SUP, NR, 3, AQ_DIAG_MODES(qmv_diag_multi_kernel, NW, SUP, NR, 3)}
static const QmvDiagMultiEntry kQmvDiagMultiTable[] = {
    AQ_QMVD_MULTI(4, 1, 1), AQ_QMVD_MULTI(4, 1, 2), AQ_QMVD_MULTI(4, 1, 4), AQ_QMVD_MULTI(2, 1, 2), AQ_QMVD_MULTI(2, 1, 4),
    AQ_QMVD_MULTI(6, 1, 1), AQ_QMVD_MULTI(8, 1, 1), AQ_QMVD_MULTI(10, 1, 1), AQ_QMVD_MULTI(12, 1, 1), AQ_QMVD_MULTI(14, 1, 1),
    AQ_QMVD_MULTI(16, 1, 1), AQ_QMVD_MULTI3(4, 1, 1), AQ_QMVD_MULTI3(4, 1, 2), AQ_QMVD_MULTI3(4, 1, 4), AQ_QMVD_MULTI3(2, 1, 2),
    AQ_QMVD_MULTI3(2, 1, 4),
};

// The multi-matrix launch of variant idx (the same arithmetic, so the same bytes, as one launch per matrix).
bool qmvd_multi_supported(int idx) {
    const QmvVariant* v = qmvd_variant(idx);
    if (!v || b8_of(*v)) return false;
    for (const QmvDiagMultiEntry& e : kQmvDiagMultiTable)
        if (e.nw == v->waves && e.sup == v->depth && e.nr == v->rows && e.cps == cps_of(*v) && !g32_of(*v)) return true;
    return false;
}

hipError_t qmvd_multi_launch(int idx, QmvMultiArgs ma, hipStream_t stream) {
    const QmvVariant* v = qmvd_variant(idx);
    const QmvDiagMultiEntry* e = nullptr;
    if (v)
        for (const QmvDiagMultiEntry& c : kQmvDiagMultiTable)
            if (c.nw == v->waves && c.sup == v->depth && c.nr == v->rows && c.cps == cps_of(*v)) e = &c;
    if (!e || ma.count < 1 || ma.count > kQmvMultiMax) return hipErrorInvalidValue;
    const int wg_rows = kDiagRows * e->nr;
    int blocks = 0;
    for (int i = 0; i < ma.count; i++) {
        blocks += (ma.N[i] + wg_rows - 1) / wg_rows;
        ma.block_end[i] = blocks;
    }
    const size_t lds = qmvd_lds_bytes_for(ma.common.M, ma.common.K, e->nw * e->nr);
    int64_t bytes = 0;
    for (int i = 0; i < ma.count; i++) bytes += (int64_t)ma.N[i] * (ma.common.K / 2);
    ma.common.stream_w = bytes >= kDiagStreamBytes ? 1 : 0;
    ma.common.early_wgs = diag_early_wgs(blocks);
    const QmvDiagMultiKernel fn = e->fn[diag_mode(ma.common.K, e->cps, ma.common.tiled != 0, ma.common.stream_w != 0)];
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fn), lds)) return rc;
    hipLaunchKernelGGL(fn, dim3((unsigned)blocks), dim3((unsigned)(e->nw * e->nr * kWave)), lds, stream, ma);
    return hipGetLastError();
}

}  // namespace aq
