// affine_qmv / gather_qmv for gfx950 on the matrix cores, M = 1..32 activation rows.
//
// Same contract as the dot2 kernels (aq_qmv.hip): replaces rocm_mlx_q4_projection* and
// rocm_mlx_q4_projection_batch* for decode-sized M
// (go/engine/hip/kernels/quant/affine_projection.hipinc:3-266, affine_projection_tuned.hipinc:166-472)
// and rocm_moe_mlx_affine_routes (go/engine/hip/kernels/moe/routing.hipinc:160-399), with the
// semantics of MLX affine_qmv / lthn_qmv_rows / gather_qmv (go/engine/metal/qmv.go:354-421,
// go/engine/metal/qmv_rows.go:14-60, kernels/moe/lthn_gather_qmv.metal:54-66).
//
// Why MFMA for a matvec: at 8 TB/s a CU must retire ~26 four-bit codes per clock, which leaves
// ~2.4 VALU lane-ops per code; unpack + dot2 + bookkeeping costs more than that.  Feeding the
// codes (bf16 128+c, exact) to v_mfma_f32_32x32x16_bf16 moves every multiply-add off the VALU:
// what is left per 32 codes is 28 unpack ops and a handful of fp32 FMAs, and the M dimension of
// the MFMA makes M = 2..32 rows cost the same weight traffic and almost the same VALU as M = 1.
//
// Work split: a workgroup owns 32 consecutive output rows; its KS wavefronts split K into
// contiguous ranges of 64-code group blocks.  In the MFMA, lane (j, h) supplies weight row n0+j
// and, per group block, the codes [32h, 32h+32); word t of those is the B operand of MFMA step t,
// so a group block is 4 MFMAs whose k-slots all lie in one quantisation group.  Loading in that
// layout directly would touch 32 rows x 32 bytes per instruction, which backs up the address
// pipeline; weights are therefore fetched as whole 128-byte row segments and transposed through
// LDS (see the kernel).  The A operand is x, staged once per workgroup into LDS in fragment order
// (for M = 1 every lane reads the same 16 bytes: a broadcast); scales and biases of the 32 rows
// are staged once as well.  Per group block:
//     P        = sum_k x[m,k] * (off + c[n,k])           (MFMA, fp32)
//     acc[m,n] += scale * P + (bias - off*scale) * Sx[m,g]   (VALU fp32, Sx from LDS)
// the reference's own factorisation (affine_dot.hipinc:546-573).  Partial sums of the KS
// wavefronts meet in LDS; 32 consecutive outputs are stored together.
#include "aq_device.h"
#include "aq_kernels.h"

namespace aq {

namespace {

// Rows of the 32x32 MFMA result a lane holds in its first MR registers:
// register r of lane (j, h) is row 8*(r/4) + 4*h + r%4, column j.
template <int MR>
struct RowClass;
template <>
struct RowClass<1> {
    static constexpr int kMaxM = 1;
    static constexpr int kSums = 4;  // Sx slots kept per group block
};
template <>
struct RowClass<4> {
    static constexpr int kMaxM = 8;
    static constexpr int kSums = 8;
};
template <>
struct RowClass<8> {
    static constexpr int kMaxM = 16;
    static constexpr int kSums = 16;
};
template <>
struct RowClass<16> {
    static constexpr int kMaxM = 32;
    static constexpr int kSums = 32;
};

}  // namespace

// One "step" of a wavefront is 128 bytes of every one of its 32 weight rows (4 group blocks at
// 4 bit, 2 at 8 bit): four global_load_dwordx4 whose 64 lanes cover 8 rows x 128 contiguous bytes
// each (whole cache lines), parked in registers, then transposed through a wavefront-private LDS
// tile (row stride 144 bytes, conflict-free both ways) into the MFMA operand layout, where lane
// (j, h) needs the 32 codes [32h, 32h+32) of row j's group block.
template <int BITS, int MR, int KS, bool GATHER>
__global__ __launch_bounds__(KS* kWave) void qmv_mfma_kernel(const QmvArgs a) {
    constexpr int NT = KS * kWave;
    constexpr int MS = RowClass<MR>::kSums;
    constexpr int GPS = BITS == 4 ? 4 : 2;           // group blocks per step
    constexpr int GROUP_BYTES = 8 * BITS;             // packed bytes of one group block of one row
    constexpr int WROW = 144;                         // LDS row stride of the weight tile
    constexpr float kOff = BITS == 4 ? kNibbleOffset : 0.0f;
    extern __shared__ __align__(16) uint8_t lds[];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int j = lane & 31;
    const int h = lane >> 5;
    const int K = a.K, N = a.N, M = a.M;
    const int G = K >> 6;  // 64-code group blocks == quantisation groups (group size 64)
    const uint32_t row_bytes = (uint32_t)K * BITS / 8;

    // LDS carve-up
    uint8_t* xfrag = lds;                                                   // [G][4][2][M] x 16 B
    float* xsum = reinterpret_cast<float*>(lds + (size_t)M * K * 2);        // [G][MS]
    uint32_t* sbuf = reinterpret_cast<uint32_t*>(xsum + (size_t)G * MS);    // [G/2][32] scale pairs
    uint32_t* bbuf = sbuf + (size_t)(G / 2) * 32;                           // [G/2][32] bias pairs
    uint8_t* wtile = reinterpret_cast<uint8_t*>(bbuf + (size_t)(G / 2) * 32) + (size_t)wave * (32 * WROW);
    float* red = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(bbuf + (size_t)(G / 2) * 32) + (size_t)KS * (32 * WROW));

    const char* wbase = reinterpret_cast<const char*>(a.w);
    const uint32_t* sbase = reinterpret_cast<const uint32_t*>(a.s);
    const uint32_t* bbase = reinterpret_cast<const uint32_t*>(a.b);
    const uint16_t* xrow = a.x;
    int64_t yoff = 0;
    bool route_ok = true;
    if constexpr (GATHER) {
        const int z = blockIdx.y;
        const int e = a.rhs[z];
        int xr = a.lhs ? a.lhs[z] : 0;
        route_ok = (unsigned)e < (unsigned)a.num_experts && (unsigned)xr < (unsigned)a.x_rows;
        const int64_t row0 = route_ok ? ((int64_t)e * a.expert_rows + a.row_base) : 0;
        if (!route_ok) xr = 0;
        wbase += row0 * row_bytes;
        sbase += row0 * (G / 2);
        bbase += row0 * (G / 2);
        xrow += (int64_t)xr * K;
        yoff = (int64_t)z * N;
    }
    const int n0 = blockIdx.x * 32;
    const int rows_here = min(32, N - n0);  // rows past it are clamped for loads, masked for stores

    // ---- 1. staging loads first: x pieces, scale and bias pairs ----
    constexpr int XPT = 2;
    const int chunks_per_row = K >> 3;
    const int pieces = M * chunks_per_row;
    uint4 xstage[XPT];
    {
        const uint4* src = reinterpret_cast<const uint4*>(xrow);
#pragma unroll
        for (int q = 0; q < XPT; q++) {
            const int p = tid + q * NT;
            if (p < pieces) xstage[q] = src[p];
        }
    }
    const int half_g = G >> 1;
    const int sb_words = 32 * half_g;  // dwords of scales (and of biases) this workgroup needs
    constexpr int SPT = 2;
    uint32_t sstage[SPT], bstage[SPT];
    {
        const uint32_t* sp = sbase + (int64_t)n0 * half_g;
        const uint32_t* bp = bbase + (int64_t)n0 * half_g;
        const int valid_words = rows_here * half_g;
#pragma unroll
        for (int q = 0; q < SPT; q++) {
            const int d = tid + q * NT;
            if (d < sb_words) {
                const int dd = min(d, valid_words - 1);
                sstage[q] = sp[dd];
                bstage[q] = bp[dd];
            }
        }
    }

    // ---- 2. this wavefront's K range and its first two steps of weights ----
    int gpw = (G + KS - 1) / KS;
    gpw = (gpw + GPS - 1) / GPS * GPS;
    const int g_begin = min(wave * gpw, G);
    const int g_end = min(G, g_begin + gpw);
    const int nsteps = (g_end - g_begin + GPS - 1) / GPS;

    wbase += (int64_t)n0 * row_bytes;
    const uint32_t lchunk = (uint32_t)(lane & 7) * 16u;
    uint32_t wrow_off[4];
#pragma unroll
    for (int i = 0; i < 4; i++) wrow_off[i] = (uint32_t)min(8 * i + (lane >> 3), rows_here - 1) * row_bytes;

    auto load_step = [&](uint4 (&r)[4], int step) {
        // byte offset of this lane's 16 bytes inside a row, kept inside the row
        const uint32_t col = min((uint32_t)(g_begin + step * GPS) * GROUP_BYTES + lchunk, row_bytes - 16u);
#pragma unroll
        for (int i = 0; i < 4; i++) r[i] = *reinterpret_cast<const uint4*>(wbase + (wrow_off[i] + col));
    };

    uint4 ra[4], rb[4];
    load_step(ra, 0);
    load_step(rb, 1);

    // ---- 3. stage x into fragment order with per-(row, group block) sums; scales/biases as [pair][row] ----
    auto stage_piece = [&](int p, uint4 v) {
        const int m = p / chunks_per_row;
        const int c = p - m * chunks_per_row;
        const int g = c >> 3, c8 = c & 7;
        float sx = 0.0f;
        sx = dot2_bf16(v.x, 0x3F803F80u, sx);
        sx = dot2_bf16(v.y, 0x3F803F80u, sx);
        sx = dot2_bf16(v.z, 0x3F803F80u, sx);
        sx = dot2_bf16(v.w, 0x3F803F80u, sx);
        // 8 consecutive lanes hold one (row, group block): xor 1, xor 2, mirror within 8
        sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0xB1, 0xF, 0xF, true));
        sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0x4E, 0xF, 0xF, true));
        sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0x141, 0xF, 0xF, true));
        if (c8 == 0) xsum[g * MS + m] = sx;
        if constexpr (BITS == 4) {
            // (x0,x1)(x2,x3)(x4,x5)(x6,x7) -> (x0,x4)(x1,x5)(x2,x6)(x3,x7): the order unpack4_word emits codes
            uint4 o;
            o.x = (v.x & 0xffffu) | (v.z << 16);
            o.y = (v.x >> 16) | (v.z & 0xffff0000u);
            o.z = (v.y & 0xffffu) | (v.w << 16);
            o.w = (v.y >> 16) | (v.w & 0xffff0000u);
            v = o;
        }
        const int t = c8 & 3, hh = c8 >> 2;
        *reinterpret_cast<uint4*>(xfrag + ((size_t)(((g * 4 + t) * 2 + hh) * M + m) << 4)) = v;
    };
    auto stage_sb = [&](int d, uint32_t sv, uint32_t bv) {
        const int row = d / half_g;
        const int q = d - row * half_g;
        sbuf[q * 32 + row] = sv;
        bbuf[q * 32 + row] = bv;
    };
    {
        // pieces is a multiple of 8 and the 8 lanes of a (row, group block) are all in or all out of
        // range together, so the DPP sums above always see their partners
        const uint4* src = reinterpret_cast<const uint4*>(xrow);
#pragma unroll
        for (int q = 0; q < XPT; q++) {
            const int p = tid + q * NT;
            if (p < pieces) stage_piece(p, xstage[q]);
        }
        for (int p = tid + XPT * NT; p < pieces; p += NT) stage_piece(p, src[p]);
        const uint32_t* sp = sbase + (int64_t)n0 * half_g;
        const uint32_t* bp = bbase + (int64_t)n0 * half_g;
        const int valid_words = rows_here * half_g;
#pragma unroll
        for (int q = 0; q < SPT; q++) {
            const int d = tid + q * NT;
            if (d < sb_words) stage_sb(d, sstage[q], bstage[q]);
        }
        for (int d = tid + SPT * NT; d < sb_words; d += NT) {
            const int dd = min(d, valid_words - 1);
            stage_sb(d, sp[dd], bp[dd]);
        }
    }
    __syncthreads();

    float acc[MR];
#pragma unroll
    for (int r = 0; r < MR; r++) acc[r] = 0.0f;

    const uint32_t mask_s = opaque_s(kNibbleMask);   // both stay in registers so that
    const uint32_t magic_v = opaque_v(kMagic128);    // (w & mask) | magic is a single v_and_or_b32
    const int arow = min(j, M - 1);                  // A-operand row of this lane (rows >= M repeat the last one)
    uint8_t* wwrite = wtile + (lane >> 3) * WROW + (lane & 7) * 16;
    const uint8_t* wread = wtile + j * WROW + h * (GROUP_BYTES / 2);

    auto process_step = [&](const uint4 (&r)[4], int step) {
#pragma unroll
        for (int i = 0; i < 4; i++) *reinterpret_cast<uint4*>(wwrite + i * 8 * WROW) = r[i];
        const int g0 = g_begin + step * GPS;
        uint32_t spair[GPS / 2], bpair[GPS / 2];
#pragma unroll
        for (int q = 0; q < GPS / 2; q++) {
            const int pi = min((g0 >> 1) + q, half_g - 1);
            spair[q] = sbuf[pi * 32 + j];
            bpair[q] = bbuf[pi * 32 + j];
        }
#pragma unroll
        for (int u = 0; u < GPS; u++) {
            const int gg = g0 + u;
            if (gg < g_end) {
                uint32_t wq[BITS == 4 ? 4 : 8];
                {
                    const uint4* wp = reinterpret_cast<const uint4*>(wread + u * GROUP_BYTES);
#pragma unroll
                    for (int v = 0; v < (BITS == 4 ? 1 : 2); v++) {
                        const uint4 d = wp[v];
                        wq[4 * v + 0] = d.x;
                        wq[4 * v + 1] = d.y;
                        wq[4 * v + 2] = d.z;
                        wq[4 * v + 3] = d.w;
                    }
                }
                f32x16_t p = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const bf16x8_t af = *reinterpret_cast<const bf16x8_t*>(
                        xfrag + ((size_t)(((gg * 4 + t) * 2 + h) * M + arow) << 4));
                    uint32_t f[4];
                    if constexpr (BITS == 4) {
                        unpack4_word(wq[t], mask_s, magic_v, f);
                    } else {
                        unpack8_word(wq[2 * t], f);
                        unpack8_word(wq[2 * t + 1], f + 2);
                    }
                    const uint4 fv = {f[0], f[1], f[2], f[3]};
                    p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, __builtin_bit_cast(bf16x8_t, fv), p, 0, 0, 0);
                }
                const uint32_t sbits = (u & 1) ? (spair[u >> 1] >> 16) : (spair[u >> 1] & 0xffffu);
                const uint32_t bbits = (u & 1) ? (bpair[u >> 1] >> 16) : (bpair[u >> 1] & 0xffffu);
                const float sc = bf16_bits_to_f32(sbits);
                const float bo = __fmaf_rn(sc, -kOff, bf16_bits_to_f32(bbits));
                if constexpr (MR == 1) {
                    const float sx = xsum[gg * MS];
                    acc[0] = __fmaf_rn(sc, p[0], acc[0]);
                    acc[0] = __fmaf_rn(bo, sx, acc[0]);
                } else {
#pragma unroll
                    for (int r4 = 0; r4 < MR / 4; r4++) {
                        const float4 sx = *reinterpret_cast<const float4*>(xsum + gg * MS + 8 * r4 + 4 * h);
                        acc[4 * r4 + 0] = __fmaf_rn(sc, p[4 * r4 + 0], acc[4 * r4 + 0]);
                        acc[4 * r4 + 1] = __fmaf_rn(sc, p[4 * r4 + 1], acc[4 * r4 + 1]);
                        acc[4 * r4 + 2] = __fmaf_rn(sc, p[4 * r4 + 2], acc[4 * r4 + 2]);
                        acc[4 * r4 + 3] = __fmaf_rn(sc, p[4 * r4 + 3], acc[4 * r4 + 3]);
                        acc[4 * r4 + 0] = __fmaf_rn(bo, sx.x, acc[4 * r4 + 0]);
                        acc[4 * r4 + 1] = __fmaf_rn(bo, sx.y, acc[4 * r4 + 1]);
                        acc[4 * r4 + 2] = __fmaf_rn(bo, sx.z, acc[4 * r4 + 2]);
                        acc[4 * r4 + 3] = __fmaf_rn(bo, sx.w, acc[4 * r4 + 3]);
                    }
                }
            }
        }
    };

    for (int st = 0; st < nsteps; st += 2) {
        process_step(ra, st);
        load_step(ra, st + 2);
        if (st + 1 < nsteps) process_step(rb, st + 1);
        load_step(rb, st + 3);
    }

    // ---- combine the KS partial sums, store 32 consecutive outputs per row ----
#pragma unroll
    for (int r = 0; r < MR; r++) red[(wave * MR + r) * kWave + lane] = acc[r];
    __syncthreads();
    for (int e = tid; e < MR * kWave; e += NT) {
        const int r = e / kWave, l = e & (kWave - 1);
        float tot = 0.0f;
#pragma unroll
        for (int w = 0; w < KS; w++) tot += red[(w * MR + r) * kWave + l];
        if (!route_ok) tot = 0.0f;
        const int m = 8 * (r >> 2) + 4 * (l >> 5) + (r & 3);
        const int col = n0 + (l & 31);
        if (m < M && col < N) {
            const int64_t o = yoff + (int64_t)m * N + col;
            if (a.out_f32) {
                reinterpret_cast<float*>(a.y)[o] = tot;
            } else {
                reinterpret_cast<uint16_t*>(a.y)[o] = f32_to_bf16_bits(tot);
            }
        }
    }
}

// ---- variant table --------------------------------------------------------

namespace {

typedef void (*QmvKernel)(const QmvArgs);
struct Entry {
    QmvVariant v;
    QmvKernel fn;
    int mr;
};

#define AQ_QMX(BITS, MR, KS, G)                                                                              \
    {                                                                                                        \
        {"qmvx_b" #BITS "_mr" #MR "_ks" #KS "_g" #G, BITS, RowClass<MR>::kMaxM, 32, KS, 2, G, 0, 1},         \
            qmv_mfma_kernel<BITS, MR, KS, (G != 0)>, MR                                                      \
    }

#define AQ_QMX_SET(BITS)                                                                                     \
    AQ_QMX(BITS, 1, 2, 0), AQ_QMX(BITS, 1, 4, 0), AQ_QMX(BITS, 1, 8, 0), AQ_QMX(BITS, 1, 16, 0),              \
        AQ_QMX(BITS, 4, 4, 0), AQ_QMX(BITS, 4, 8, 0), AQ_QMX(BITS, 4, 16, 0), AQ_QMX(BITS, 8, 4, 0),          \
        AQ_QMX(BITS, 8, 8, 0), AQ_QMX(BITS, 8, 16, 0), AQ_QMX(BITS, 16, 4, 0), AQ_QMX(BITS, 16, 8, 0),        \
        AQ_QMX(BITS, 16, 16, 0), AQ_QMX(BITS, 1, 1, 1), AQ_QMX(BITS, 1, 2, 1), AQ_QMX(BITS, 1, 4, 1),         \
        AQ_QMX(BITS, 1, 8, 1)

const Entry kTable[] = {AQ_QMX_SET(4), AQ_QMX_SET(8)};

}  // namespace

int qmvx_variant_count() { return (int)(sizeof(kTable) / sizeof(kTable[0])); }

const QmvVariant* qmvx_variant(int idx) {
    if (idx < 0 || idx >= qmvx_variant_count()) return nullptr;
    return &kTable[idx].v;
}

size_t qmvx_lds_bytes(int idx, const QmvArgs& a) {
    if (idx < 0 || idx >= qmvx_variant_count()) return 0;
    const Entry& e = kTable[idx];
    const size_t G = (size_t)a.K / 64;
    size_t ms = e.mr == 1 ? 4 : (e.mr == 4 ? 8 : (e.mr == 8 ? 16 : 32));
    return (size_t)a.M * a.K * 2 + G * ms * 4 + 2 * (G / 2) * 32 * 4 + (size_t)e.v.waves * 32 * 144 +
           (size_t)e.v.waves * e.mr * kWave * 4;
}

hipError_t qmvx_launch(int idx, const QmvArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmvx_variant_count()) return hipErrorInvalidValue;
    const Entry& e = kTable[idx];
    dim3 grid((unsigned)((a.N + 31) / 32), e.v.gather ? (unsigned)a.routes : 1u, 1u);
    dim3 block((unsigned)(e.v.waves * kWave), 1u, 1u);
    const size_t lds = qmvx_lds_bytes(idx, a);
    if (lds > 48 * 1024) {
        hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(e.fn),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (rc != hipSuccess) return rc;
    }
    hipLaunchKernelGGL(e.fn, grid, block, lds, stream, a);
    return hipGetLastError();
}

}  // namespace aq
