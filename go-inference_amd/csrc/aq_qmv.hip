// affine_qmv / gather_qmv for gfx950, M = 1..4 activation rows.
//
// Replaces rocm_mlx_q4_projection* (go/engine/hip/kernels/quant/affine_projection.hipinc:3-266,
// row body affine_dot.hipinc:524-679) and rocm_moe_mlx_affine_routes
// (go/engine/hip/kernels/moe/routing.hipinc:160-399); semantics are those of
// MLX affine_qmv / affine_gather_qmv as driven by go/engine/metal/qmv.go:354-421
// and kernels/moe/lthn_gather_qmv.metal:54-66.
//
// Shape of the computation (HBM-bound; the packed weights are read exactly once):
//   * a wavefront owns R consecutive output rows; a row's packed codes are cut
//     into "slices" of 64 x 16 bytes, so every global_load_dwordx4 of a
//     wavefront is one fully coalesced 1 KiB read (32 codes per lane at 4 bit,
//     16 at 8 bit); `DEPTH` slices are kept in flight per wavefront;
//   * the activations are staged once per workgroup into LDS as bf16 pairs in
//     the order the unpacker produces codes, and read back 64 B per lane;
//   * codes become bf16 pairs with one v_and_or_b32 per pair (4 bit) or
//     cvt_f32_ubyte + v_perm (8 bit) and feed v_dot2c_f32_bf16 (fp32 sums);
//   * per 16-byte chunk: acc += scale * dot + (bias - off*scale) * sum(x),
//     the reference's own factorisation (affine_dot.hipinc:546-573);
//   * a DPP wave reduction, then lane 0 stores bf16 (RNE) or fp32.
#include "aq_device.h"
#include "aq_kernels.h"

namespace aq {

template <int BITS>
struct Codec;

template <>
struct Codec<4> {
    static constexpr int kCodesPerChunk = 32;  // one 16-byte chunk
    static constexpr int kPairs = 16;          // bf16 pairs per chunk
    static constexpr float kOffset = kNibbleOffset;
};
template <>
struct Codec<8> {
    static constexpr int kCodesPerChunk = 16;
    static constexpr int kPairs = 8;
    static constexpr float kOffset = 0.0f;
};

// One slice of R rows held in registers (plus, in direct-x mode, the lane's x chunk).
template <int R, int XREGS>
struct Slice {
    uint4 w[R];
    uint16_t s[R];
    uint16_t b[R];
    uint4 x[XREGS > 0 ? XREGS : 1];
};

// XMODE 0: x staged once per workgroup into LDS (x loads are issued before any weight load so the
//          barrier never waits for HBM); XMODE 1 (M == 1 only): every lane pulls its own 64-byte
//          x chunk straight from global/L2 with the slice, no LDS and no barrier.
// bx: this workgroup's position among those of one weight matrix (blockIdx.x for a plain launch).
template <int BITS, int M, int R, int NW, int DEPTH, bool GATHER, int XMODE>
__device__ __forceinline__ void qmv_dot2_body(const QmvArgs& a, const int bx) {
    using C = Codec<BITS>;
    constexpr int CPC = C::kCodesPerChunk;
    constexpr int PAIRS = C::kPairs;
    constexpr int XREGS = XMODE == 1 ? PAIRS / 4 : 0;
    static_assert(XMODE == 0 || M == 1, "direct x mode is single-row only");
    extern __shared__ uint32_t xs[];  // [M][K/2] bf16 pairs, unpack order (XMODE 0)

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int K = a.K;
    const int N = a.N;
    const int chunks_per_row = K / CPC;  // 16-byte chunks in a packed row
    const uint32_t row_bytes = (uint32_t)chunks_per_row * 16u;
    const int groups_per_row = K >> a.gs_shift;
    const int nslices = (chunks_per_row + kWave - 1) / kWave;

    const char* wbase = reinterpret_cast<const char*>(a.w);
    const char* sbase = reinterpret_cast<const char*>(a.s);
    const char* bbase = reinterpret_cast<const char*>(a.b);
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
        sbase += row0 * groups_per_row * 2;
        bbase += row0 * groups_per_row * 2;
        xrow += (int64_t)xr * K;
        yoff = (int64_t)z * N;
    }

    // wave-uniform 64-bit bases + 32-bit lane offsets: rows past N are clamped onto the last row
    const int row_first = (bx * NW + wave) * R;
    const int row_base_clamped = min(row_first, N - 1);
    wbase += (int64_t)row_base_clamped * row_bytes;
    sbase += (int64_t)row_base_clamped * groups_per_row * 2;
    bbase += (int64_t)row_base_clamped * groups_per_row * 2;
    uint32_t rel[R];
#pragma unroll
    for (int r = 0; r < R; r++) rel[r] = (uint32_t)min(r, N - 1 - row_base_clamped);

    // Stage x (XMODE 0): global loads first, so that nothing below queues ahead of them.
    constexpr int XPT = 4;  // 16-byte x pieces held per thread between load and LDS write
    uint4 xstage[XPT];
    const int pieces = M * (K / 8);
    if constexpr (XMODE == 0) {
        const uint4* src = reinterpret_cast<const uint4*>(xrow);
#pragma unroll
        for (int q = 0; q < XPT; q++) {
            const int p = threadIdx.x + q * NW * kWave;
            if (p < pieces) xstage[q] = src[p];
        }
    }

    auto load_slice = [&](Slice<R, XREGS>& t, int sl) {
        const int c = sl * kWave + lane;
        if (sl < nslices && c < chunks_per_row) {
            const uint32_t g2 = (uint32_t)((c * CPC) >> a.gs_shift) * 2u;
            if constexpr (XMODE == 1) {
                const uint4* xp = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(xrow) + (uint32_t)c * (PAIRS * 4u));
#pragma unroll
                for (int q = 0; q < XREGS; q++) t.x[q] = xp[q];
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                t.s[r] = *reinterpret_cast<const uint16_t*>(sbase + (rel[r] * (uint32_t)groups_per_row * 2u + g2));
                t.b[r] = *reinterpret_cast<const uint16_t*>(bbase + (rel[r] * (uint32_t)groups_per_row * 2u + g2));
            }
#pragma unroll
            for (int r = 0; r < R; r++)
                t.w[r] = *reinterpret_cast<const uint4*>(wbase + (rel[r] * row_bytes + (uint32_t)c * 16u));
        }
    };

    Slice<R, XREGS> ring[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_slice(ring[d], d);

    if constexpr (XMODE == 0) {
        auto permute = [](uint4 v) {
            if constexpr (BITS == 4) {
                // (x0,x1)(x2,x3)(x4,x5)(x6,x7) -> (x0,x4)(x1,x5)(x2,x6)(x3,x7)
                uint4 o;
                o.x = (v.x & 0xffffu) | (v.z << 16);
                o.y = (v.x >> 16) | (v.z & 0xffff0000u);
                o.z = (v.y & 0xffffu) | (v.w << 16);
                o.w = (v.y >> 16) | (v.w & 0xffff0000u);
                return o;
            } else {
                return v;
            }
        };
        uint4* dst = reinterpret_cast<uint4*>(xs);
#pragma unroll
        for (int q = 0; q < XPT; q++) {
            const int p = threadIdx.x + q * NW * kWave;
            if (p < pieces) dst[p] = permute(xstage[q]);
        }
        // long activations: the rest goes through without the early issue
        const uint4* src = reinterpret_cast<const uint4*>(xrow);
        for (int p = threadIdx.x + XPT * NW * kWave; p < pieces; p += NW * kWave) dst[p] = permute(src[p]);
        __syncthreads();
    }

    float acc[R][M];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < M; m++) acc[r][m] = 0.0f;

    const uint32_t mask_s = opaque_s(kNibbleMask);   // both stay in registers so that
    const uint32_t magic_v = opaque_v(kMagic128);  // (w & mask) | magic is a single v_and_or_b32

    auto compute_slice = [&](const Slice<R, XREGS>& t, int sl) {
        const int c = sl * kWave + lane;
        if (sl < nslices && c < chunks_per_row) {
            uint32_t xq[M][PAIRS];
            float xsum[M];
#pragma unroll
            for (int m = 0; m < M; m++) {
                if constexpr (XMODE == 1) {
#pragma unroll
                    for (int q = 0; q < PAIRS / 4; q++) {
                        const uint4 v = t.x[q];
                        if constexpr (BITS == 4) {
                            xq[m][4 * q + 0] = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
                            xq[m][4 * q + 1] = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
                            xq[m][4 * q + 2] = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
                            xq[m][4 * q + 3] = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
                        } else {
                            xq[m][4 * q + 0] = v.x;
                            xq[m][4 * q + 1] = v.y;
                            xq[m][4 * q + 2] = v.z;
                            xq[m][4 * q + 3] = v.w;
                        }
                    }
                } else {
                    const uint4* xp = reinterpret_cast<const uint4*>(xs + (size_t)m * (K / 2) + (size_t)c * PAIRS);
#pragma unroll
                    for (int q = 0; q < PAIRS / 4; q++) {
                        const uint4 v = xp[q];
                        xq[m][4 * q + 0] = v.x;
                        xq[m][4 * q + 1] = v.y;
                        xq[m][4 * q + 2] = v.z;
                        xq[m][4 * q + 3] = v.w;
                    }
                }
                float sx = 0.0f;
#pragma unroll
                for (int q = 0; q < PAIRS; q++) sx = dot2_bf16(xq[m][q], 0x3F803F80u, sx);
                xsum[m] = sx;
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                const uint32_t wd[4] = {t.w[r].x, t.w[r].y, t.w[r].z, t.w[r].w};
                float d[M];
#pragma unroll
                for (int m = 0; m < M; m++) d[m] = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    if constexpr (BITS == 4) {
                        uint32_t p[4];
                        unpack4_word(wd[i], mask_s, magic_v, p);
#pragma unroll
                        for (int m = 0; m < M; m++) {
#pragma unroll
                            for (int j = 0; j < 4; j++) d[m] = dot2_bf16(p[j], xq[m][4 * i + j], d[m]);
                        }
                    } else {
                        uint32_t p[2];
                        unpack8_word(wd[i], p);
#pragma unroll
                        for (int m = 0; m < M; m++) {
                            d[m] = dot2_bf16(p[0], xq[m][2 * i + 0], d[m]);
                            d[m] = dot2_bf16(p[1], xq[m][2 * i + 1], d[m]);
                        }
                    }
                }
                const float sc = bf16_bits_to_f32(t.s[r]);
                const float bi = bf16_bits_to_f32(t.b[r]);
                const float bo = __fmaf_rn(sc, -C::kOffset, bi);  // bias with the unpack offset folded in
#pragma unroll
                for (int m = 0; m < M; m++) {
                    acc[r][m] = __fmaf_rn(sc, d[m], acc[r][m]);
                    acc[r][m] = __fmaf_rn(bo, xsum[m], acc[r][m]);
                }
            }
        }
    };

    for (int s0 = 0; s0 < nslices; s0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            compute_slice(ring[d], s0 + d);
            load_slice(ring[d], s0 + d + DEPTH);
        }
    }

#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            float tot = wave_sum(acc[r][m]);
            if (!route_ok) tot = 0.0f;
            const int row = row_first + r;
            if (lane == 0 && row < N) {
                const int64_t o = yoff + (int64_t)m * N + row;
                if (a.out_f32) {
                    reinterpret_cast<float*>(a.y)[o] = tot;
                } else {
                    reinterpret_cast<uint16_t*>(a.y)[o] = f32_to_bf16_bits(tot);
                }
            }
        }
    }
}

template <int BITS, int M, int R, int NW, int DEPTH, bool GATHER, int XMODE>
__global__ __launch_bounds__(NW* kWave) void qmv_dot2_kernel(const QmvArgs a) {
    qmv_dot2_body<BITS, M, R, NW, DEPTH, GATHER, XMODE>(a, blockIdx.x);
}

// Several weight matrices against the same activations in one launch (q|k|v, gate|up): the
// workgroups of all matrices form one grid, and each looks up which matrix it belongs to.
template <int BITS, int M, int R, int NW, int DEPTH>
__global__ __launch_bounds__(NW* kWave) void qmv_dot2_multi_kernel(const QmvMultiArgs ma) {
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
    qmv_dot2_body<BITS, M, R, NW, DEPTH, false, 0>(a, (int)blockIdx.x - (set ? ma.block_end[set - 1] : 0));
}

// ---- variant table --------------------------------------------------------

typedef void (*QmvKernel)(const QmvArgs);

struct QmvEntry {
    QmvVariant v;
    QmvKernel fn;
};

#define AQ_QMV_X(BITS, M, R, NW, DEPTH, G, X)                                                           \
    {                                                                                                   \
        {"qmv_b" #BITS "_m" #M "_r" #R "_w" #NW "_d" #DEPTH "_g" #G "_x" #X, BITS, M, R, NW, DEPTH, G, X}, \
            qmv_dot2_kernel<BITS, M, R, NW, DEPTH, (G != 0), X>                                         \
    }
#define AQ_QMV(BITS, M, R, NW, DEPTH, G) AQ_QMV_X(BITS, M, R, NW, DEPTH, G, 0)

#define AQ_QMV_M1_SET(BITS, G)                                                                     \
    AQ_QMV(BITS, 1, 1, 4, 2, G), AQ_QMV(BITS, 1, 1, 4, 4, G), AQ_QMV(BITS, 1, 1, 8, 2, G),         \
        AQ_QMV(BITS, 1, 2, 2, 2, G), AQ_QMV(BITS, 1, 2, 4, 2, G), AQ_QMV(BITS, 1, 2, 4, 4, G),     \
        AQ_QMV(BITS, 1, 2, 8, 2, G), AQ_QMV(BITS, 1, 4, 2, 2, G), AQ_QMV(BITS, 1, 4, 4, 2, G),     \
        AQ_QMV(BITS, 1, 4, 4, 4, G), AQ_QMV(BITS, 1, 4, 8, 2, G), AQ_QMV(BITS, 1, 8, 2, 2, G),     \
        AQ_QMV(BITS, 1, 8, 4, 2, G), AQ_QMV(BITS, 1, 7, 4, 2, G), AQ_QMV(BITS, 1, 7, 8, 2, G),       \
        AQ_QMV_X(BITS, 1, 1, 4, 2, G, 1), AQ_QMV_X(BITS, 1, 2, 4, 2, G, 1), AQ_QMV_X(BITS, 1, 4, 4, 2, G, 1), \
        AQ_QMV_X(BITS, 1, 2, 8, 2, G, 1), AQ_QMV_X(BITS, 1, 4, 8, 2, G, 1), AQ_QMV_X(BITS, 1, 4, 2, 2, G, 1), \
        AQ_QMV_X(BITS, 1, 2, 4, 4, G, 1), AQ_QMV_X(BITS, 1, 8, 4, 2, G, 1), AQ_QMV_X(BITS, 1, 4, 1, 2, G, 1), \
        AQ_QMV_X(BITS, 1, 2, 1, 2, G, 1), AQ_QMV_X(BITS, 1, 8, 1, 2, G, 1), AQ_QMV_X(BITS, 1, 4, 4, 1, G, 1)

#define AQ_QMV_MN_SET(BITS, M)                                                                     \
    AQ_QMV(BITS, M, 1, 4, 2, 0), AQ_QMV(BITS, M, 2, 4, 2, 0), AQ_QMV(BITS, M, 4, 4, 2, 0),         \
        AQ_QMV(BITS, M, 2, 8, 2, 0), AQ_QMV(BITS, M, 4, 8, 2, 0)

static const QmvEntry kQmvTable[] = {
    AQ_QMV_M1_SET(4, 0), AQ_QMV_M1_SET(8, 0), AQ_QMV_M1_SET(4, 1), AQ_QMV_M1_SET(8, 1),
    AQ_QMV_MN_SET(4, 2), AQ_QMV_MN_SET(4, 3), AQ_QMV_MN_SET(4, 4),
    AQ_QMV_MN_SET(8, 2), AQ_QMV_MN_SET(8, 3), AQ_QMV_MN_SET(8, 4),
};

int qmv_variant_count() { return (int)(sizeof(kQmvTable) / sizeof(kQmvTable[0])); }

const QmvVariant* qmv_variant(int idx) {
    if (idx < 0 || idx >= qmv_variant_count()) return nullptr;
    return &kQmvTable[idx].v;
}

size_t qmv_lds_bytes(int idx, const QmvArgs& a) {
    const QmvVariant* v = qmv_variant(idx);
    if (!v || v->xmode == 1) return 0;
    return (size_t)v->m * (size_t)a.K * 2;
}

hipError_t qmv_launch(int idx, const QmvArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmv_variant_count()) return hipErrorInvalidValue;
    const QmvEntry& e = kQmvTable[idx];
    const int rows_per_wg = e.v.rows * e.v.waves;
    dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), e.v.gather ? (unsigned)a.routes : 1u, 1u);
    dim3 block((unsigned)(e.v.waves * kWave), 1u, 1u);
    const size_t lds = qmv_lds_bytes(idx, a);
    if (lds > 48 * 1024) {
        hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(e.fn),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (rc != hipSuccess) return rc;
    }
    hipLaunchKernelGGL(e.fn, grid, block, lds, stream, a);
    return hipGetLastError();
}

typedef void (*QmvMultiKernel)(const QmvMultiArgs);
struct QmvMultiEntry {
    int bits, m, rows;
    QmvMultiKernel fn;
};
#define AQ_QMV_MULTI(BITS, M, R) {BITS, M, R, qmv_dot2_multi_kernel<BITS, M, R, 4, 2>}
static const QmvMultiEntry kQmvMultiTable[] = {
    AQ_QMV_MULTI(4, 1, 1), AQ_QMV_MULTI(4, 1, 2), AQ_QMV_MULTI(4, 1, 4), AQ_QMV_MULTI(8, 1, 1), AQ_QMV_MULTI(8, 1, 2),
    AQ_QMV_MULTI(8, 1, 4), AQ_QMV_MULTI(4, 2, 2), AQ_QMV_MULTI(4, 3, 2), AQ_QMV_MULTI(4, 4, 2), AQ_QMV_MULTI(8, 2, 2),
    AQ_QMV_MULTI(8, 3, 2), AQ_QMV_MULTI(8, 4, 2),
};

bool qmv_multi_supported(int bits, int m, int rows) {
    for (const QmvMultiEntry& e : kQmvMultiTable)
        if (e.bits == bits && e.m == m && e.rows == rows) return true;
    return false;
}

hipError_t qmv_multi_launch(int bits, int m, int rows, QmvMultiArgs ma, hipStream_t stream) {
    const QmvMultiEntry* e = nullptr;
    for (const QmvMultiEntry& c : kQmvMultiTable)
        if (c.bits == bits && c.m == m && c.rows == rows) e = &c;
    if (!e || ma.count < 1 || ma.count > kQmvMultiMax) return hipErrorInvalidValue;
    const int rows_per_wg = rows * 4;
    int blocks = 0;
    for (int i = 0; i < ma.count; i++) {
        blocks += (ma.N[i] + rows_per_wg - 1) / rows_per_wg;
        ma.block_end[i] = blocks;
    }
    const size_t lds = (size_t)m * (size_t)ma.common.K * 2;
    if (lds > 48 * 1024) {
        hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(e->fn),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (rc != hipSuccess) return rc;
    }
    hipLaunchKernelGGL(e->fn, dim3((unsigned)blocks), dim3(4 * kWave), lds, stream, ma);
    return hipGetLastError();
}

}  // namespace aq
