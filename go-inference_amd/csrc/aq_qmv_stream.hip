// affine_qmv / gather_qmv for gfx950, one activation row: the streaming dot2 kernel.
//
// Same contract and arithmetic as aq_qmv.hip (replaces rocm_mlx_q4_projection*,
// go/engine/hip/kernels/quant/affine_projection.hipinc:3-266, and rocm_moe_mlx_affine_routes,
// go/engine/hip/kernels/moe/routing.hipinc:160-399; per 16-byte chunk
// acc += scale * dot + (bias - off*scale) * sum(x), affine_dot.hipinc:546-573).
//
// The tile-per-wavefront kernel in aq_qmv.hip spends more instructions around a tile (activation
// staging, address arithmetic, reduction, bounds) than on it, and at 4 issue cycles per wavefront
// instruction that, not HBM, bounds it.  Here a wavefront is long-lived instead:
//   * wavefront `wid` of W owns rows wid, wid + W, ...; lane L owns the 16-byte chunks
//     s*64 + L (s = 0..NS-1) of every row, so its activations never change: they are read once into
//     registers, already permuted to the unpack order, together with their sums;
//   * DEPTH rows of loads stay in flight per wavefront also while it computes: the ring has DEPTH + 1
//     register sets, and the row DEPTH further on is requested before the arithmetic of the current
//     one starts.  A row costs its NS coalesced 1 KiB loads, the scale/bias load, the unpack + dot2
//     arithmetic, and a quarter of one cross-lane reduction and store: four rows are folded together
//     (the permlane swaps merge two rows per swap + add, then four DPP steps leave row r's total in
//     lanes 16r..16r+15);
//   * scales and biases of a row travel in ONE dword load where they fit 64 lanes (lanes 0.. fetch the
//     row's scales two groups a dword, the lanes after them its biases) and reach the lanes that need
//     them through ds_bpermute_b32; 2-byte loads are slow in the address unit and cost 0.6 us of 8.9;
//   * no LDS, no barrier, no cross-wavefront traffic.
// K must be exactly NS slices of 64 chunks (NS = 1, 2, 4 or 7); other shapes use aq_qmv.hip.
#include "aq_device.h"
#include "aq_kernels.h"

namespace aq {

namespace {

typedef const __attribute__((address_space(1))) char* sgptr_t;
typedef uint32_t su32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ sgptr_t s_uniform_ptr(const char* p) {
    const uint64_t u = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return reinterpret_cast<sgptr_t>(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ uint4 s_load_u128(sgptr_t base, uint32_t off) {
    const su32x4_t v = *reinterpret_cast<const __attribute__((address_space(1))) su32x4_t*>(base + off);
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ uint32_t s_load_u16(sgptr_t base, uint32_t off) {
    return *reinterpret_cast<const __attribute__((address_space(1))) uint16_t*>(base + off);
}

}  // namespace

// SBW: the row's scales and biases (K / group dwords in all) fit one 64-lane dword load.
template <int BITS, int NS, int DEPTH, bool GATHER, bool SBW>
__global__ __launch_bounds__(256) void qmv_stream_kernel(const QmvArgs a) {
    constexpr int CPC = BITS == 4 ? 32 : 16;   // codes in a 16-byte chunk
    constexpr int PAIRS = CPC / 2;             // bf16 pairs of activations per chunk
    constexpr float OFFSET = BITS == 4 ? kNibbleOffset : 0.0f;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int K = a.K;
    const int N = a.N;
    const uint32_t row_bytes = (uint32_t)NS * 1024u;
    const uint32_t sb_row_bytes = (uint32_t)(K >> a.gs_shift) * 2u;

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
        sbase += row0 * sb_row_bytes;
        bbase += row0 * sb_row_bytes;
        xrow += (int64_t)xr * K;
        yoff = (int64_t)z * N;
    }

    const int W = gridDim.x * 4;             // wavefronts that share the rows
    const int wid = blockIdx.x * 4 + wave;
    const int L = wid < N ? (N - wid + W - 1) / W : 0;  // rows of this wavefront
    if (L == 0) return;

    // this lane's activations, once: global loads first, the weight ring right behind them
    uint4 xraw[NS][PAIRS / 4];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const uint4* src = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(xrow) + ((size_t)s * 64 + lane) * (PAIRS * 4));
#pragma unroll
        for (int q = 0; q < PAIRS / 4; q++) xraw[s][q] = src[q];
    }

    const uint32_t woff = (uint32_t)lane * 16u;
    const uint32_t goff = (((uint32_t)lane * CPC) >> a.gs_shift) * 2u;  // group of chunk `lane`, slice 0
    const uint32_t gstep = ((64u * CPC) >> a.gs_shift) * 2u;            // bytes of scales per slice

    // SBW: lane l < dw fetches scale dword l of the row, lane dw + l bias dword l (dw = groups / 2);
    // the consumer of slice s, lane L wants group s*gps + L/lpg: dword (that >> 1), half (that & 1)
    const int lpg_shift = a.gs_shift - (BITS == 4 ? 5 : 4);  // log2(lanes per group)
    const uint32_t dw = (uint32_t)(K >> a.gs_shift) >> 1;
    // lanes past both arrays (fewer than 64 groups) re-read dword 0
    const uint32_t sb_lane_off = ((uint32_t)lane < dw ? (uint32_t)lane : (uint32_t)lane < 2u * dw ? (uint32_t)lane - dw : 0u) * 4u;
    const bool sb_is_bias = (uint32_t)lane >= dw;
    int sb_src[NS];       // byte address (lane * 4) of the scale dword for ds_bpermute; the bias dword is dw lanes on
    uint32_t sb_sel;      // v_perm selector that moves the wanted half into the high half of a word
    {
        const uint32_t gl = (uint32_t)lane >> lpg_shift;
        sb_sel = (gl & 1u) ? 0x03020c0cu : 0x01000c0cu;
#pragma unroll
        for (int s = 0; s < NS; s++) sb_src[s] = (int)(((((uint32_t)s * 64u) >> lpg_shift) + gl) >> 1) * 4;
    }

    struct Row {
        uint4 w[NS];
        uint32_t s[SBW ? 1 : NS];  // SBW: s[0] = this lane's dword of the row's scales / biases
        uint32_t b[SBW ? 1 : NS];
    };
    // the row the next load_row call fetches, as running pointers: rows advance by W; past the end of
    // the list they stay on the last row (a cache hit)
    const char* wnext = wbase + (int64_t)wid * row_bytes;
    const char* snext = sbase + (int64_t)wid * sb_row_bytes;
    const char* bnext = bbase + (int64_t)wid * sb_row_bytes;
    const int64_t wstride = (int64_t)W * row_bytes;
    const int64_t sstride = (int64_t)W * sb_row_bytes;
    int loaded = 0;
    auto load_row = [&](Row& t, uint32_t wo, uint32_t go) {
        const sgptr_t wp = s_uniform_ptr(wnext);
        if constexpr (SBW) {
            t.s[0] = *reinterpret_cast<const uint32_t*>((sb_is_bias ? bnext : snext) + go);
        } else {
            const sgptr_t sp = s_uniform_ptr(snext);
            const sgptr_t bp = s_uniform_ptr(bnext);
#pragma unroll
            for (int s = 0; s < NS; s++) {
                t.s[s] = s_load_u16(sp, go + (uint32_t)s * gstep);
                t.b[s] = s_load_u16(bp, go + (uint32_t)s * gstep);
            }
        }
#pragma unroll
        for (int s = 0; s < NS; s++) t.w[s] = s_load_u128(wp, wo + (uint32_t)s * 1024u);
        loaded++;
        const bool advance = loaded < L;
        wnext += advance ? wstride : 0;
        snext += advance ? sstride : 0;
        bnext += advance ? sstride : 0;
    };
    const uint32_t sboff = SBW ? sb_lane_off : goff;

    Row ring[DEPTH + 1];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_row(ring[d], woff, sboff);

    uint32_t xq[NS][PAIRS];
    float xsum[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        float sx = 0.0f;
#pragma unroll
        for (int q = 0; q < PAIRS / 4; q++) {
            const uint4 v = xraw[s][q];
            sx = dot2_bf16(v.x, 0x3F803F80u, sx);
            sx = dot2_bf16(v.y, 0x3F803F80u, sx);
            sx = dot2_bf16(v.z, 0x3F803F80u, sx);
            sx = dot2_bf16(v.w, 0x3F803F80u, sx);
            if constexpr (BITS == 4) {
                // codes of a word unpack as (c0,c4)(c1,c5)(c2,c6)(c3,c7)
                xq[s][4 * q + 0] = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
                xq[s][4 * q + 1] = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
                xq[s][4 * q + 2] = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
                xq[s][4 * q + 3] = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
            } else {
                xq[s][4 * q + 0] = v.x;
                xq[s][4 * q + 1] = v.y;
                xq[s][4 * q + 2] = v.z;
                xq[s][4 * q + 3] = v.w;
            }
        }
        xsum[s] = sx;
    }

    const uint32_t mask_s = opaque_s(kNibbleMask);
    const uint32_t magic_v = opaque_v(kMagic128);

    auto compute_row = [&](const Row& t) {
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const uint32_t wd[4] = {t.w[s].x, t.w[s].y, t.w[s].z, t.w[s].w};
            float d0 = 0.0f, d1 = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if constexpr (BITS == 4) {
                    uint32_t p[4];
                    unpack4_word(wd[i], mask_s, magic_v, p);
                    d0 = dot2_bf16(p[0], xq[s][4 * i + 0], d0);
                    d1 = dot2_bf16(p[1], xq[s][4 * i + 1], d1);
                    d0 = dot2_bf16(p[2], xq[s][4 * i + 2], d0);
                    d1 = dot2_bf16(p[3], xq[s][4 * i + 3], d1);
                } else {
                    uint32_t p[2];
                    unpack8_word(wd[i], p);
                    d0 = dot2_bf16(p[0], xq[s][2 * i + 0], d0);
                    d1 = dot2_bf16(p[1], xq[s][2 * i + 1], d1);
                }
            }
            float sc, bi;
            if constexpr (SBW) {
                const int sw = __builtin_amdgcn_ds_bpermute(sb_src[s], (int)t.s[0]);
                const int bw = __builtin_amdgcn_ds_bpermute(sb_src[s] + (int)dw * 4, (int)t.s[0]);
                sc = __uint_as_float(__builtin_amdgcn_perm(0u, (uint32_t)sw, sb_sel));
                bi = __uint_as_float(__builtin_amdgcn_perm(0u, (uint32_t)bw, sb_sel));
            } else {
                sc = bf16_bits_to_f32(t.s[s]);
                bi = bf16_bits_to_f32(t.b[s]);
            }
            const float bo = __fmaf_rn(sc, -OFFSET, bi);  // bias with the unpack offset folded in
            acc = __fmaf_rn(sc, d0 + d1, acc);
            acc = __fmaf_rn(bo, xsum[s], acc);
        }
        return acc;
    };

    // four rows' per-lane sums -> row r's total in every lane of DPP row r
    auto fold4 = [](float v0, float v1, float v2, float v3) {
        const auto a01 = __builtin_amdgcn_permlane16_swap(__float_as_uint(v0), __float_as_uint(v1), false, false);
        const auto a23 = __builtin_amdgcn_permlane16_swap(__float_as_uint(v2), __float_as_uint(v3), false, false);
        const float m01 = __uint_as_float(a01[0]) + __uint_as_float(a01[1]);  // rows [v0 01, v1 01, v0 23, v1 23]
        const float m23 = __uint_as_float(a23[0]) + __uint_as_float(a23[1]);
        const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(m01), __float_as_uint(m23), false, false);
        float v = __uint_as_float(b[0]) + __uint_as_float(b[1]);              // rows [v0, v1, v2, v3]
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
        return v;
    };

    // Rounds of U rows, U a multiple of 4 and of the ring size DEPTH + 1: row t lives in register set
    // t % (DEPTH + 1); the set freed by row t - 1 is reloaded with row t + DEPTH before row t is worked on;
    // every fourth row the four pending sums are folded and stored by lanes 0, 16, 32, 48.
    constexpr int RING = DEPTH + 1;
    constexpr int U = (RING % 4 == 0) ? RING : (RING % 2 == 0 ? 2 * RING : 4 * RING);
    const int64_t ystride = (int64_t)W;
    for (int t0 = 0; t0 < L; t0 += U) {
        const uint32_t wo = opaque_v(woff);   // lane offsets defined in this basic block: the loads keep
        const uint32_t go = opaque_v(sboff);  // the SGPR-base + 32-bit-offset form
        float pend[4];
#pragma unroll
        for (int d = 0; d < U; d++) {
            load_row(ring[(d + DEPTH) % RING], wo, go);
            __builtin_amdgcn_sched_barrier(0);
            pend[d & 3] = compute_row(ring[d % RING]);
            if ((d & 3) == 3) {
                float tot = fold4(pend[0], pend[1], pend[2], pend[3]);
                if (!route_ok) tot = 0.0f;
                const int t = t0 + d - 3 + (lane >> 4);  // the row of this lane's DPP row
                if ((lane & 15) == 0 && t < L) {
                    const int64_t o = yoff + wid + (int64_t)t * ystride;
                    if (a.out_f32) {
                        reinterpret_cast<float*>(a.y)[o] = tot;
                    } else {
                        reinterpret_cast<uint16_t*>(a.y)[o] = f32_to_bf16_bits(tot);
                    }
                }
                if (t0 + d + 1 >= L) break;  // nothing but re-read rows from here on
            }
        }
    }
}

// ---- variant table and launch plan ------------------------------------------------------------

typedef void (*StreamKernel)(const QmvArgs);
struct StreamEntry {
    QmvVariant v;  // rows = 1, waves = 4, depth = ring depth, xmode = slices per row, kind = 3
    StreamKernel fn;      // scales and biases as 2-byte loads per slice
    StreamKernel fn_sbw;  // ... as one dword load per row
};
#define AQ_STREAM(BITS, NS, D, G)                                                             \
    {{"qmvs_b" #BITS "_ns" #NS "_d" #D "_g" #G, BITS, 1, 1, 4, D, G, NS, 3},                  \
     qmv_stream_kernel<BITS, NS, D, (G != 0), false>, qmv_stream_kernel<BITS, NS, D, (G != 0), true>}
#define AQ_STREAM_SET(BITS, G)                                                                  \
    AQ_STREAM(BITS, 1, 1, G), AQ_STREAM(BITS, 1, 3, G), AQ_STREAM(BITS, 2, 3, G), \
        AQ_STREAM(BITS, 2, 1, G), AQ_STREAM(BITS, 4, 1, G), AQ_STREAM(BITS, 4, 3, G), AQ_STREAM(BITS, 7, 1, G)
static const StreamEntry kStreamTable[] = {AQ_STREAM_SET(4, 0), AQ_STREAM_SET(8, 0), AQ_STREAM_SET(4, 1), AQ_STREAM_SET(8, 1)};

int qmvs_variant_count() { return (int)(sizeof(kStreamTable) / sizeof(kStreamTable[0])); }
const QmvVariant* qmvs_variant(int idx) {
    if (idx < 0 || idx >= qmvs_variant_count()) return nullptr;
    return &kStreamTable[idx].v;
}

bool qmvs_plan(const QmvArgs& a, int bits, int group_size, bool gather, int cu_count, int forced_idx, StreamPlan* out) {
    if (bits != 4 && bits != 8) return false;
    if (group_size != 32 && group_size != 64 && group_size != 128) return false;
    if (a.M != 1 || a.K <= 0 || a.N <= 0) return false;
    const int slice_codes = 64 * (bits == 4 ? 32 : 16);
    if (a.K % slice_codes != 0) return false;
    const int ns = a.K / slice_codes;
    if ((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.w)) & 15) return false;
    int idx = -1;
    if (forced_idx >= 0) {
        const QmvVariant* v = qmvs_variant(forced_idx);
        if (!v || v->bits != bits || (v->gather != 0) != gather || v->xmode != ns) return false;
        idx = forced_idx;
    } else {
        const int want_depth = ns >= 7 ? 1 : 3;
        for (int i = 0; i < qmvs_variant_count(); i++) {
            const QmvVariant* v = qmvs_variant(i);
            if (v->bits != bits || (v->gather != 0) != gather || v->xmode != ns) continue;
            if (idx < 0 || v->depth == want_depth) idx = i;
            if (v->depth == want_depth) break;
        }
        if (idx < 0) return false;
    }
    // wavefronts: 2 to 4 per SIMD, whichever leaves the rows most evenly divided
    const int cus = cu_count > 0 ? cu_count : 256;
    const int routes = gather && a.routes > 1 ? a.routes : 1;
    int best_w = 0;
    double best_cost = 0.0;
    for (int wps = 4; wps >= 2; wps--) {
        if (ns >= 7 && wps > 2) continue;  // register budget: 7 slices of activations per lane
        int64_t waves = (int64_t)cus * 4 * wps / routes;
        waves = (waves + 3) / 4 * 4;
        if (waves < 4) waves = 4;
        const int64_t cap = ((int64_t)a.N + 3) / 4 * 4;
        if (waves > cap) waves = cap;
        const int64_t per = (a.N + waves - 1) / waves;
        const double cost = (double)per * waves / a.N;  // 1.0 = perfectly even
        if (best_w == 0 || cost < best_cost - 1e-9) {
            best_w = (int)waves;
            best_cost = cost;
        }
    }
    out->idx = idx;
    out->nwg = best_w / 4;
    // one dword load for a row's scales and biases: both fit 64 lanes, rows of them stay dword-aligned,
    // and a lane's chunk lies inside one group
    const int groups = a.K / group_size;
    out->sbw = groups <= 64 && groups % 2 == 0 && group_size >= (bits == 4 ? 32 : 16) &&
               ((reinterpret_cast<uintptr_t>(a.s) | reinterpret_cast<uintptr_t>(a.b)) & 3) == 0;
    return true;
}

hipError_t qmvs_launch(const StreamPlan& p, const QmvArgs& a, hipStream_t stream) {
    if (p.idx < 0 || p.idx >= qmvs_variant_count()) return hipErrorInvalidValue;
    const StreamEntry& e = kStreamTable[p.idx];
    dim3 grid((unsigned)p.nwg, e.v.gather ? (unsigned)a.routes : 1u, 1u);
    hipLaunchKernelGGL(p.sbw ? e.fn_sbw : e.fn, grid, dim3(256), 0, stream, a);
    return hipGetLastError();
}

}  // namespace aq
