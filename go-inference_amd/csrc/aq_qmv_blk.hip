// affine_qmv / gather_qmv for gfx950, M = 1..16 activation rows: the block-MFMA kernel.
//
// Same contract as the dot2 kernel (aq_qmv.hip): replaces rocm_mlx_q4_projection*
// (go/engine/hip/kernels/quant/affine_projection.hipinc:3-266) and rocm_moe_mlx_affine_routes
// (go/engine/hip/kernels/moe/routing.hipinc:160-399), semantics of MLX affine_qmv /
// affine_gather_qmv (go/engine/metal/qmv.go:354-421).
//
// The dot2 kernel spends four VALU issue slots per wavefront instruction and is bound by them, not
// by HBM.  Here the multiply-adds move to the matrix pipe without any data shuffling:
//   * v_mfma_f32_4x4x4_16b_bf16 computes 16 independent 4x4x4 products, one per group of four
//     consecutive lanes.  Lane (blk, j) supplies as B column its OWN four codes (row j of the
//     current row group, 16-byte piece blk of the wavefront's K range) and as A row the
//     activations of token j at that piece; D[i][j] = token i . row j lands in lane (blk, j),
//     register i.  So up to four tokens cost the same as one, and no lane ever needs another
//     lane's weights;
//   * a wavefront load covers 4 rows x 256 bytes; the NW wavefronts of a workgroup split K among
//     them (KI pieces each) and keep their activations in registers for the whole kernel;
//   * workgroups are persistent: each walks row groups wg, wg + gridDim.x, ... with DEPTH row
//     groups of loads in flight per wavefront.  DEPTH is small on purpose: with every load of the
//     kernel issued up front, the memory system is one long queue, a workgroup that starts last gets
//     its first bytes last, and no arithmetic overlaps the stream;
//   * scales and biases never travel as 2-byte loads (sub-dword loads are slow in the address unit):
//     per batch of row groups a wavefront fetches the scales and biases of its own K range with one
//     or two 8-byte loads per lane and leaves them in its private part of LDS as fp32
//     (scale, bias - off*scale) pairs; every lane then picks its pair with one LDS read per row group;
//   * per lane and row group: acc += scale * D + (bias - off*scale) * sum(x) (the reference's own
//     factorisation, affine_dot.hipinc:546-573); then two DPP rotations and two permlane swaps
//     fold the 16 blocks, and the NW partial sums meet in LDS once per batch of row groups.
#include "aq_device.h"
#include "aq_kernels.h"

namespace aq {

typedef __attribute__((ext_vector_type(4))) short s16x4_t;

namespace {

__device__ __forceinline__ s16x4_t pack_pairs(uint32_t lo, uint32_t hi) {
    const uint2 v = make_uint2(lo, hi);
    return __builtin_bit_cast(s16x4_t, v);
}

// Pins a wave-uniform address into SGPRs, so that loads take the "SGPR base + 32-bit lane offset" form
// and the per-lane part needs no 64-bit VALU arithmetic.
typedef const __attribute__((address_space(1))) char* gptr_t;
__device__ __forceinline__ gptr_t uniform_ptr(const char* p) {
    const uint64_t u = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return reinterpret_cast<gptr_t>(((uint64_t)hi << 32) | lo);
}
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 load_u128_at(gptr_t base, uint32_t lane_off) {
    const u32x4_t v = *reinterpret_cast<const __attribute__((address_space(1))) u32x4_t*>(base + lane_off);
    return make_uint4(v[0], v[1], v[2], v[3]);
}

}  // namespace

template <int BITS, int MCAP, int KI, int DEPTH, bool GATHER>
__global__ __launch_bounds__(512) void qmv_blk_kernel(const QmvArgs a, const BlkGeom g) {
    constexpr int CPC = BITS == 4 ? 32 : 16;  // codes in a 16-byte piece
    constexpr int MT = (MCAP + 3) / 4;        // token tiles of four
    constexpr int U = DEPTH > 4 ? DEPTH : 4;  // row groups per round: a multiple of 4 and of the ring depth
    constexpr int AOPS = BITS == 4 ? 8 : 4;   // MFMA A operands per (piece, token tile)
    constexpr float OFFSET = BITS == 4 ? kNibbleOffset : 0.0f;
    static_assert(KI == 1 || KI == 2 || KI == 4, "pieces per wavefront");
    constexpr int SP = 2;            // staging passes per batch
    extern __shared__ float part[];  // [batch][MCAP][NW][4] partial sums, then the staged scale pairs, then a counter

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int nw = blockDim.x / kWave;
    const int j = lane & 3;
    const int blk = lane >> 2;

    const int K = a.K;
    const int N = a.N;
    const int M = a.M;
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
        wbase += row0 * g.row_bytes;
        sbase += row0 * g.sb_row_bytes;
        bbase += row0 * g.sb_row_bytes;
        xrow += (int64_t)xr * K;
        yoff = (int64_t)z * N;
    }

    const uint32_t piece0 = (uint32_t)wave * 16u + (uint32_t)blk;  // 16-byte piece of the row, K piece 0
    const uint32_t woff = (uint32_t)j * g.row_bytes + piece0 * 16u;
    // staged (scale, bias - off*scale) fp32 pairs, private to the wavefront:
    //   [stage_bufs][NW][batch][4 rows][KI][gpw groups of one K piece]
    const int gpw = g.gpw;
    const uint32_t wave_pairs = (uint32_t)g.batch * 4u * KI * gpw;
    float2* const pairs = reinterpret_cast<float2*>(part + (size_t)g.batch * MCAP * nw * 4) + (size_t)wave * wave_pairs;
    const uint32_t buf_pairs = (uint32_t)nw * wave_pairs;
    int* const arrivals = reinterpret_cast<int*>(reinterpret_cast<float2*>(part + (size_t)g.batch * MCAP * nw * 4) +
                                                 (size_t)g.stage_bufs * buf_pairs);
    const uint32_t pair_lane = (uint32_t)j * KI * gpw + (((uint32_t)blk * CPC) >> a.gs_shift);

    const int nwg = gridDim.x;
    const int wg = blockIdx.x;
    const int L = (g.total_rg - wg + nwg - 1) / nwg;  // row groups of this workgroup

    // Staging of batch b: a lane owns 4 consecutive groups (8 bytes of scales, 8 of biases) of one
    // (row group, row, K piece); 64 lanes cover g.rpp row groups, a batch takes at most SP passes.
    // Lanes past the end redo the last row group (same data to the same LDS words).
    uint2 st_s[SP], st_b[SP];
    const int st_h = lane & ((1 << g.hh_shift) - 1);
    const int st_i = (lane >> g.hh_shift) & (KI - 1);
    const int st_j = (lane >> (g.hh_shift + (KI == 1 ? 0 : KI == 2 ? 1 : 2))) & 3;
    const int st_q = lane >> (g.hh_shift + (KI == 1 ? 0 : KI == 2 ? 1 : 2) + 2);
    const uint32_t st_src = (uint32_t)st_j * g.sb_row_bytes + (((uint32_t)wave + (uint32_t)st_i * nw) * gpw + st_h * 4u) * 2u;
    const uint32_t st_dst = ((uint32_t)st_j * KI + st_i) * gpw + st_h * 4u;
    auto stage_tl = [&](int b, int sp) {
        const int first = b * g.batch;
        const int cntb = (L - first) < g.batch ? (L - first) : g.batch;
        const int tl = sp * g.rpp + st_q;
        return tl < cntb ? tl : cntb - 1;
    };
    auto stage_load = [&](int b) {
#pragma unroll
        for (int sp = 0; sp < SP; sp++) {
            const int rg = wg + (b * g.batch + stage_tl(b, sp)) * nwg;
            const size_t off = (size_t)rg * 4 * g.sb_row_bytes + st_src;
            st_s[sp] = *reinterpret_cast<const uint2*>(sbase + off);
            st_b[sp] = *reinterpret_cast<const uint2*>(bbase + off);
        }
    };
    auto stage_store = [&](int b) {
        float2* dst = pairs + (size_t)(b & (g.stage_bufs - 1)) * buf_pairs;
#pragma unroll
        for (int sp = 0; sp < SP; sp++) {
            const uint32_t sv[2] = {st_s[sp].x, st_s[sp].y};
            const uint32_t bv[2] = {st_b[sp].x, st_b[sp].y};
            float4* q = reinterpret_cast<float4*>(dst + (size_t)stage_tl(b, sp) * 4 * KI * gpw + st_dst);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const float s0 = __uint_as_float(sv[h] << 16), s1 = __uint_as_float(sv[h] & 0xffff0000u);
                const float b0 = __uint_as_float(bv[h] << 16), b1 = __uint_as_float(bv[h] & 0xffff0000u);
                // the unpack offset folded into the bias, as one fused multiply-add
                q[h] = make_float4(s0, __fmaf_rn(s0, -OFFSET, b0), s1, __fmaf_rn(s1, -OFFSET, b1));
            }
        }
    };
    stage_load(0);

    // activations next: they come from L2 and must not queue behind the weight stream
    uint4 xraw[KI][MT][AOPS / 2];
#pragma unroll
    for (int i = 0; i < KI; i++) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            int token = 4 * mt + j;
            token = token < M ? token : M - 1;
            const uint4* src = reinterpret_cast<const uint4*>(
                reinterpret_cast<const char*>(xrow) + ((size_t)token * K + (size_t)(piece0 + (uint32_t)i * nw * 16u) * CPC) * 2u);
#pragma unroll
            for (int q = 0; q < AOPS / 2; q++) xraw[i][mt][q] = src[q];
        }
    }

    struct Slot {
        uint4 w[KI];
    };
    // wo: the lane offset, handed in as a value defined in the calling basic block.  A 32-bit offset
    // that was widened in another block would cost a 64-bit VALU add per load instead of the
    // "SGPR base + 32-bit lane offset" addressing form.
    auto load_slot = [&](Slot& t, int it, uint32_t wo) {
        // past the end of the list: re-read its last row group (distinct per workgroup, so no address
        // becomes a hot spot)
        const int rg = wg + (it < L ? it : L - 1) * nwg;
        const char* wp = wbase + (int64_t)rg * (4 * (int64_t)g.row_bytes);
#pragma unroll
        for (int i = 0; i < KI; i++) t.w[i] = load_u128_at(uniform_ptr(wp + (size_t)i * g.wstep), wo);
    };

    Slot ring[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_slot(ring[d], d, woff);

    // A operands and per-token piece sums
    s16x4_t xa[KI][MT][AOPS];
    float xsum[KI][MT * 4];
#pragma unroll
    for (int i = 0; i < KI; i++) {
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            float own = 0.0f;
#pragma unroll
            for (int q = 0; q < AOPS / 2; q++) {
                const uint4 v = xraw[i][mt][q];
                own = dot2_bf16(v.x, 0x3F803F80u, own);
                own = dot2_bf16(v.y, 0x3F803F80u, own);
                own = dot2_bf16(v.z, 0x3F803F80u, own);
                own = dot2_bf16(v.w, 0x3F803F80u, own);
                if constexpr (BITS == 4) {
                    // codes of a word unpack as (c0,c4)(c1,c5)(c2,c6)(c3,c7)
                    xa[i][mt][2 * q + 0] = pack_pairs(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u),
                                                      __builtin_amdgcn_perm(v.z, v.x, 0x07060302u));
                    xa[i][mt][2 * q + 1] = pack_pairs(__builtin_amdgcn_perm(v.w, v.y, 0x05040100u),
                                                      __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
                } else {
                    xa[i][mt][2 * q + 0] = pack_pairs(v.x, v.y);
                    xa[i][mt][2 * q + 1] = pack_pairs(v.z, v.w);
                }
            }
            // token r of the tile sits in lane (blk, r): broadcast inside the quad
            const int o = __builtin_bit_cast(int, own);
            xsum[i][mt * 4 + 0] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, o, 0x00, 0xF, 0xF, true));
            xsum[i][mt * 4 + 1] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, o, 0x55, 0xF, 0xF, true));
            xsum[i][mt * 4 + 2] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, o, 0xAA, 0xF, 0xF, true));
            xsum[i][mt * 4 + 3] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, o, 0xFF, 0xF, 0xF, true));
        }
    }

    const uint32_t mask_s = opaque_s(kNibbleMask);
    const uint32_t magic_v = opaque_v(kMagic128);

    // everything is in flight: a cheap moment for the one barrier the arrival counter needs
    if (threadIdx.x == 0) *arrivals = 0;
    __syncthreads();
    stage_store(0);
    const int nb = (L + g.batch - 1) / g.batch;  // batches of this workgroup
    int bi = 0;
    if (nb > 1) stage_load(1);
    const float2* pairs_cur = pairs;

    // sums of one row group into acc[]: per lane, this lane's piece(s) of row j for every token
    auto compute_slot = [&](const Slot& t, int tl, float (&acc)[MCAP]) {
#pragma unroll
        for (int q = 0; q < MCAP; q++) acc[q] = 0.0f;
#pragma unroll
        for (int i = 0; i < KI; i++) {
            // two accumulation chains per token tile so that consecutive MFMAs are independent
            f32x4_t d0[MT], d1[MT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                d0[mt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                d1[mt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            }
            const uint32_t wd[4] = {t.w[i].x, t.w[i].y, t.w[i].z, t.w[i].w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                if constexpr (BITS == 4) {
                    uint32_t p[4];
                    unpack4_word(wd[k], mask_s, magic_v, p);
                    const s16x4_t b0 = pack_pairs(p[0], p[1]);
                    const s16x4_t b1 = pack_pairs(p[2], p[3]);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        d0[mt] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xa[i][mt][2 * k + 0], b0, d0[mt], 0, 0, 0);
                        d1[mt] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xa[i][mt][2 * k + 1], b1, d1[mt], 0, 0, 0);
                    }
                } else {
                    uint32_t p[2];
                    unpack8_word(wd[k], p);
                    const s16x4_t b0 = pack_pairs(p[0], p[1]);
#pragma unroll
                    for (int mt = 0; mt < MT; mt++) {
                        if (k & 1)
                            d1[mt] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xa[i][mt][k], b0, d1[mt], 0, 0, 0);
                        else
                            d0[mt] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(xa[i][mt][k], b0, d0[mt], 0, 0, 0);
                    }
                }
            }
            const float2 sb = pairs_cur[(uint32_t)tl * 4u * KI * gpw + pair_lane + (uint32_t)i * gpw];
            const float sc = sb.x;
            const float bo = sb.y;
#pragma unroll
            for (int q = 0; q < MCAP; q++) {
                const float d = d0[q / 4][q % 4] + d1[q / 4][q % 4];
                acc[q] = __fmaf_rn(sc, d, acc[q]);
                acc[q] = __fmaf_rn(bo, xsum[i][q], acc[q]);
            }
        }
    };

    // Cross-lane part for NS row groups at once.  Lanes of one class j = lane & 3 are summed over the
    // 16 blocks: two DPP rotations inside each row of 16 lanes, then the two permlane swaps, which
    // exchange rows between two registers and so fold two row groups per swap + add.  With NS = 4 the
    // total of row group tl + r ends up in DPP row r (lanes 16r .. 16r+15, every lane of a class the
    // same value); all 16 lanes of a row store it to the same LDS word, which needs no branch.
    auto rot_sum = [](float v) {
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, true));  // row_ror:8
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, true));  // row_ror:4
        return v;
    };
    auto swap16_sum = [](float x, float y) {  // rows [x0+x1, y0+y1, x2+x3, y2+y3]
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    };
    auto swap32_sum = [](float x, float y) {  // rows [x0+x2, x1+x3, y0+y2, y1+y3]
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
        return __uint_as_float(r[0]) + __uint_as_float(r[1]);
    };
    const int row16 = lane >> 4;
    auto reduce4 = [&](float (&a0)[MCAP], float (&a1)[MCAP], float (&a2)[MCAP], float (&a3)[MCAP], int tl) {
#pragma unroll
        for (int q = 0; q < MCAP; q++) {
            const float ab = swap16_sum(rot_sum(a0[q]), rot_sum(a1[q]));
            const float cd = swap16_sum(rot_sum(a2[q]), rot_sum(a3[q]));
            part[(((tl + row16) * MCAP + q) * nw + wave) * 4 + j] = swap32_sum(ab, cd);
        }
    };
    // one round: U row groups starting at list position t (batch-local tl), four at a time.  Every
    // slot is reloaded right after its use with the row group DEPTH further down the list (past the
    // end: a re-read of the last one, at most DEPTH wasted cache hits per wavefront).
    auto round = [&](int t, int tl) {
#pragma unroll
        for (int d0 = 0; d0 < U; d0 += 4) {
            if (t + d0 >= L) break;
            const uint32_t wo = opaque_v(woff);  // defined in this basic block, see load_slot
            float acc[4][MCAP];
#pragma unroll
            for (int n = 0; n < 4; n++) {
                compute_slot(ring[(d0 + n) % DEPTH], tl + d0 + n, acc[n]);
                load_slot(ring[(d0 + n) % DEPTH], t + d0 + n + DEPTH, wo);
                __builtin_amdgcn_sched_barrier(0);
            }
            reduce4(acc[0], acc[1], acc[2], acc[3], tl + d0);
        }
    };

    // Fold the NW K-range partials of row groups [t_first, t_first + cnt) of this workgroup's list with
    // `nthreads` threads (this one is number `tid`); 4 consecutive threads own the 4 rows of a row group.
    auto fold = [&](int t_first, int cnt, int tid, int nthreads) {
        const int nout = cnt * M * 4;
        for (int o = tid; o < nout; o += nthreads) {
            const int jj = o & 3;
            const int q = (o >> 2) % M;
            const int tl = (o >> 2) / M;
            const float* p = part + (size_t)((tl * MCAP + q) * nw) * 4 + jj;
            float tot = 0.0f;
            for (int w = 0; w < nw; w++) tot += p[w * 4];
            if (!route_ok) tot = 0.0f;
            const int row = (wg + (t_first + tl) * nwg) * 4 + jj;
            const int64_t oi = yoff + (int64_t)q * N + row;
            if (a.out_f32) {
                reinterpret_cast<float*>(a.y)[oi] = tot;
            } else {
                reinterpret_cast<uint16_t*>(a.y)[oi] = f32_to_bf16_bits(tot);
            }
        }
    };

    // Rounds of U row groups; the partial sums and the staged scales turn over once per batch.
    int tl0 = 0;  // t modulo the batch
    for (int t = 0; t < L; t += U) {
        round(t, tl0);
        tl0 += U;
        if (tl0 == g.batch && t + U < L) {
            // a batch is complete and another follows: publish its scales (other buffer) together
            // with the partial sums, fold, then start fetching the scales of the batch after it
            stage_store(bi + 1);
            __syncthreads();
            fold(t + U - g.batch, g.batch, threadIdx.x, blockDim.x);
            __syncthreads();
            tl0 = 0;
            bi++;
            pairs_cur = pairs + (size_t)(bi & (g.stage_bufs - 1)) * buf_pairs;
            if (bi + 1 < nb) stage_load(bi + 1);
        }
    }
    // The last batch: nobody waits.  Each wavefront announces its partial sums; the one that arrives
    // last folds them alone.
    int before = 0;
    if (lane == 0) before = __hip_atomic_fetch_add(arrivals, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
    before = __builtin_amdgcn_readfirstlane(before);
    if (before == nw - 1) fold(bi * g.batch, L - bi * g.batch, lane, kWave);
}

// ---- variant table and launch plan ------------------------------------------

typedef void (*BlkKernel)(const QmvArgs, const BlkGeom);

struct BlkEntry {
    QmvVariant v;  // m = most activation rows, depth = K pieces per wavefront, waves = ring depth, kind = 2
    BlkKernel fn;
};

#define AQ_BLK(BITS, MCAP, KI, D, G)                                                                \
    {                                                                                               \
        {"qmvb_b" #BITS "_m" #MCAP "_ki" #KI "_d" #D "_g" #G, BITS, MCAP, 4, D, KI, G, 0, 2},        \
            qmv_blk_kernel<BITS, MCAP, KI, D, (G != 0)>                                             \
    }
// v.depth = K pieces per wavefront, v.waves = ring depth (row groups in flight per wavefront)
// the ring depths the plan asks for: two row groups in flight with one or two K pieces per wavefront, one with four
#define AQ_BLK_M(BITS, MCAP, G) AQ_BLK(BITS, MCAP, 1, 2, G), AQ_BLK(BITS, MCAP, 2, 2, G), AQ_BLK(BITS, MCAP, 4, 1, G)
#define AQ_BLK_SET(BITS)                                                                            \
    AQ_BLK_M(BITS, 1, 0), AQ_BLK_M(BITS, 2, 0), AQ_BLK_M(BITS, 3, 0), AQ_BLK_M(BITS, 4, 0),         \
        AQ_BLK(BITS, 8, 1, 2, 0), AQ_BLK(BITS, 8, 2, 2, 0), AQ_BLK(BITS, 12, 1, 2, 0),              \
        AQ_BLK(BITS, 16, 1, 2, 0), AQ_BLK_M(BITS, 1, 1)

static const BlkEntry kBlkTable[] = {AQ_BLK_SET(4), AQ_BLK_SET(8)};

int qmvb_variant_count() { return (int)(sizeof(kBlkTable) / sizeof(kBlkTable[0])); }

const QmvVariant* qmvb_variant(int idx) {
    if (idx < 0 || idx >= qmvb_variant_count()) return nullptr;
    return &kBlkTable[idx].v;
}

bool qmvb_plan(const QmvArgs& a, int bits, int group_size, bool gather, int cu_count, int forced_idx, BlkPlan* out) {
    if (bits != 4 && bits != 8) return false;
    if (group_size != 32 && group_size != 64 && group_size != 128) return false;
    const int cpc = bits == 4 ? 32 : 16;
    const int wave_codes = 16 * cpc;  // codes one wavefront load covers per row
    if (a.K <= 0 || a.K % wave_codes != 0 || a.N % 4 != 0 || a.M < 1 || a.M > 16) return false;
    if (gather && a.M != 1) return false;
    const uintptr_t al = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.w) |
                         reinterpret_cast<uintptr_t>(a.s) | reinterpret_cast<uintptr_t>(a.b);
    if (al & 15) return false;
    const int groups = a.K / group_size;
    const int np = a.K / wave_codes;  // K pieces per row
    const int mt = (a.M + 3) / 4;
    int idx = -1, ki = 0;
    if (forced_idx >= 0) {
        const QmvVariant* v = qmvb_variant(forced_idx);
        if (!v || v->bits != bits || (v->gather != 0) != gather || v->m < a.M) return false;
        ki = v->depth;
        if (np % ki != 0 || np / ki > 8) return false;
        idx = forced_idx;
    } else {
        for (int cand : {1, 2, 4}) {
            if (np % cand != 0 || np / cand > 8 || cand * mt > 4) continue;
            ki = cand;
            break;
        }
        if (!ki) return false;
        // smallest row capacity that fits, then about two 16-byte loads in flight per wavefront
        // (deeper rings measured slower: the arithmetic cannot start until the queue has drained)
        const int want_ring = ki == 1 ? 2 : ki == 2 ? 2 : 1;
        for (int i = 0; i < qmvb_variant_count(); i++) {
            const QmvVariant* v = qmvb_variant(i);
            if (v->bits != bits || (v->gather != 0) != gather || v->depth != ki || v->m < a.M) continue;
            if (idx < 0 || v->m < qmvb_variant(idx)->m ||
                (v->m == qmvb_variant(idx)->m && v->waves == want_ring && qmvb_variant(idx)->waves != want_ring))
                idx = i;
        }
        if (idx < 0) return false;
    }
    const int nw = np / ki;
    const int total_rg = a.N / 4;
    const int cus = cu_count > 0 ? cu_count : 256;
    int wgpc = 16 / nw;  // about 16 wavefronts per CU
    if (wgpc < 1) wgpc = 1;
    int64_t want = (int64_t)cus * wgpc;
    if (gather && a.routes > 1) want = (want + a.routes - 1) / a.routes;
    if (want < 1) want = 1;
    int nwg = (int)(want < total_rg ? want : total_rg);
    // even out the last round: same number of rounds, fewest workgroups
    const int rounds = (total_rg + nwg - 1) / nwg;
    nwg = (total_rg + rounds - 1) / rounds;
    const int mcap = qmvb_variant(idx)->m;
    const int ring = qmvb_variant(idx)->waves;
    const int round_len = ring > 4 ? ring : 4;  // row groups per round of the kernel
    const int rounds_wg = (total_rg + nwg - 1) / nwg;  // most row groups a workgroup walks
    // Scale staging: a lane takes 4 groups of one (row group, row, K piece), a batch at most 2 passes
    // of 64 lanes; a batch is a multiple of the round length.
    const int gpw = wave_codes / group_size;  // groups in a wavefront's K piece
    if (gpw < 4 || gpw % 4 != 0) return false;
    const int hh = gpw / 4;
    const int lanes_per_rg = 4 * ki * hh;
    if (lanes_per_rg > 32) return false;
    const int rpp = 64 / lanes_per_rg;
    int batch = 2 * rpp < 16 ? 2 * rpp : 16;
    batch -= batch % round_len;
    int stage_bufs = 1;
    size_t lds = 0;
    for (;; batch -= round_len) {
        if (batch < round_len) return false;
        stage_bufs = rounds_wg > batch ? 2 : 1;
        lds = (size_t)batch * mcap * nw * 16 + (size_t)stage_bufs * nw * batch * 4 * ki * gpw * 8 + 16;
        if (lds <= 64 * 1024) break;
    }
    out->idx = idx;
    out->nw = nw;
    out->nwg = nwg;
    out->geom.row_bytes = (uint32_t)((int64_t)a.K * bits / 8);
    out->geom.sb_row_bytes = (uint32_t)groups * 2u;
    out->geom.wstep = (uint32_t)nw * 256u;
    out->geom.gpw = gpw;
    out->geom.hh_shift = hh == 1 ? 0 : hh == 2 ? 1 : 2;
    out->geom.rpp = rpp;
    out->geom.stage_bufs = stage_bufs;
    out->geom.total_rg = total_rg;
    out->geom.batch = batch;
    out->lds = lds;
    return true;
}

hipError_t qmvb_launch(const BlkPlan& p, const QmvArgs& a, hipStream_t stream) {
    if (p.idx < 0 || p.idx >= qmvb_variant_count()) return hipErrorInvalidValue;
    const BlkEntry& e = kBlkTable[p.idx];
    dim3 grid((unsigned)p.nwg, e.v.gather ? (unsigned)a.routes : 1u, 1u);
    dim3 block((unsigned)(p.nw * kWave), 1u, 1u);
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e.fn), (size_t)p.lds)) return rc;
    hipLaunchKernelGGL(e.fn, grid, block, p.lds, stream, a, p.geom);
    return hipGetLastError();
}

}  // namespace aq
