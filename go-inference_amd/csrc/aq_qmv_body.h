// The dot2 matvec body shared by the plain, multi-matrix and activation-fused kernels (M = 1..4 rows).
#pragma once
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
template <int R>
struct Slice {
    uint4 w[R];
    uint16_t s[R];
    uint16_t b[R];
};

// x is staged once per workgroup into LDS (its loads are issued before any weight load so the barrier never waits
// for HBM).
// bx: this workgroup's position among those of one weight matrix (blockIdx.x for a plain launch).
// FUSE 0: y = W x.
// FUSE 1: a wavefront owns R rows of the `gate` matrix (w, s, b) and the same R rows of the `up` matrix
//         (w2, s2, b2) and stores act(gate . x) * (up . x), the epilogue of rocm_mlx_q4_gelu_tanh_multiply
//         (go/engine/hip/kernels/quant/affine_gelu_tanh.hipinc:3-182; gathered: kernels/moe/routing.hipinc:312).
// FUSE 2: the activations are bf16(act(x) * x2), formed while x is staged, as lthn_gather_qmv_gelu does
//         (go/engine/metal/kernels/moe/lthn_gather_qmv.metal:98-132, lthn_gelu_qmv_impl.h:24-33).
// FUSE 3: nothing but each wavefront's best packed (score, row) leaves the kernel; their maximum is what
//         rocm_mlx_q4_projection_greedy accumulates with atomicMax
//         (kernels/quant/affine_projection_fused.hipinc:190-248).
// FUSE 4: every row's packed (score, row) is stored, as rocm_mlx_q4_projection_scores does (:411-446).
template <int BITS, int M, int R, int NW, int DEPTH, bool GATHER, int FUSE = 0>
__device__ __forceinline__ void qmv_dot2_body(const QmvArgs& a, const int bx) {
    using C = Codec<BITS>;
    constexpr int CPC = C::kCodesPerChunk;
    constexpr int PAIRS = C::kPairs;
    constexpr int RS = FUSE == 1 ? 2 * R : R;  // row slots a wavefront streams
    extern __shared__ uint32_t xs[];  // [M][K/2] bf16 pairs, unpack order

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
    const char* wbase2 = reinterpret_cast<const char*>(a.w2);
    const char* sbase2 = reinterpret_cast<const char*>(a.s2);
    const char* bbase2 = reinterpret_cast<const char*>(a.b2);
    const uint16_t* xrow = a.x;
    const uint16_t* xrow2 = a.x2;
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
        if constexpr (FUSE == 1) {
            const int64_t row2 = route_ok ? ((int64_t)e * a.expert_rows + a.row_base2) : 0;
            wbase2 += row2 * row_bytes;
            sbase2 += row2 * groups_per_row * 2;
            bbase2 += row2 * groups_per_row * 2;
        }
        if constexpr (FUSE == 2) xrow2 += (int64_t)xr * K;
    }

    // wave-uniform 64-bit bases + 32-bit lane offsets: rows past N are clamped onto the last row
    const int row_first = (bx * NW + wave) * R;
    const int row_base_clamped = min(row_first, N - 1);
    wbase += (int64_t)row_base_clamped * row_bytes;
    sbase += (int64_t)row_base_clamped * groups_per_row * 2;
    bbase += (int64_t)row_base_clamped * groups_per_row * 2;
    if constexpr (FUSE == 1) {
        wbase2 += (int64_t)row_base_clamped * row_bytes;
        sbase2 += (int64_t)row_base_clamped * groups_per_row * 2;
        bbase2 += (int64_t)row_base_clamped * groups_per_row * 2;
    }
    uint32_t rel[R];
#pragma unroll
    for (int r = 0; r < R; r++) rel[r] = (uint32_t)min(r, N - 1 - row_base_clamped);

    // Stage x: global loads first, so that nothing below queues ahead of them.
    constexpr int XPT = 4;  // 16-byte x pieces held per thread between load and LDS write
    uint4 xstage[XPT];
    uint4 xstage2[FUSE == 2 ? XPT : 1];
    const int pieces = M * (K / 8);
    {
        const uint4* src = reinterpret_cast<const uint4*>(xrow);
#pragma unroll
        for (int q = 0; q < XPT; q++) {
            const int p = threadIdx.x + q * NW * kWave;
            if (p < pieces) xstage[q] = src[p];
        }
        if constexpr (FUSE == 2) {
            const uint4* src2 = reinterpret_cast<const uint4*>(xrow2);
#pragma unroll
            for (int q = 0; q < XPT; q++) {
                const int p = threadIdx.x + q * NW * kWave;
                if (p < pieces) xstage2[q] = src2[p];
            }
        }
    }

    auto load_slice = [&](Slice<RS>& t, int sl) {
        const int c = sl * kWave + lane;
        if (sl < nslices && c < chunks_per_row) {
            const uint32_t g2 = (uint32_t)((c * CPC) >> a.gs_shift) * 2u;
#pragma unroll
            for (int r = 0; r < RS; r++) {
                const bool up = FUSE == 1 && r >= R;
                const uint32_t off = rel[up ? r - R : r] * (uint32_t)groups_per_row * 2u + g2;
                t.s[r] = *reinterpret_cast<const uint16_t*>((up ? sbase2 : sbase) + off);
                t.b[r] = *reinterpret_cast<const uint16_t*>((up ? bbase2 : bbase) + off);
            }
#pragma unroll
            for (int r = 0; r < RS; r++) {
                const bool up = FUSE == 1 && r >= R;
                const char* wp = (up ? wbase2 : wbase) + (rel[up ? r - R : r] * row_bytes + (uint32_t)c * 16u);
                if constexpr (GATHER) {
                    t.w[r] = *reinterpret_cast<const uint4*>(wp);
                } else {
                    // dense: read once, 1 KiB of a row per instruction: the non-temporal hint lets the L1 give the line up
                    typedef uint32_t u32x4_nt __attribute__((ext_vector_type(4)));
                    const u32x4_nt v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_nt*>(wp));
                    t.w[r] = make_uint4(v[0], v[1], v[2], v[3]);
                }
            }
        }
    };

    Slice<RS> ring[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; d++) load_slice(ring[d], d);

    {
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
            if constexpr (FUSE == 2) {
                if (p < pieces) dst[p] = permute(act_mul_bf16x8(xstage[q], xstage2[q], a.act));
            } else {
                if (p < pieces) dst[p] = permute(xstage[q]);
            }
        }
        // long activations: the rest goes through without the early issue
        const uint4* src = reinterpret_cast<const uint4*>(xrow);
        for (int p = threadIdx.x + XPT * NW * kWave; p < pieces; p += NW * kWave) {
            if constexpr (FUSE == 2) {
                dst[p] = permute(act_mul_bf16x8(src[p], reinterpret_cast<const uint4*>(xrow2)[p], a.act));
            } else {
                dst[p] = permute(src[p]);
            }
        }
        __syncthreads();
    }

    float acc[RS][M];
#pragma unroll
    for (int r = 0; r < RS; r++)
#pragma unroll
        for (int m = 0; m < M; m++) acc[r][m] = 0.0f;

    const uint32_t mask_s = opaque_s(kNibbleMask);   // both stay in registers so that
    const uint32_t magic_v = opaque_v(kMagic128);  // (w & mask) | magic is a single v_and_or_b32

    auto compute_slice = [&](const Slice<RS>& t, int sl) {
        const int c = sl * kWave + lane;
        if (sl < nslices && c < chunks_per_row) {
            uint32_t xq[M][PAIRS];
            float xsum[M];
#pragma unroll
            for (int m = 0; m < M; m++) {
                {
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
            for (int r = 0; r < RS; r++) {
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

    if constexpr (FUSE == 3 || FUSE == 4) {
        static_assert(FUSE < 3 || (M == 1 && !GATHER), "the head epilogues take one activation row");
        unsigned long long wave_best = 0;
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float tot = wave_sum(acc[r][0]);
            const int row = row_first + r;
            unsigned long long packed = 0;
            if (row < N && isfinite(tot) && !token_suppressed((uint32_t)row, a.suppress, a.suppress_count))
                packed = pack_score_index(tot, (uint32_t)row);
            if constexpr (FUSE == 4) {
                if (lane == 0 && row < N) reinterpret_cast<unsigned long long*>(a.y)[row] = packed;
            } else {
                wave_best = packed > wave_best ? packed : wave_best;
            }
        }
        if constexpr (FUSE == 3) {
            // one private slot per wavefront: tens of thousands of wavefronts meeting on one address, be it
            // only to read it or to take a ticket, cost more than the projection itself (measured)
            if (lane == 0) a.partial[(size_t)bx * NW + wave] = wave_best;
        }
        return;
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int m = 0; m < M; m++) {
            float tot = wave_sum(acc[r][m]);
            if constexpr (FUSE == 1) tot = fmul_unfused(act_value(a.act, tot), wave_sum(acc[r + R][m]));
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

}  // namespace aq
