// affine_qmv for gfx950, 8-bit codes in groups of 64, 1..16 rows of x: the MFMA matvec for byte codes.
//
// Same contract as the other matvec kernels: replaces the q8 forms of rocm_mlx_q4_projection*
// (go/engine/hip/kernels/quant/affine_projection.hipinc:105-149, affine_projection_tuned.hipinc:561-1051); semantics
// of MLX affine_qmv (go/engine/metal/qmv.go:354-421) and of its M-row form (go/engine/metal/qmv_rows.go:14-60).
//
// With byte codes the layout that the memory pipeline likes and the layout of v_mfma_f32_16x16x32_bf16 coincide:
//   * lane (n = lane % 16, j = lane / 16) loads 16 bytes of weight row n: one instruction covers 64 contiguous bytes of
//     each of 16 rows, and those 64 codes are exactly one quantisation group.  The lane's 16 codes are the B operands of
//     two MFMAs (8 each; v_cvt_f32_ubyte + v_perm, exact: a code has 8 significant bits), so D = sum over the group
//     of code * x, with no separation of groups to arrange;
//   * the 16 rows of A are 16 TOKENS (activation rows): up to 16 rows of x cost what one costs.  x sits in LDS in its
//     natural order (rows padded by 16 bytes against bank conflicts); lane (t, j) reads x[t][64 g + 16 j + 8 i ..];
//   * per group: acc += scale * D, four FMAs per lane (D lands as lane (n, j), register r -> token 4 j + r, row n); the
//     scales and biases of a step of 16 groups are one 8-byte load each per lane (lane group j takes groups 4 j .. 4 j + 3),
//     passed to the lanes that need them with ds_bpermute;
//   * the affine term bias * sum(x) is MFMA work: the group sums of x are split into three bf16 terms when x is staged
//     (exact), and two MFMAs per step multiply A = (X0 X1 X2 0 | X0' X1' X2' 0) with B = (b b b 0 | b' b' b' 0), two
//     groups per lane group;
//   * NW wavefronts share K in steps of 1024 codes (one each) for the same 16 rows and meet in LDS; everything a
//     wavefront reads is requested up front.  Up to two rows of x: every wavefront stages the activations of its own
//     step and nobody waits at a barrier before the arithmetic.
// Every variant computes the same bytes for a token whatever the number of rows of x.
#include "aq_device.h"
#include "aq_kernels.h"

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
__device__ __forceinline__ uint2 load_u64_at(gptr_t base, uint32_t off) {
    const u32x2_t v = *reinterpret_cast<const __attribute__((address_space(1))) u32x2_t*>(base + off);
    return make_uint2(v[0], v[1]);
}
__device__ __forceinline__ bf16x8_t as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    const uint4 v = make_uint4(a, b, c, d);
    return __builtin_bit_cast(bf16x8_t, v);
}

constexpr int kD8Rows = 16;     // weight rows per set of wavefronts
constexpr int kD8Step = 1024;   // codes of a row per wavefront (16 groups)
constexpr int kD8MaxM = 16;
constexpr int kD8Pad = 16;      // bytes behind every row of x in LDS
constexpr int kD8WaveRows = 2;  // most rows of x a wavefront stages for itself (4 measured no faster for 3 and 4 rows, slower for 1)

}  // namespace

// LDS: x [M][K * 2 + 16], the split group sums [M][K / 128][16 bytes] (two groups each), 64 zero bytes; the partial sums
// of the wavefronts [sets x NW][4][64] fp32 take the place of x once every wavefront is done with it.
__host__ __device__ inline size_t qmvd8_lds_bytes(int M, int K, int nw) {
    const size_t xb = (size_t)M * ((size_t)K * 2 + kD8Pad) + (size_t)M * ((K + 127) / 128) * 16 + 64;
    const size_t rb = (size_t)nw * 4 * 64 * 4;
    return xb > rb ? xb : rb;
}

// NR sets of NW wavefronts: a set works on 16 weight rows, its wavefronts share K; all sets read the same staged x (more
// rows of x need more LDS, so fewer, larger workgroups keep every CU holding one).
template <int NW, int NR>
__global__ __launch_bounds__(NR* NW* kWave) void qmv_d8_kernel(const QmvArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave_wg = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = wave_wg % NW;  // which step of K
    const int rg = wave_wg / NW;    // which 16 rows of the workgroup's NR x 16
    const int n = lane & 15;
    const int j = lane >> 4;
    const int K = a.K, N = a.N, M = a.M;
    const int groups = K >> 6;
    const int pairs = (groups + 1) >> 1;           // 16-byte entries of split sums per row of x
    const uint32_t pitch = (uint32_t)K * 2u + kD8Pad;
    const uint32_t a2_off = (uint32_t)M * pitch;
    const uint32_t zero_off = a2_off + (uint32_t)M * (uint32_t)pairs * 16u;
    const int g0 = wave * 16;                      // first group of this wavefront's step
    const int gn = min(16, groups - g0);           // groups of the step that exist (<= 0: an idle wavefront)

    const gptr_t xg = uniform_ptr(a.x);
    // ---- the first pieces of x are requested before the weights, so that they arrive first ----
    const bool wstage = M <= kD8WaveRows;
    const int ppt = K >> 3;  // 16-byte pieces per row of x
    const int pieces = M * ppt;
    constexpr int PRE = 2 * kD8WaveRows;
    uint4 pre[PRE];
    int pre_p[PRE];
#pragma unroll
    for (int q = 0; q < PRE; q++) {
        if (wstage) {
            const int pl = wave * 128 + (q & 1) * 64 + lane;  // piece of row q / 2 inside this wavefront's step
            pre_p[q] = (q >> 1) < M && pl < ppt ? (q >> 1) * ppt + pl : pieces;
        } else {
            pre_p[q] = q < 2 ? tid + q * NR * NW * kWave : pieces;
            if (pre_p[q] >= pieces) pre_p[q] = pieces;
        }
        pre[q] = load_u128_at(xg, (uint32_t)min(pre_p[q], pieces - 1) * 16u);
    }
    if (lane < 4 && (wstage || wave_wg == 0)) *reinterpret_cast<uint4*>(lds_raw + zero_off + lane * 16) = make_uint4(0, 0, 0, 0);

    // ---- weights, scales, biases of the step: everything up front ----
    const int row0 = ((int)blockIdx.x * NR + rg) * kD8Rows;
    const int row = min(row0 + n, N - 1);
    const gptr_t wg = uniform_ptr(a.w), sg = uniform_ptr(a.s), bg = uniform_ptr(a.b);
    const uint32_t w_lane = (uint32_t)row * (uint32_t)K + (uint32_t)j * 16u;            // bytes (one byte per code)
    // lane group j takes the scales of groups 4 j .. 4 j + 3 of the step; past the end of the row: re-read the last ones
    const int gq = min(g0 + 4 * j, max(groups - 4, 0));
    const uint2 sv = load_u64_at(sg, (uint32_t)row * (uint32_t)groups * 2u + (uint32_t)gq * 2u);
    const uint2 bv = load_u64_at(bg, (uint32_t)row * (uint32_t)groups * 2u + (uint32_t)gq * 2u);
    uint4 wq[16];
#pragma unroll
    for (int g = 0; g < 16; g++) {
        const int gc = min(g0 + g, groups - 1);  // past the end of K: a valid address, the data is not used
        wq[g] = load_u128_at(wg, w_lane + (uint32_t)gc * 64u);
    }

    // ---- stage x: natural order, group sums split into three bf16 terms ----
    auto stage = [&](int p, const uint4 v) {
        const uint32_t t = (uint32_t)p / (uint32_t)ppt;
        const uint32_t c = (uint32_t)p - t * (uint32_t)ppt;  // piece of the row
        *reinterpret_cast<uint4*>(lds_raw + t * pitch + c * 16u) = v;
        const uint32_t ones = 0x3f803f80u;
        float sum = dot2_bf16(v.x, ones, 0.0f);
        sum = dot2_bf16(v.y, ones, sum);
        sum = dot2_bf16(v.z, ones, sum);
        sum = dot2_bf16(v.w, ones, sum);
        // the eight pieces of a group sit in eight consecutive, aligned lanes
        sum += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0xB1, 0xF, 0xF, true));
        sum += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0x4E, 0xF, 0xF, true));
        sum += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sum), 0x141, 0xF, 0xF, true));
        if ((c & 7u) == 0) {
            const uint32_t u0 = __float_as_uint(sum) & 0xffff0000u;
            const float r1 = sum - __uint_as_float(u0);
            const uint32_t u1 = __float_as_uint(r1) & 0xffff0000u;
            const float r2 = r1 - __uint_as_float(u1);
            const uint32_t u2 = __float_as_uint(r2) & 0xffff0000u;
            const uint32_t g = c >> 3;
            uint32_t* e = reinterpret_cast<uint32_t*>(lds_raw + a2_off + (t * (uint32_t)pairs + (g >> 1)) * 16u + (g & 1u) * 8u);
            e[0] = (u0 >> 16) | u1;  // (X0, X1)
            e[1] = u2 >> 16;         // (X2, 0)
            if ((groups & 1) && (int)g == groups - 1) {
                e[2] = 0;  // the missing second group of the last pair adds nothing
                e[3] = 0;
            }
        }
    };
#pragma unroll
    for (int q = 0; q < PRE; q++)
        if (pre_p[q] < pieces) stage(pre_p[q], pre[q]);
    if (wstage) {
        // LDS operations of one wavefront complete in order: what its lanes wrote is there for its later reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    } else {
        for (int p = tid + 2 * NR * NW * kWave; p < pieces; p += NR * NW * kWave) stage(p, load_u128_at(xg, (uint32_t)p * 16u));
        __syncthreads();
    }

    // ---- per-lane constants ----
    // A operand: lane (t = lane % 16, j): token t (past M: the last one, never stored), 16 bytes at 64 g + 16 j + 8 i codes
    const int at = min(n, M - 1);
    const uint32_t x_lane = (uint32_t)at * pitch + (uint32_t)j * 32u;
    const uint32_t a2_lane = a2_off + (uint32_t)at * (uint32_t)pairs * 16u;
    const int sc_addr = n * 4;

    f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
    f32x4_t dsum = {0.0f, 0.0f, 0.0f, 0.0f};
    if (gn > 0) {
        // affine term: MFMA q covers groups 4 j' + 2 q, 4 j' + 2 q + 1 of every lane group j'
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const uint32_t bw = q ? bv.y : bv.x;
            const int gp = g0 + 4 * j + 2 * q;  // first group of this lane's pair
            const bool have = gp < groups && gq == g0 + 4 * j;
            const bf16x8_t b2 = as_bf16x8(__builtin_amdgcn_perm(bw, bw, 0x01000100u), __builtin_amdgcn_perm(0u, bw, 0x0C0C0100u),
                                          __builtin_amdgcn_perm(bw, bw, 0x03020302u), __builtin_amdgcn_perm(0u, bw, 0x0C0C0302u));
            const uint32_t addr = have ? a2_lane + (uint32_t)(gp >> 1) * 16u : zero_off;
            const bf16x8_t a2 = *reinterpret_cast<const bf16x8_t*>(lds_raw + addr);
            dsum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a2, b2, dsum, 0, 0, 0);
        }
#pragma unroll
        for (int g = 0; g < 16; g++) {
            if (g >= gn) continue;  // (uniform; a `break` keeps the loop from being unrolled and the loads from staying up front)
            const uint32_t ww[4] = {wq[g].x, wq[g].y, wq[g].z, wq[g].w};
            f32x4_t d = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const bf16x8_t af = *reinterpret_cast<const bf16x8_t*>(lds_raw + x_lane + (uint32_t)(g0 + g) * 128u + (uint32_t)i * 16u);
                uint32_t p[4];
                unpack8_word(ww[2 * i], p);
                unpack8_word(ww[2 * i + 1], p + 2);
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, as_bf16x8(p[0], p[1], p[2], p[3]), d, 0, 0, 0);
            }
            // the scale of group g of the step sits in lane group g / 4, word (g % 4) / 2, half g % 2
            const uint32_t sw = (uint32_t)__builtin_amdgcn_ds_bpermute(sc_addr + (g >> 2) * 64, (int)((g & 2) ? sv.y : sv.x));
            const float sc = (g & 1) ? __uint_as_float(sw & 0xffff0000u) : __uint_as_float(sw << 16);
#pragma unroll
            for (int r = 0; r < 4; r++) acc[r] = __builtin_fmaf(sc, d[r], acc[r]);
        }
    }
#pragma unroll
    for (int r = 0; r < 4; r++) acc[r] += dsum[r];

    // ---- the wavefronts' partial sums meet in LDS; the first wavefront adds them in order and stores ----
    float* red = reinterpret_cast<float*>(lds_raw);
    __syncthreads();  // every wavefront has read what it needs of x
#pragma unroll
    for (int r = 0; r < 4; r++) red[(wave_wg * 4 + r) * 64 + lane] = acc[r];
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            float total = red[(wave_wg * 4 + r) * 64 + lane];
#pragma unroll
            for (int w2 = 1; w2 < NW; w2++) total += red[((wave_wg + w2) * 4 + r) * 64 + lane];
            const int t = 4 * j + r, rr = row0 + n;
            if (t < M && rr < N) {
                const size_t o = (size_t)t * N + rr;
                if (a.out_f32) {
                    static_cast<float*>(a.y)[o] = total;
                } else {
                    static_cast<uint16_t*>(a.y)[o] = f32_to_bf16_bits(total);
                }
            }
        }
    }
}

// ---- variant table --------------------------------------------------------

typedef void (*QmvD8Kernel)(const QmvArgs);
struct QmvD8Entry {
    QmvVariant v;  // m = most rows of x, rows = sets of 16 rows per workgroup, waves = wavefronts that share K
    QmvD8Kernel fn;
};
#define AQ_QMVD8(NW, NR)                                                                             \
    {                                                                                                \
        {"qmvd8_b8_m16_r" #NR "_w" #NW, 8, kD8MaxM, NR, NW, 1, 0, 0, 7}, qmv_d8_kernel<NW, NR>       \
    }
static const QmvD8Entry kQmvD8Table[] = {AQ_QMVD8(1, 1), AQ_QMVD8(2, 1), AQ_QMVD8(4, 1), AQ_QMVD8(8, 1), AQ_QMVD8(16, 1),
                                          AQ_QMVD8(1, 4), AQ_QMVD8(2, 4), AQ_QMVD8(4, 2), AQ_QMVD8(4, 4), AQ_QMVD8(8, 2)};

int qmvd8_variant_count() { return (int)(sizeof(kQmvD8Table) / sizeof(kQmvD8Table[0])); }
const QmvVariant* qmvd8_variant(int idx) {
    if (idx < 0 || idx >= qmvd8_variant_count()) return nullptr;
    return &kQmvD8Table[idx].v;
}

bool qmvd8_fits(const QmvArgs& a, int bits, int group_size, int idx) {
    const QmvVariant* v = qmvd8_variant(idx);
    if (!v || bits != 8 || group_size != 64) return false;
    if (a.M < 1 || a.M > v->m || a.N < 1 || a.K < 256 || a.K % 256 != 0) return false;
    if ((a.K + kD8Step - 1) / kD8Step > v->waves) return false;
    const uintptr_t al16 = reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.w);
    const uintptr_t al8 = reinterpret_cast<uintptr_t>(a.s) | reinterpret_cast<uintptr_t>(a.b);
    if ((al16 & 15) || (al8 & 7)) return false;
    if ((uint64_t)a.N * (uint64_t)a.K >= (1ull << 32)) return false;  // 32-bit byte offsets into the packed matrix
    return qmvd8_lds_bytes(a.M, a.K, v->waves * v->rows) <= 150 * 1024;
}

hipError_t qmvd8_launch(int idx, const QmvArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmvd8_variant_count()) return hipErrorInvalidValue;
    const QmvD8Entry& e = kQmvD8Table[idx];
    const size_t lds = qmvd8_lds_bytes(a.M, a.K, e.v.waves * e.v.rows);
    if (lds > 48 * 1024) {
        hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(e.fn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)lds);
        if (rc != hipSuccess) return rc;
    }
    const int wg_rows = kD8Rows * e.v.rows;
    hipLaunchKernelGGL(e.fn, dim3((unsigned)((a.N + wg_rows - 1) / wg_rows)), dim3((unsigned)(e.v.rows * e.v.waves * kWave)), lds,
                       stream, a);
    return hipGetLastError();
}

// The variant whose wavefronts cover K one step each, or -1: as many sets of 16 rows per workgroup as 16 wavefronts hold,
// up to four (with many rows the staged x takes most of a CU's LDS: one workgroup each).
int qmvd8_pick(int M, int K, int N) {
    if (M < 1 || M > kD8MaxM || K < 256 || K % 256 != 0) return -1;
    const int steps = (K + kD8Step - 1) / kD8Step;
    int nw = 1;
    while (nw < steps) nw *= 2;
    if (nw > 16) return -1;
    int want = 16 / nw;  // (four sets measured fastest for every row count at 4096 x 14336)
    if (want > 4) want = 4;
    while (want > 1 && (N + kD8Rows * want - 1) / (kD8Rows * want) < 128) want >>= 1;  // keep the grid wide
    int best = -1;
    for (int i = 0; i < qmvd8_variant_count(); i++) {
        const QmvVariant& v = kQmvD8Table[i].v;
        if (v.waves != nw || v.rows > want) continue;
        if (best < 0 || v.rows > kQmvD8Table[best].v.rows) best = i;
    }
    return best;
}

}  // namespace aq
