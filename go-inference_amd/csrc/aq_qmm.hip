// affine_qmm for gfx950: y[M,N] = x[M,K] . dequant(w[N,K])^T on the bf16 MFMA pipe.
//
// Replaces rocm_mlx_q4_projection_batch* (go/engine/hip/kernels/quant/affine_projection_tuned.hipinc:166-1109,
// selector go/engine/hip/hip_projection_launch.go:5192-5287) with the semantics of MLX affine_qmm_t
// (go/engine/metal/quant_seam_backend.go:77-109, go/engine/metal/attention.go:731-751).
//
// The matrix cores are fed the CODES, not dequantised weights: a 4-bit code c becomes the bf16
// value 16+c (8-bit: c itself), both exact, and the activations are bf16 already, so every
// product is exact and the fp32 accumulation inside the MFMA carries no weight-rounding error.
// Per 64-code block of K ("group block"):
//     P[m,n]   = sum_k x[m,k] * (off + c[n,k])                 4 x v_mfma_f32_32x32x16_bf16
//     out[m,n] += scale[n,g] * P[m,n]                           one v_fma_f32 per accumulator
// and once per four group blocks one extra MFMA adds the affine terms
//     out[m,n] += sum_g (bias[n,g] - off*scale[n,g]) * Sx[m,g], Sx[m,g] = sum_{k in g} x[m,k]
// with Sx split into two bf16 values (hi + lo) and bias, -off*scale exact in bf16.
// This is the factorisation the reference kernels use (affine_dot.hipinc:546-573), moved onto MFMA.
//
// Data movement: x tiles are staged through LDS in MFMA-fragment order (each A-operand read is
// one contiguous, conflict-free 1 KiB ds_read_b128 per wavefront), double buffered, one barrier
// per group block.  Packed weights go global -> registers directly: lane (j, h) of a wavefront
// owns weight row n0+j and loads the 16 bytes (4 bit) or 32 bytes (8 bit) that hold codes
// [32h, 32h+32) of the group block; word t of those feeds MFMA step t, so one load serves four
// MFMAs and the packed bytes are never expanded in memory.
#include "aq_device.h"
#include "aq_kernels.h"
#include "aq_qmm.h"

#include <cstring>

#include "../../include/aq_mi355.h"

namespace aq {

namespace {

constexpr uint32_t kMask16 = 0x00780078u;   // a nibble moved to mantissa bits [6:3]
constexpr uint32_t kMagic16 = 0x41804180u;  // bf16 16.0 in both halves: 16 + code, exact

template <int BITS>
struct MmaCodec;
template <>
struct MmaCodec<4> {
    static constexpr int kWordsPerLane = 4;  // 32 codes
    static constexpr float kOffset = 16.0f;
};
template <>
struct MmaCodec<8> {
    static constexpr int kWordsPerLane = 8;
    static constexpr float kOffset = 0.0f;
};

// 8 codes -> bf16x8 in k-slot order.  4 bit: slots (c0,c4)(c1,c5)(c2,c6)(c3,c7); 8 bit: natural.
__device__ __forceinline__ bf16x8_t unpack_frag4(uint32_t w, uint32_t mask_s, uint32_t magic_v) {
    uint32_t p0 = and_or(w << 3, mask_s, magic_v);
    uint32_t p1 = and_or(w >> 1, mask_s, magic_v);
    uint32_t p2 = and_or(w >> 5, mask_s, magic_v);
    uint32_t p3 = and_or(w >> 9, mask_s, magic_v);
    uint4 v = {p0, p1, p2, p3};
    return __builtin_bit_cast(bf16x8_t, v);
}

__device__ __forceinline__ bf16x8_t unpack_frag8(uint32_t w0, uint32_t w1) {
    uint32_t p[4];
    unpack8_word(w0, p);
    unpack8_word(w1, p + 2);
    uint4 v = {p[0], p[1], p[2], p[3]};
    return __builtin_bit_cast(bf16x8_t, v);
}

__device__ __forceinline__ uint32_t dup16(uint32_t h) { return (h & 0xffffu) | (h << 16); }

}  // namespace

template <int BITS, int MB, int NB, int WM, int WN>
__global__ __launch_bounds__(WM* WN* kWave) void qmm_kernel(const QmmArgs a) {
    using C = MmaCodec<BITS>;
    constexpr int BM = WM * MB * 32;
    constexpr int BN = WN * NB * 32;
    constexpr int NT = WM * WN * kWave;
    constexpr int MBLK = BM / 32;
    constexpr int XF_STAGE = MBLK * 4 * 1024;  // bytes of fragment-major x per group block
    constexpr int PPT = BM * 8 / NT;           // 16-byte x pieces staged per thread per group block
    constexpr int WPL = C::kWordsPerLane;
    static_assert(BM * 8 % NT == 0, "x staging must divide evenly");

    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* xf = lds;                                               // [2][XF_STAGE]
    uint32_t* xsum = reinterpret_cast<uint32_t*>(lds + 2 * XF_STAGE);  // [BM][8] (hi | lo << 16)

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = tid / kWave;
    const int wave_m = wave / WN;
    const int wave_n = wave % WN;
    const int j = lane & 31;
    const int h = lane >> 5;

    const int K = a.K, M = a.M, N = a.N;
    const int G = K / 64;                       // 64-code group blocks along K
    const int sb_per_row = G / a.gs_blocks;     // scales per weight row
    const int64_t words_per_row = (int64_t)K * BITS / 32;
    const int m0 = blockIdx.y * BM;
    const int n0 = blockIdx.x * BN;

    for (int i = tid; i < BM * 8; i += NT) xsum[i] = 0u;

    // weight rows of this lane, clamped so loads stay in range (stores are masked)
    const uint32_t* wrow[NB];
    const uint16_t* srow[NB];
    const uint16_t* brow[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int n = min(n0 + (wave_n * NB + nb) * 32 + j, N - 1);
        wrow[nb] = a.w + (int64_t)n * words_per_row + h * WPL;
        srow[nb] = a.s + (int64_t)n * sb_per_row;
        brow[nb] = a.b + (int64_t)n * sb_per_row;
    }

    uint4 xpiece[PPT];
    uint32_t raw[NB][WPL], raw_next[NB][WPL];
    uint32_t sbits[NB], bbits[NB], sbits_next[NB], bbits_next[NB];

    auto load_x = [&](int g) {
#pragma unroll
        for (int q = 0; q < PPT; q++) {
            const int p = tid + q * NT;
            const int row = p >> 3, c8 = p & 7;
            const int m = m0 + row;
            uint4 v = {0u, 0u, 0u, 0u};
            if (m < M) v = *reinterpret_cast<const uint4*>(a.x + (int64_t)m * K + g * 64 + c8 * 8);
            xpiece[q] = v;
        }
    };
    auto load_w = [&](int g, uint32_t (&dst)[NB][WPL], uint32_t (&sd)[NB], uint32_t (&bd)[NB]) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const uint4* p = reinterpret_cast<const uint4*>(wrow[nb] + (int64_t)g * (2 * WPL));
#pragma unroll
            for (int q = 0; q < WPL / 4; q++) {
                uint4 v = p[q];
                dst[nb][4 * q + 0] = v.x;
                dst[nb][4 * q + 1] = v.y;
                dst[nb][4 * q + 2] = v.z;
                dst[nb][4 * q + 3] = v.w;
            }
            sd[nb] = srow[nb][g / a.gs_blocks];
            bd[nb] = brow[nb][g / a.gs_blocks];
        }
    };
    auto store_x = [&](int g) {
        uint8_t* dst = xf + (g & 1) * XF_STAGE;
#pragma unroll
        for (int q = 0; q < PPT; q++) {
            const int p = tid + q * NT;
            const int row = p >> 3, c8 = p & 7;
            uint4 v = xpiece[q];
            float sx = 0.0f;
            sx = dot2_bf16(v.x, 0x3F803F80u, sx);
            sx = dot2_bf16(v.y, 0x3F803F80u, sx);
            sx = dot2_bf16(v.z, 0x3F803F80u, sx);
            sx = dot2_bf16(v.w, 0x3F803F80u, sx);
            // the 8 lanes that hold one row's group block: xor 1, xor 2, mirror within 8
            sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0xB1, 0xF, 0xF, true));
            sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0x4E, 0xF, 0xF, true));
            sx += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sx), 0x141, 0xF, 0xF, true));
            if (c8 == 0) {
                const uint32_t hi = f32_to_bf16_bits(sx);
                const uint32_t lo = f32_to_bf16_bits(sx - bf16_bits_to_f32(hi));
                xsum[row * 8 + (g & 7)] = hi | (lo << 16);
            }
            if constexpr (BITS == 4) {
                uint4 o;
                o.x = (v.x & 0xffffu) | (v.z << 16);
                o.y = (v.x >> 16) | (v.z & 0xffff0000u);
                o.z = (v.y & 0xffffu) | (v.w << 16);
                o.w = (v.y >> 16) | (v.w & 0xffff0000u);
                v = o;
            }
            const int t = c8 & 3, hh = c8 >> 2;
            *reinterpret_cast<uint4*>(dst + ((row >> 5) * 4 + t) * 1024 + (hh * 32 + (row & 31)) * 16) = v;
        }
    };

    f32x16_t out[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) out[mb][nb][r] = 0.0f;

    uint32_t sq[NB][4], bq[NB][4];  // scale / bias bits of the current four group blocks
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int q = 0; q < 4; q++) sq[nb][q] = bq[nb][q] = 0u;

    const uint32_t mask_s = opaque_s(kMask16);   // both stay in registers so that
    const uint32_t magic_v = opaque_v(kMagic16);  // (w & mask) | magic is a single v_and_or_b32

    load_x(0);
    load_w(0, raw, sbits, bbits);
    __syncthreads();  // xsum zero fill
    store_x(0);
    __syncthreads();

    for (int g = 0; g < G; g++) {
        const bool more = g + 1 < G;
        if (more) {
            load_x(g + 1);
            load_w(g + 1, raw_next, sbits_next, bbits_next);
        }

        bf16x8_t bfrag[NB][4];
        float sc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
#pragma unroll
            for (int t = 0; t < 4; t++) {
                if constexpr (BITS == 4) {
                    bfrag[nb][t] = unpack_frag4(raw[nb][t], mask_s, magic_v);
                } else {
                    bfrag[nb][t] = unpack_frag8(raw[nb][2 * t], raw[nb][2 * t + 1]);
                }
            }
            sc[nb] = bf16_bits_to_f32(sbits[nb]);
            sq[nb][g & 3] = sbits[nb];
            bq[nb][g & 3] = bbits[nb];
        }

        const uint8_t* xbuf = xf + (g & 1) * XF_STAGE;
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
            bf16x8_t afrag[4];
#pragma unroll
            for (int t = 0; t < 4; t++)
                afrag[t] = *reinterpret_cast<const bf16x8_t*>(xbuf + ((wave_m * MB + mb) * 4 + t) * 1024 + lane * 16);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                f32x16_t p = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; t++) p = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afrag[t], bfrag[nb][t], p, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; r++) out[mb][nb][r] = __fmaf_rn(sc[nb], p[r], out[mb][nb][r]);
            }
        }

        if ((g & 3) == 3 || !more) {
            // affine terms of up to four group blocks in one MFMA: k-slots (2q, 2q+1) carry
            // (Sx_hi, Sx_lo) of block q on the A side; lanes h=0 pair them with bias,
            // lanes h=1 with -off*scale.
            bf16x8_t bb[NB];
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
                uint32_t v[4];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t neg = __float_as_uint(bf16_bits_to_f32(sq[nb][q]) * -C::kOffset) >> 16;
                    v[q] = dup16(h ? neg : bq[nb][q]);
                    sq[nb][q] = 0u;
                    bq[nb][q] = 0u;
                }
                uint4 u = {v[0], v[1], v[2], v[3]};
                bb[nb] = __builtin_bit_cast(bf16x8_t, u);
            }
            const int quad = (g >> 2) & 1;
#pragma unroll
            for (int mb = 0; mb < MB; mb++) {
                const int row = (wave_m * MB + mb) * 32 + j;
                const bf16x8_t aa = *reinterpret_cast<const bf16x8_t*>(xsum + row * 8 + quad * 4);
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    out[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(aa, bb[nb], out[mb][nb], 0, 0, 0);
            }
        }

        if (more) {
            store_x(g + 1);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) {
#pragma unroll
                for (int q = 0; q < WPL; q++) raw[nb][q] = raw_next[nb][q];
                sbits[nb] = sbits_next[nb];
                bbits[nb] = bbits_next[nb];
            }
        }
        __syncthreads();
    }

    // D layout of v_mfma_f32_32x32x*: lane (j, h), register r -> row 8*(r/4) + 4*h + r%4, column j
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const int n = n0 + (wave_n * NB + nb) * 32 + j;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + (wave_m * MB + mb) * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
                if (m < M && n < N) {
                    const int64_t o = (int64_t)m * N + n;
                    if (a.out_f32) {
                        reinterpret_cast<float*>(a.y)[o] = out[mb][nb][r];
                    } else {
                        reinterpret_cast<uint16_t*>(a.y)[o] = f32_to_bf16_bits(out[mb][nb][r]);
                    }
                }
            }
        }
    }
}

__global__ __launch_bounds__(256) void fill_zero_kernel(uint32_t* p, size_t words, uint8_t* tail, size_t tail_bytes) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t k = i; k < words; k += stride) p[k] = 0u;
    if (i < tail_bytes) tail[i] = 0;
}

hipError_t fill_zero_launch(void* p, size_t bytes, hipStream_t stream) {
    uint8_t* b = static_cast<uint8_t*>(p);
    size_t head = (4 - (reinterpret_cast<uintptr_t>(b) & 3)) & 3;
    if (head > bytes) head = bytes;
    // unaligned head and tail bytes go through the byte path
    const size_t words = (bytes - head) / 4;
    const size_t tail = bytes - head - words * 4;
    if (head) hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(256), 0, stream, nullptr, 0, b, head);
    size_t blocks = (words + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       reinterpret_cast<uint32_t*>(b + head), words, b + head + words * 4, tail);
    return hipGetLastError();
}

// ---- variant table --------------------------------------------------------

typedef void (*QmmKernel)(const QmmArgs);
struct QmmEntry {
    QmmVariant v;
    QmmKernel fn;
    int lds_bytes;
};

#define AQ_QMM(BITS, MB, NB, WM, WN)                                                    \
    {                                                                                   \
        {"qmm_b" #BITS "_mb" #MB "_nb" #NB "_wm" #WM "_wn" #WN, BITS, MB, NB, WM, WN},  \
            qmm_kernel<BITS, MB, NB, WM, WN>, 2 * (WM * MB) * 4096 + (WM * MB * 32) * 32 \
    }

#define AQ_QMM_SET(BITS)                                                                         \
    AQ_QMM(BITS, 1, 1, 1, 4), AQ_QMM(BITS, 1, 2, 1, 4), AQ_QMM(BITS, 1, 2, 1, 2),                \
        AQ_QMM(BITS, 2, 2, 1, 4), AQ_QMM(BITS, 2, 2, 2, 2), AQ_QMM(BITS, 2, 2, 2, 4),            \
        AQ_QMM(BITS, 2, 1, 2, 4), AQ_QMM(BITS, 4, 1, 1, 4), AQ_QMM(BITS, 4, 1, 2, 4),            \
        AQ_QMM(BITS, 3, 2, 2, 2), AQ_QMM(BITS, 4, 2, 1, 4)

static const QmmEntry kQmmTable[] = {AQ_QMM_SET(4), AQ_QMM_SET(8)};

int qmm_variant_count() { return (int)(sizeof(kQmmTable) / sizeof(kQmmTable[0])); }
const QmmVariant* qmm_variant(int idx) {
    if (idx < 0 || idx >= qmm_variant_count()) return nullptr;
    return &kQmmTable[idx].v;
}
const char* qmm_variant_name(int idx) {
    const QmmVariant* v = qmm_variant(idx);
    return v ? v->name : "";
}

hipError_t qmm_launch(int idx, const QmmArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmm_variant_count()) return hipErrorInvalidValue;
    const QmmEntry& e = kQmmTable[idx];
    const int bm = e.v.wm * e.v.mb * 32, bn = e.v.wn * e.v.nb * 32;
    dim3 grid((unsigned)((a.N + bn - 1) / bn), (unsigned)((a.M + bm - 1) / bm), 1u);
    dim3 block((unsigned)(e.v.wm * e.v.wn * kWave), 1u, 1u);
    if (e.lds_bytes > 48 * 1024) {
        hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(e.fn),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, e.lds_bytes);
        if (rc != hipSuccess) return rc;
    }
    hipLaunchKernelGGL(e.fn, grid, block, (size_t)e.lds_bytes, stream, a);
    return hipGetLastError();
}

static int find_qmm(int bits, int mb, int nb, int wm, int wn) {
    for (int i = 0; i < qmm_variant_count(); i++) {
        const QmmVariant& v = kQmmTable[i].v;
        if (v.bits == bits && v.mb == mb && v.nb == nb && v.wm == wm && v.wn == wn) return i;
    }
    return -1;
}

// Makes ws hold at least `need` bytes.  Growing frees the old block, so everything queued on the stream
// is drained first; a stream that is being captured cannot be drained.
static int grow_workspace(Workspace* ws, size_t need, hipStream_t stream, FailFn fail) {
    ws->touched = true;
    if (ws->bytes >= need) return AQ_OK;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (stream != nullptr && hipStreamIsCapturing(stream, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone)
        return fail(AQ_ERR_UNSUPPORTED,
                    "the context's workspace must grow to %zu bytes, which cannot happen during stream capture; "
                    "run the call once, or call aq_reserve_workspace / aq_reserve_workspace_bytes, before capturing", need);
    hipError_t rc = hipStreamSynchronize(stream);
    if (rc != hipSuccess) return fail((int)rc, "rocm.hip.hipStreamSynchronize: HIP returned %d", (int)rc);
    if (ws->ptr) (void)hipFree(ws->ptr);
    ws->ptr = nullptr;
    ws->bytes = 0;
    ws->generation++;  // graphs captured over the old block must not run again
    const size_t want = need + need / 4;  // headroom: prompts grow a little from call to call
    rc = hipMalloc(&ws->ptr, want);
    if (rc != hipSuccess) return fail(AQ_ERR_NOMEM, "aq_qmm: cannot allocate a %zu-byte workspace (HIP %d)", want, (int)rc);
    ws->bytes = want;
    return AQ_OK;
}

int workspace_reserve(hipStream_t stream, Workspace* ws, size_t need, FailFn fail) {
    return grow_workspace(ws, need, stream, fail);
}

size_t qmm_scratch_bytes(int M, int K, int N) {
    const size_t xbytes = (qmmt_workspace_bytes(M, K) + 255) & ~(size_t)255;
    const size_t partial = (M > 4 && M <= 64) ? qmmt_splitk_bytes(M, N, 16) : 0;
    return xbytes + ((partial + 255) & ~(size_t)255);
}

int qmm_reserve(hipStream_t stream, Workspace* ws, int M, int K, FailFn fail) {
    return grow_workspace(ws, qmmt_workspace_bytes(M, K), stream, fail);
}

static int find_qmmt(int bits, int mb, int nb, int wm, int wn) {
    for (int i = 0; i < qmmt_variant_count(); i++) {
        const QmmVariant* v = qmmt_variant(i);
        if (v->bits == bits && v->mb == mb && v->nb == nb && v->wm == wm && v->wn == wn) return i;
    }
    return -1;
}

static int find_qmmt_named(const char* name) {
    for (int i = 0; i < qmmt_variant_count(); i++)
        if (strcmp(qmmt_variant(i)->name, name) == 0) return i;
    return -1;
}

int qmm_dispatch(hipStream_t stream, Workspace* ws, int cu_count, int forced, const char** last_variant, const void* x,
                 const void* packed, const void* scales, const void* biases, void* y, int M, int K, int N,
                 int group_size, int bits, bool out_f32, FailFn fail) {
    const bool mfma_ok = (bits == 4 || bits == 8) && (group_size == 64 || group_size == 128) && K % 64 == 0 &&
                         (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0;
    if (!mfma_ok) {
        // any other geometry: the any-width matvec kernel walks the rows of x
        QmvArgs q{};
        q.x = static_cast<const uint16_t*>(x);
        q.w = static_cast<const uint32_t*>(packed);
        q.s = static_cast<const uint16_t*>(scales);
        q.b = static_cast<const uint16_t*>(biases);
        q.y = y;
        q.K = K;
        q.N = N;
        q.M = M;
        q.out_f32 = out_f32 ? 1 : 0;
        q.routes = 1;
        *last_variant = "qmv_generic";
        hipError_t rc = qmv_generic_launch(q, bits, group_size, false, stream);
        if (rc != hipSuccess) return fail((int)rc, "rocm.hip.hipLaunchKernel: HIP returned %d", (int)rc);
        return AQ_OK;
    }
    QmmArgs a{};
    a.x = static_cast<const uint16_t*>(x);
    a.w = static_cast<const uint32_t*>(packed);
    a.s = static_cast<const uint16_t*>(scales);
    a.b = static_cast<const uint16_t*>(biases);
    a.y = y;
    a.M = M;
    a.K = K;
    a.N = N;
    a.gs_blocks = group_size / 64;
    a.out_f32 = out_f32 ? 1 : 0;
    int idx = forced;
    const int n_direct = qmm_variant_count();
    int tile_idx = -1;
    if (idx >= n_direct) {
        tile_idx = idx - n_direct;
        const QmmVariant* v = qmmt_variant(tile_idx);
        if (!v || v->bits != bits) return fail(AQ_ERR_ARG, "aq_qmm: forced variant %d does not fit bits=%d", idx, bits);
        if (qmmt_variant_stages_quads(tile_idx) && !qmmt_quad_staging_ok(a))
            return fail(AQ_ERR_ARG, "aq_qmm: forced variant %d needs group size 64, K %% 512 == 0 and 16-byte aligned scales", idx);
    } else if (idx < 0 && M >= 64) {
        // prefill sizes: the LDS-staged 128 x 128 tiles (four 64 x 64 wavefront tiles, two workgroups a CU);
        // the 128 x 64 wavefront tiles need more registers than two wavefronts a SIMD leave and measure slower
        tile_idx = find_qmmt(bits, 2, 2, 2, 2);
        // 4 bit, enough 256 x 128 tiles to fill the chip twice over: the kernels whose MFMA operand carries
        // scale * (code - 8) as fp16 (half the vector instructions per MFMA, no fp32 work on the accumulators;
        // measured 10 % faster at 2048 x 14336)
        if (bits == 4 && (int64_t)((M + 255) / 256) * ((N + 127) / 128) >= 2 * (cu_count > 0 ? cu_count : 256)) {
            int half = find_qmmt_named("qmmh_b4_mb4_nb2_wm2_wn2_s2c");
            // at least one 256 x 256 tile per CU: eight wavefronts on a tile that feeds twice the MFMAs per byte of x
            // copied into LDS, three stages (the copies of x were at two thirds of what a CU takes in; measured
            // 0.305 -> 0.277 ms at 2048 x 14336 x 4096)
            if ((int64_t)((M + 255) / 256) * ((N + 255) / 256) >= (cu_count > 0 ? cu_count : 256)) {
                const int wide = find_qmmt_named("qmmh_b4_mb4_nb2_wm2_wn4");
                if (wide >= 0) half = wide;
            }
            if (half >= 0) tile_idx = half;
        }
    }
    // Few rows of x: M x N tiles alone would occupy a fraction of the chip (56 workgroups for 32 x 14336), so
    // K is shared out as well and a small kernel adds the partial tiles.
    int ksplit = 1;
    if (idx < 0 && M > 4 && M <= 64 && (K / 64) % 4 == 0) {
        // the kernels whose LDS stages hold four blocks of K: 32 or 64 rows by 256 (8 bit: 128) columns per workgroup
        const int bm = M <= 32 ? 32 : 64, bn = bits == 4 ? 256 : 128;
        const int want = find_qmmt_named(bits == 4 ? (M <= 32 ? "qmmf_b4_mb1_nb2_wm1_wn4" : "qmmf_b4_mb2_nb2_wm1_wn4")
                                                   : (M <= 32 ? "qmmf_b8_mb1_nb1_wm1_wn4" : "qmmf_b8_mb2_nb1_wm1_wn4"));
        if (want >= 0) {
            const int tiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn);
            const int cus = cu_count > 0 ? cu_count : 256;
            // as many workgroups as CUs at most (their LDS allows one each); every workgroup takes whole quads of K
            // and at least two of them; at most 16 partial tiles per output tile
            int ks = 1;
            for (int k = 2; k <= 16; k++)
                if ((K / 64) % (4 * k) == 0 && tiles * k <= cus && (K / 64) / k >= 8) ks = k;
            tile_idx = want;
            ksplit = ks;
        }
    }
    if (tile_idx >= 0) {
        const size_t xbytes = (qmmt_workspace_bytes(M, K) + 255) & ~(size_t)255;
        if (int rc = grow_workspace(ws, xbytes + qmmt_splitk_bytes(M, N, ksplit), stream, fail)) return rc;
        *last_variant = qmmt_variant(tile_idx)->name;
        hipError_t rc = qmmt_launch_splitk(tile_idx, a, ws->ptr, ksplit, stream);
        if (rc != hipSuccess) return fail((int)rc, "rocm.hip.hipLaunchKernel: HIP returned %d (%s)", (int)rc, hipGetErrorString(rc));
        return AQ_OK;
    }
    if (idx >= 0) {
        const QmmVariant* v = qmm_variant(idx);
        if (!v || v->bits != bits) return fail(AQ_ERR_ARG, "aq_qmm: forced variant %d does not fit bits=%d", idx, bits);
    } else {
        if (M <= 32) {
            idx = find_qmm(bits, 1, 2, 1, 4);
        } else if (M <= 64) {
            idx = find_qmm(bits, 2, 2, 1, 4);
        } else {
            idx = find_qmm(bits, 2, 2, 2, 2);
        }
        if (idx < 0) return fail(AQ_ERR_UNSUPPORTED, "aq_qmm: no kernel variant for bits=%d", bits);
    }
    *last_variant = kQmmTable[idx].v.name;
    hipError_t rc = qmm_launch(idx, a, stream);
    if (rc != hipSuccess) return fail((int)rc, "rocm.hip.hipLaunchKernel: HIP returned %d (%s)", (int)rc, hipGetErrorString(rc));
    return AQ_OK;
}

}  // namespace aq
