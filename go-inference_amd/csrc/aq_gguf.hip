// GGUF block formats -> the affine layout, on the device: the tensor stays in HBM, where the reference
// copies it to the host, repacks it there and uploads three tensors again
// (synthesizeGemma4GGUFAffineTensor, go/engine/hip/hip_gguf_affine_adapter.go:199-218; the per-format
// loops hipRepackGGUF*ToAffine :342-648, hipQuantizeGGUFF32ToAffine8 :650-720).
//
// HBM-bound byte work.  One thread owns a span of 32 columns: it reads its piece of the block, writes the
// span's `bits` output words (consecutive threads write consecutive pieces, so a wavefront writes one
// contiguous 1..2 KB run) and the span's one or two (scale, bias) pairs.  Because every format's span is a
// whole number of words and of groups, the tensor is one flat run of spans and the kernel needs no row
// arithmetic.  Nibbles and 6-bit fields are moved eight at a time with 64-bit mask-and-shift steps rather
// than a code at a time.
//
// The arithmetic on scales follows the reference to the bit: half -> float by the integer recipe of
// hipFloat16ToFloat32 (hip_projection_reference.go:240-261; the hardware conversion would quiet signalling
// NaNs), products in fp32, float -> bf16 by adding 0x7fff + lsb to the bit pattern with NO NaN case
// (hipFloat32ToBFloat16, hip_bf16_portable.go:19-23).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "aq_kernels.h"

namespace aq {
namespace {

constexpr int kSpanThreads = 256;

__device__ __forceinline__ float half_bits_to_f32(uint32_t h) {
    const uint32_t sign = (h & 0x8000u) << 16;
    const uint32_t exponent = (h >> 10) & 0x1fu;
    uint32_t fraction = h & 0x03ffu;
    uint32_t bits;
    if (exponent == 0) {
        if (fraction == 0) {
            bits = sign;
        } else {  // subnormal half: normalise
            const int shift = __clz(fraction) - 21;  // brings the leading one to bit 10
            fraction = (fraction << shift) & 0x03ffu;
            bits = sign | (uint32_t)(127 - 14 - shift) << 23 | fraction << 13;
        }
    } else if (exponent == 0x1f) {
        bits = sign | 0x7f800000u | fraction << 13;
    } else {
        bits = sign | (exponent + 112u) << 23 | fraction << 13;
    }
    return __uint_as_float(bits);
}

__device__ __forceinline__ uint16_t bf16_bits_no_nan_case(float v) {
    uint32_t bits = __float_as_uint(v);
    bits += 0x7fffu + ((bits >> 16) & 1u);
    return (uint16_t)(bits >> 16);
}

// Block fields sit at odd offsets (18-, 34- and 210-byte blocks): the loads are written as copies of unknown
// alignment and the compiler picks the widest access the target allows for them.
__device__ __forceinline__ uint32_t rd16(const uint8_t* p) {
    uint16_t v;
    __builtin_memcpy(&v, p, 2);
    return v;
}
__device__ __forceinline__ uint32_t rd32(const uint8_t* p) {
    uint32_t v;
    __builtin_memcpy(&v, p, 4);
    return v;
}
__device__ __forceinline__ uint64_t rd64(const uint8_t* p) {
    uint64_t v;
    __builtin_memcpy(&v, p, 8);
    return v;
}

// The low nibbles of eight bytes -> one word, byte i's nibble at bits [4i, 4i+4).
__device__ __forceinline__ uint32_t squeeze_nibbles(uint64_t v) {
    v &= 0x0f0f0f0f0f0f0f0fULL;
    v = (v | v >> 4) & 0x00ff00ff00ff00ffULL;
    v = (v | v >> 8) & 0x0000ffff0000ffffULL;
    return (uint32_t)(v | v >> 16);
}

// Eight bytes holding values below 64 -> 48 bits, byte i's value at bits [6i, 6i+6).
__device__ __forceinline__ uint64_t squeeze_sixes(uint64_t v) {
    v = (v & 0x003f003f003f003fULL) | ((v >> 2) & 0x0fc00fc00fc00fc0ULL);
    v = (v & 0x00000fff00000fffULL) | ((v >> 4) & 0x00fff00000fff000ULL);
    return (v & 0x0000000000ffffffULL) | ((v >> 8) & 0x0000ffffff000000ULL);
}

// Four 48-bit pieces (32 six-bit codes) -> the span's six words.
__device__ __forceinline__ void store_sixes(uint32_t* w, uint64_t t0, uint64_t t1, uint64_t t2, uint64_t t3) {
    uint2* out = reinterpret_cast<uint2*>(w);  // 24 bytes per span: 8-byte aligned
    out[0] = make_uint2((uint32_t)t0, (uint32_t)(t0 >> 32) | (uint32_t)t1 << 16);
    out[1] = make_uint2((uint32_t)(t1 >> 16), (uint32_t)t2);
    out[2] = make_uint2((uint32_t)(t2 >> 32) | (uint32_t)t3 << 16, (uint32_t)(t3 >> 16));
}

// The 6-bit (scale, min) pair of group g from a K-quant block's 12 packed bytes, given as three words
// (hipGGUFQ4KScaleMin, hip_gguf_affine_adapter.go:793-799): groups 0..3 use the low six bits of bytes g and g+4;
// groups 4..7 a nibble of byte g+4 with the top two bits of byte g-4 (scale) or of byte g (min).  No branch:
// with l = g % 4 the three bytes involved are l, l+4 and l+8 either way.
__device__ __forceinline__ void k_scale_min(uint32_t w0, uint32_t w1, uint32_t w2, int g, uint32_t* scale,
                                            uint32_t* min) {
    const int sh = 8 * (g & 3);
    const uint32_t a = (w0 >> sh) & 0xffu, c = (w1 >> sh) & 0xffu, e = (w2 >> sh) & 0xffu;
    *scale = g < 4 ? (a & 63u) : ((e & 0x0fu) | ((a >> 6) << 4));
    *min = g < 4 ? (c & 63u) : ((e >> 4) | ((c >> 6) << 4));
}

template <int TYPE>
__global__ __launch_bounds__(kSpanThreads) void gguf_repack_kernel(const uint8_t* __restrict__ src,
                                                                   uint32_t* __restrict__ w, uint16_t* __restrict__ s,
                                                                   uint16_t* __restrict__ b, int64_t spans) {
    const int64_t span = (int64_t)blockIdx.x * kSpanThreads + threadIdx.x;
    if (span >= spans) return;
    if constexpr (TYPE == kGgufQ4_0 || TYPE == kGgufQ4_1) {
        constexpr int kHeader = TYPE == kGgufQ4_0 ? 2 : 4;
        const uint8_t* blk = src + span * (kHeader + 16);
        const float d = half_bits_to_f32(rd16(blk));
        const float bias = TYPE == kGgufQ4_0 ? -8.0f * d : half_bits_to_f32(rd16(blk + 2));
        const uint64_t lo = rd64(blk + kHeader), hi = rd64(blk + kHeader + 8);
        // lanes 0..15 are the low nibbles of the 16 bytes, lanes 16..31 their high nibbles
        *reinterpret_cast<uint4*>(w + span * 4) =
            make_uint4(squeeze_nibbles(lo), squeeze_nibbles(hi), squeeze_nibbles(lo >> 4), squeeze_nibbles(hi >> 4));
        s[span] = bf16_bits_no_nan_case(d);
        b[span] = bf16_bits_no_nan_case(bias);
    } else if constexpr (TYPE == kGgufQ8_0) {
        const uint8_t* blk = src + span * 34;
        const float d = half_bits_to_f32(rd16(blk));
        uint32_t word[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) word[i] = rd32(blk + 2 + 4 * i) ^ 0x80808080u;  // int8 + 128: top bit flipped
        uint4* out = reinterpret_cast<uint4*>(w + span * 8);
        out[0] = make_uint4(word[0], word[1], word[2], word[3]);
        out[1] = make_uint4(word[4], word[5], word[6], word[7]);
        s[span] = bf16_bits_no_nan_case(d);
        b[span] = bf16_bits_no_nan_case(-128.0f * d);
    } else if constexpr (TYPE == kGgufQ4_K || TYPE == kGgufQ5_K) {
        constexpr int kBlockBytes = TYPE == kGgufQ4_K ? 144 : 176;
        const uint8_t* blk = src + (span >> 3) * kBlockBytes;
        const int g = (int)(span & 7);
        const uint32_t head = rd32(blk);
        const float d = half_bits_to_f32(head & 0xffffu), dmin = half_bits_to_f32(head >> 16);
        uint32_t sc, mn;
        k_scale_min(rd32(blk + 4), rd32(blk + 8), rd32(blk + 12), g, &sc, &mn);
        s[span] = bf16_bits_no_nan_case(d * (float)sc);
        b[span] = bf16_bits_no_nan_case(-dmin * (float)mn);
        const int pair = g >> 1, nib_shift = (g & 1) * 4;
        if constexpr (TYPE == kGgufQ4_K) {
            const uint8_t* qs = blk + 16 + pair * 32;
            uint32_t word[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) word[i] = squeeze_nibbles(rd64(qs + 8 * i) >> nib_shift);
            *reinterpret_cast<uint4*>(w + span * 4) = make_uint4(word[0], word[1], word[2], word[3]);
        } else {
            const uint8_t* qh = blk + 16;
            const uint8_t* qs = blk + 48 + pair * 32;
            uint64_t t[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {  // code = nibble + 16 * (bit 2*pair + (g & 1) of qh[lane])
                const uint64_t nib = (rd64(qs + 8 * i) >> nib_shift) & 0x0f0f0f0f0f0f0f0fULL;
                const uint64_t top = (rd64(qh + 8 * i) >> (2 * pair + (g & 1))) & 0x0101010101010101ULL;
                t[i] = squeeze_sixes(nib | top << 4);
            }
            store_sixes(w + span * 6, t[0], t[1], t[2], t[3]);
        }
    } else if constexpr (TYPE == kGgufQ6_K) {
        // span p of a block = groups 2p and 2p+1 (16 lanes each): the same half `ip` and quartile `q`, lane
        // offsets 0 and 16, i.e. 32 consecutive bytes of ql and of qh (hipGGUFQ6KQuant, :822-841)
        const uint8_t* blk = src + (span >> 3) * 210;
        const int p = (int)(span & 7), ip = p >> 2, q = p & 3;
        const float d = half_bits_to_f32(rd16(blk + 208));
        const uint32_t two = rd16(blk + 192 + 2 * p);
        const float s0 = d * (float)(int)(int8_t)(two & 0xff), s1 = d * (float)(int)(int8_t)(two >> 8);
        s[2 * span] = bf16_bits_no_nan_case(s0);
        s[2 * span + 1] = bf16_bits_no_nan_case(s1);
        b[2 * span] = bf16_bits_no_nan_case(-32.0f * s0);
        b[2 * span + 1] = bf16_bits_no_nan_case(-32.0f * s1);
        const uint8_t* ql = blk + ip * 64 + (q & 1) * 32;
        const uint8_t* qh = blk + 128 + ip * 32;
        uint64_t t[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint64_t nib = (rd64(ql + 8 * i) >> ((q & 2) * 2)) & 0x0f0f0f0f0f0f0f0fULL;
            const uint64_t top = (rd64(qh + 8 * i) >> (2 * q)) & 0x0303030303030303ULL;
            t[i] = squeeze_sixes(nib | top << 4);
        }
        store_sixes(w + span * 6, t[0], t[1], t[2], t[3]);
    } else {  // F32 -> eight bits, groups of 32: min/max quantiser of :677-718
        const float* f = reinterpret_cast<const float*>(src) + span * 32;
        float v[32];
        float lo = 0.0f, hi = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            float x = f[i];
            if ((__float_as_uint(x) & 0x7f800000u) == 0x7f800000u) x = 0.0f;  // NaN and infinities count as zero
            v[i] = x;
            if (i == 0 || x < lo) lo = x;  // strict comparisons: the first of equal values (signed zeros) stays
            if (i == 0 || x > hi) hi = x;
        }
        float scale = __fdiv_rn(hi - lo, 255.0f);
        if (scale == 0.0f) scale = 1.0f;
        s[span] = bf16_bits_no_nan_case(scale);
        b[span] = bf16_bits_no_nan_case(lo);
        uint32_t word[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            uint32_t acc = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t code = 0;
                if (hi != lo) {
                    const float r = __builtin_roundf(__fdiv_rn(v[4 * i + j] - lo, scale));  // half away from zero
                    code = r >= 255.0f ? 255u : (uint32_t)r;
                }
                acc |= code << (8 * j);
            }
            word[i] = acc;
        }
        uint4* out = reinterpret_cast<uint4*>(w + span * 8);
        out[0] = make_uint4(word[0], word[1], word[2], word[3]);
        out[1] = make_uint4(word[4], word[5], word[6], word[7]);
    }
}

template <int TYPE>
hipError_t launch_type(const uint8_t* src, uint32_t* w, uint16_t* s, uint16_t* b, int64_t spans, hipStream_t stream) {
    const dim3 grid((unsigned)((spans + kSpanThreads - 1) / kSpanThreads)), block(kSpanThreads);
    hipLaunchKernelGGL((gguf_repack_kernel<TYPE>), grid, block, 0, stream, src, w, s, b, spans);
    return hipGetLastError();
}

}  // namespace

bool gguf_format(int type, GgufFormat* f) {
    switch (type) {
        case kGgufF32: *f = {32, 128, 8, 32}; return true;
        case kGgufQ4_0: *f = {32, 18, 4, 32}; return true;
        case kGgufQ4_1: *f = {32, 20, 4, 32}; return true;
        case kGgufQ8_0: *f = {32, 34, 8, 32}; return true;
        case kGgufQ4_K: *f = {256, 144, 4, 32}; return true;
        case kGgufQ5_K: *f = {256, 176, 6, 32}; return true;
        case kGgufQ6_K: *f = {256, 210, 6, 16}; return true;
        default: return false;
    }
}

hipError_t gguf_repack_launch(int type, const uint8_t* src, uint32_t* w, uint16_t* s, uint16_t* b, int64_t spans,
                              hipStream_t stream) {
    switch (type) {
        case kGgufF32: return launch_type<kGgufF32>(src, w, s, b, spans, stream);
        case kGgufQ4_0: return launch_type<kGgufQ4_0>(src, w, s, b, spans, stream);
        case kGgufQ4_1: return launch_type<kGgufQ4_1>(src, w, s, b, spans, stream);
        case kGgufQ8_0: return launch_type<kGgufQ8_0>(src, w, s, b, spans, stream);
        case kGgufQ4_K: return launch_type<kGgufQ4_K>(src, w, s, b, spans, stream);
        case kGgufQ5_K: return launch_type<kGgufQ5_K>(src, w, s, b, spans, stream);
        case kGgufQ6_K: return launch_type<kGgufQ6_K>(src, w, s, b, spans, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace aq
