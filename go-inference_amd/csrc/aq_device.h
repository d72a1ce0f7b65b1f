// Device-side helpers shared by the gfx950 affine kernels: bf16 codecs that
// match the reference's integer RNE codec bit for bit, the packed-code ->
// bf16-pair unpackers, and a 64-lane DPP sum.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aq {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr int kWave = 64;

// bf16 -> f32 is a 16-bit left shift (go/model/quant/mlxaffine/mlxaffine.go:239-241).
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// f32 -> bf16, round-to-nearest-even on the kept LSB, NaN forced quiet: the
// same integer recipe as go/model/quant/mlxaffine/mlxaffine.go:229-237, so a
// store of the same fp32 value gives the same 16 bits as the CPU path.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

// Two fp32 -> two bf16 in one word (lo in the low half) with gfx950's conversion instruction
// (v_cvt_pk_bf16_f32).  It rounds to nearest even and quiets NaNs exactly as f32_to_bf16_bits does: the two
// were compared on the device over all 2^32 input patterns, NaN payloads included, without a mismatch.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_local_t;
    const f32x2_local_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// (a & mask) | magic, meant to become one v_and_or_b32.  gfx9 VOP3 cannot carry 32-bit literals,
// so with literal constants the compiler emits two VOP2 ops; callers therefore pass the mask and
// the magic through opaque_s / opaque_v, which hides their values and leaves them in registers.
// Plain C on purpose: an inline-asm VALU instruction is invisible to the compiler's hazard
// recogniser, and next to MFMAs (operands or results in VGPRs) that produced wrong sums.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) { return (a & mask) | magic; }

// Launder a constant through an empty asm so that it stays in an SGPR / VGPR.
__device__ __forceinline__ uint32_t opaque_s(uint32_t v) {
    asm volatile("" : "+s"(v));
    return v;
}
__device__ __forceinline__ uint32_t opaque_v(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
}

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc,
                                           false);
}

// One packed word of eight 4-bit codes c0..c7 -> four bf16 pairs
//   p[i] = (128 + c_i, 128 + c_{i+4})        (low half, high half)
// 0x4300 is bf16 128.0, whose mantissa LSB weighs exactly 1, so OR-ing a
// nibble into the low mantissa bits gives 128 + code with no rounding.  The
// matching activation order is (x_i, x_{i+4}); the 128 offset is removed by
// the caller through the chunk's activation sum.
constexpr uint32_t kNibbleMask = 0x000F000Fu;
constexpr uint32_t kMagic128 = 0x43004300u;
constexpr float kNibbleOffset = 128.0f;

__device__ __forceinline__ void unpack4_word(uint32_t w, uint32_t mask_s, uint32_t magic_v, uint32_t p[4]) {
    p[0] = and_or(w, mask_s, magic_v);
    p[1] = and_or(w >> 4, mask_s, magic_v);
    p[2] = and_or(w >> 8, mask_s, magic_v);
    p[3] = and_or(w >> 12, mask_s, magic_v);
}

// One packed word of four 8-bit codes c0..c3 -> two bf16 pairs (c0,c1),(c2,c3).
// Codes <= 255 have 8 significant bits, so float(code) has a zero low half
// and taking the high halves is an exact bf16 conversion.
__device__ __forceinline__ void unpack8_word(uint32_t w, uint32_t p[2]) {
    uint32_t f0 = __float_as_uint((float)(w & 0xffu));
    uint32_t f1 = __float_as_uint((float)((w >> 8) & 0xffu));
    uint32_t f2 = __float_as_uint((float)((w >> 16) & 0xffu));
    uint32_t f3 = __float_as_uint((float)(w >> 24));
    p[0] = __builtin_amdgcn_perm(f1, f0, 0x07060302u);
    p[1] = __builtin_amdgcn_perm(f3, f2, 0x07060302u);
}

// Activations of the fused kernels.  1: tanh-approximated GELU with the operation order of
// rocm_gelu_tanh_value (go/engine/hip/kernels/common/math.hipinc:3-9); 2: SiLU, v / (1 + exp(-v))
// (go/model/attn/gated_delta.go:228).  Contraction is off, so every step is one fp32 operation and each
// kernel that inlines this computes the same bits for the same input.
__device__ __forceinline__ float act_value(int act, float v) {
#pragma clang fp contract(off)
    if (act == 2) return v / (1.0f + expf(-v));
    const float v3 = (v * v) * v;
    const float arg = 0.7978845608028654f * __builtin_fmaf(0.044715f, v3, v);
    return (0.5f * v) * (1.0f + tanhf(arg));
}

__device__ __forceinline__ float fmul_unfused(float a, float b) {
#pragma clang fp contract(off)
    return a * b;
}

// Eight consecutive outputs of the `up` projection (columns n .. n + 7 of a row of N, element offset o) times the
// activation of the `gate` projection's fp32 sums at the same places: the element-wise step of a gated MLP as the
// epilogue of the second projection.  The same two operations, in the same order, as the stand-alone kernel over two
// fp32 matrices (act_mul_f32_launch), so the fused and the unfused route store the same bytes.
__device__ __forceinline__ void gate_mul8(const float* gate, int act, int64_t o, int n, int N, float4& lo, float4& hi) {
    float g[8];
    if ((reinterpret_cast<uintptr_t>(gate) & 15) == 0 && (N & 3) == 0 && n + 8 <= N) {
        const float4 a = *reinterpret_cast<const float4*>(gate + o), b = *reinterpret_cast<const float4*>(gate + o + 4);
        g[0] = a.x, g[1] = a.y, g[2] = a.z, g[3] = a.w, g[4] = b.x, g[5] = b.y, g[6] = b.z, g[7] = b.w;
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) g[e] = n + e < N ? gate[o + e] : 0.0f;
    }
    lo.x = fmul_unfused(act_value(act, g[0]), lo.x);
    lo.y = fmul_unfused(act_value(act, g[1]), lo.y);
    lo.z = fmul_unfused(act_value(act, g[2]), lo.z);
    lo.w = fmul_unfused(act_value(act, g[3]), lo.w);
    hi.x = fmul_unfused(act_value(act, g[4]), hi.x);
    hi.y = fmul_unfused(act_value(act, g[5]), hi.y);
    hi.z = fmul_unfused(act_value(act, g[6]), hi.z);
    hi.w = fmul_unfused(act_value(act, g[7]), hi.w);
}

// bf16(act(gate) * up): fp32 inside, one rounding at the end, as lthn_gelu_gate_mul_one
// (go/engine/metal/kernels/moe/lthn_gelu_qmv_impl.h:24-33).
__device__ __forceinline__ uint32_t act_mul_bf16x2(uint32_t g, uint32_t u, int act) {
#pragma clang fp contract(off)
    const float lo = act_value(act, bf16_bits_to_f32(g & 0xffffu)) * bf16_bits_to_f32(u & 0xffffu);
    const float hi = act_value(act, bf16_bits_to_f32(g >> 16)) * bf16_bits_to_f32(u >> 16);
    return (uint32_t)f32_to_bf16_bits(lo) | ((uint32_t)f32_to_bf16_bits(hi) << 16);
}
__device__ __forceinline__ uint4 act_mul_bf16x8(uint4 g, uint4 u, int act) {
    uint4 o;
    o.x = act_mul_bf16x2(g.x, u.x, act);
    o.y = act_mul_bf16x2(g.y, u.y, act);
    o.z = act_mul_bf16x2(g.z, u.z, act);
    o.w = act_mul_bf16x2(g.w, u.w, act);
    return o;
}

// Score and row index packed so that an unsigned 64-bit maximum picks the highest score and, among equal
// scores, the lowest index: rocm_ordered_float_key / rocm_pack_score_index
// (go/engine/hip/kernels/common/numeric.hipinc:84-96; host side hipPackGreedyBest,
// go/engine/hip/hip_projection_launch.go:2393-2395).  0 means "no candidate".
__device__ __forceinline__ uint32_t ordered_float_key(float v) {
    const uint32_t bits = __float_as_uint(v);
    return (bits & 0x80000000u) ? ~bits : (bits ^ 0x80000000u);
}
__device__ __forceinline__ unsigned long long pack_score_index(float score, uint32_t index) {
    return ((unsigned long long)ordered_float_key(score) << 32) | (unsigned long long)(~index);
}
// rocm_mlx_q4_token_suppressed (go/engine/hip/kernels/quant/affine_fused_validate.hipinc:3-15)
__device__ __forceinline__ bool token_suppressed(uint32_t row, const int32_t* suppress, int count) {
    for (int i = 0; i < count; i++)
        if (suppress[i] == (int32_t)row) return true;
    return false;
}

// Sum over the 64 lanes of a wavefront; every lane returns the total.
// Four DPP adds fold each 16-lane row, then the four row totals are read
// through SGPRs.
__device__ __forceinline__ float wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (a + b) + (c + d);
}

}  // namespace aq
