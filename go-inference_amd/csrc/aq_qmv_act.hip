// Activation-fused matvec kernels for the MLP of a decode step (one activation row).
//
//   pair fusion    y[n] = act(gate[n,:] . x) * (up[n,:] . x): both projections and the activation in one
//                  launch, as rocm_mlx_q4_gelu_tanh_multiply does
//                  (go/engine/hip/kernels/quant/affine_gelu_tanh.hipinc:3-182); with expert ids read on the
//                  device it is the gate|up half of rocm_moe_mlx_affine_routes
//                  (go/engine/hip/kernels/moe/routing.hipinc:160-399, epilogue :312).
//   x-load fusion  y[n] = w[n,:] . bf16(act(g[k]) * u[k]): the down projection that forms its own gated
//                  input, as lthn_gelu_qmv / lthn_gather_qmv_gelu do
//                  (go/engine/metal/kernels/moe/lthn_gather_qmv.metal:98-132).
//   act_mul        the stand-alone bf16(act(g) * u) of rocm_gelu_tanh_multiply / lthn_gelu_gate_mul_bf16, and
//                  its fp32-input form that closes the unfused fallback.
//
// The streaming part is the dot2 body of aq_qmv.hip; a pair-fused wavefront streams R gate rows and the
// same R up rows, so the weights are still read exactly once and x is staged once for both.
#include "aq_qmv_body.h"

namespace aq {

template <int BITS, int R, bool GATHER, int FUSE>
__global__ __launch_bounds__(4 * kWave) void qmv_act_kernel(const QmvArgs a) {
    qmv_dot2_body<BITS, 1, R, 4, 2, GATHER, FUSE>(a, blockIdx.x);
}

typedef void (*QmvActKernel)(const QmvArgs);
struct QmvActEntry {
    int bits, fuse, rows, gather;
    QmvActKernel fn;
};
#define AQ_ACT(BITS, FUSE, R, G) {BITS, FUSE, R, G, qmv_act_kernel<BITS, R, (G != 0), FUSE>}
#define AQ_ACT_SET(BITS, G)                                                                            \
    AQ_ACT(BITS, 1, 1, G), AQ_ACT(BITS, 1, 2, G), AQ_ACT(BITS, 2, 1, G), AQ_ACT(BITS, 2, 2, G), \
        AQ_ACT(BITS, 2, 4, G)
static const QmvActEntry kActTable[] = {AQ_ACT_SET(4, 0), AQ_ACT_SET(4, 1), AQ_ACT_SET(8, 0), AQ_ACT_SET(8, 1)};

static const QmvActEntry* find_act(int bits, int fuse, int rows, bool gather) {
    for (const QmvActEntry& e : kActTable)
        if (e.bits == bits && e.fuse == fuse && e.rows == rows && (e.gather != 0) == gather) return &e;
    return nullptr;
}

bool qmv_act_supported(int bits, int fuse, int rows, bool gather) { return find_act(bits, fuse, rows, gather) != nullptr; }

hipError_t qmv_act_launch(int bits, int fuse, int rows, bool gather, const QmvArgs& a, hipStream_t stream) {
    const QmvActEntry* e = find_act(bits, fuse, rows, gather);
    if (!e || a.M != 1) return hipErrorInvalidValue;
    const int rows_per_wg = rows * 4;
    dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), gather ? (unsigned)a.routes : 1u, 1u);
    const size_t lds = (size_t)a.K * 2;
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e->fn), (size_t)lds)) return rc;
    hipLaunchKernelGGL(e->fn, grid, dim3(4 * kWave), lds, stream, a);
    return hipGetLastError();
}

// ---- element-wise forms ---------------------------------------------------

__global__ __launch_bounds__(256) void act_mul_bf16_kernel(const uint16_t* __restrict__ g, const uint16_t* __restrict__ u,
                                                           uint16_t* __restrict__ y, int64_t n, int act, int vec_ok) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    if (vec_ok) {
        const int64_t n8 = n >> 3;
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += stride)
            reinterpret_cast<uint4*>(y)[i] =
                act_mul_bf16x8(reinterpret_cast<const uint4*>(g)[i], reinterpret_cast<const uint4*>(u)[i], act);
        for (int64_t i = (n8 << 3) + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
            y[i] = (uint16_t)act_mul_bf16x2(g[i], u[i], act);
    } else {
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride)
            y[i] = (uint16_t)act_mul_bf16x2(g[i], u[i], act);
    }
}

__global__ __launch_bounds__(256) void act_mul_f32_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                          void* __restrict__ y, int64_t n, int act, int out_f32) {
#pragma clang fp contract(off)
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) {
        const float v = act_value(act, g[i]) * u[i];
        if (out_f32) {
            static_cast<float*>(y)[i] = v;
        } else {
            static_cast<uint16_t*>(y)[i] = f32_to_bf16_bits(v);
        }
    }
}

static unsigned elementwise_blocks(int64_t work_items) {
    int64_t b = (work_items + 255) / 256;
    if (b < 1) b = 1;
    if (b > 4096) b = 4096;
    return (unsigned)b;
}

hipError_t act_mul_launch(const uint16_t* gate, const uint16_t* up, uint16_t* y, int64_t n, int act, hipStream_t stream) {
    if (n <= 0) return hipSuccess;
    const uintptr_t bits = reinterpret_cast<uintptr_t>(gate) | reinterpret_cast<uintptr_t>(up) | reinterpret_cast<uintptr_t>(y);
    const int vec_ok = (bits & 15) == 0;
    hipLaunchKernelGGL(act_mul_bf16_kernel, dim3(elementwise_blocks(vec_ok ? (n + 7) / 8 : n)), dim3(256), 0, stream, gate,
                       up, y, n, act, vec_ok);
    return hipGetLastError();
}

hipError_t act_mul_f32_launch(const float* gate, const float* up, void* y, int64_t n, int act, int out_f32,
                              hipStream_t stream) {
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(act_mul_f32_kernel, dim3(elementwise_blocks(n)), dim3(256), 0, stream, gate, up, y, n, act, out_f32);
    return hipGetLastError();
}

}  // namespace aq
