// The two device steps on either side of the expert-gathered projections.
//
// moe_route_kernel: per token row, the top-k experts by (score descending, expert id ascending), their
//   softmax weights and the route -> token map, written as the int32 / float32 arrays aq_gather_qmv reads.
//   Selection and weights follow rocm_moe_router (go/engine/hip/kernels/moe/routing.hipinc:3-77) and the
//   host router it shadows, hipGemma4MoEBatchRouteGroups (go/engine/hip/hip_gemma4_moe.go:294-366):
//   softmax over the selected scores, times an optional per-expert scale.  With normalise off the weights
//   are the softmax over ALL experts gathered at the selection (hipQwen3MoERouterSelect,
//   go/engine/hip/hip_qwen3_moe_router.go:25-88).  The reference copies the scores to the host, groups
//   routes by expert and uploads chunks every step; here nothing leaves the device.
//
// moe_combine_kernel: out[row, :] = sum over ranks of route_rows[row*top_k + rank, :] * weight, ranks
//   ascending, the product rounded to fp32 before it is added: rocm_moe_batch_scatter_routes followed by
//   rocm_moe_batch_reduce_routes (routing.hipinc:100-158).  With bf16 steps every product and every partial
//   sum is rounded to bf16, the chain lthn_moe_weighted_sum_bf16 reproduces
//   (go/engine/metal/kernels/moe/lthn_moe_weighted_sum.metal:17-38).
//
// One wavefront per token row; expert scores sit in registers, lane l holding experts l, l+64, ...
#include <cfloat>
#include <climits>

#include "aq_device.h"
#include "aq_kernels.h"

namespace aq {

// Wave-wide maximum / minimum through DPP inside each row of 16 lanes (old value = the identity for lanes a
// pattern leaves without a source) and SGPR reads across the four rows.
__device__ __forceinline__ float wave_max_f32(float v) {
    const int ninf = __float_as_int(-INFINITY);
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(ninf, __float_as_int(v), 0xB1, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(ninf, __float_as_int(v), 0x4E, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(ninf, __float_as_int(v), 0x141, 0xF, 0xF, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(ninf, __float_as_int(v), 0x140, 0xF, 0xF, false)));
    const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
    const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
    const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
    const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}
__device__ __forceinline__ int wave_min_i32(int v) {
    v = min(v, __builtin_amdgcn_update_dpp(INT_MAX, v, 0xB1, 0xF, 0xF, false));
    v = min(v, __builtin_amdgcn_update_dpp(INT_MAX, v, 0x4E, 0xF, 0xF, false));
    v = min(v, __builtin_amdgcn_update_dpp(INT_MAX, v, 0x141, 0xF, 0xF, false));
    v = min(v, __builtin_amdgcn_update_dpp(INT_MAX, v, 0x140, 0xF, 0xF, false));
    return min(min(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 16)),
               min(__builtin_amdgcn_readlane(v, 32), __builtin_amdgcn_readlane(v, 48)));
}

template <int PER>
__global__ __launch_bounds__(256) void moe_route_kernel(const MoeRouteArgs a) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= a.rows) return;  // whole wavefronts leave together
    const int E = a.num_experts;

    float v[PER];
    bool open[PER];  // in range and not yet selected
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const int e = lane + j * kWave;
        open[j] = e < E;
        float s = -INFINITY;
        if (open[j]) {
            s = a.logits_bf16 ? bf16_bits_to_f32(static_cast<const uint16_t*>(a.logits)[(int64_t)row * E + e])
                              : static_cast<const float*>(a.logits)[(int64_t)row * E + e];
            if (s != s) s = -INFINITY;  // a NaN score never wins a comparison; rank it last
        }
        v[j] = s;
    }

    float all_max = 0.0f, all_total = 1.0f;
    if (!a.normalise) {
        float m = -INFINITY;
#pragma unroll
        for (int j = 0; j < PER; j++)
            if (open[j]) m = fmaxf(m, v[j]);
        all_max = wave_max_f32(m);
        float t = 0.0f;
#pragma unroll
        for (int j = 0; j < PER; j++)
            if (open[j]) t += expf(v[j] - all_max);
        all_total = wave_sum(t);
        if (all_total == 0.0f) all_total = 1.0f;
    }

    int my_id = 0;
    float my_score = 0.0f;
    for (int k = 0; k < a.top_k; k++) {
        float bv = -INFINITY;
        int bi = INT_MAX;
#pragma unroll
        for (int j = 0; j < PER; j++) {
            // ascending expert id inside a lane, so the strict comparison keeps the lowest id of equals
            if (open[j] && (bi == INT_MAX || v[j] > bv)) {
                bv = v[j];
                bi = lane + j * kWave;
            }
        }
        const float best = wave_max_f32(bv);
        const int winner = wave_min_i32((bi != INT_MAX && bv == best) ? bi : INT_MAX);
        if ((winner & (kWave - 1)) == lane) {
#pragma unroll
            for (int j = 0; j < PER; j++)
                if (j == (winner >> 6)) open[j] = false;
        }
        if (lane == k) {
            my_id = winner;
            my_score = best;
        }
    }

    const bool mine = lane < a.top_k;
    float p;
    if (a.normalise) {
        // the first selection holds the largest score
        const float top = __shfl(my_score, 0, kWave);
        const float e = mine ? expf(my_score - top) : 0.0f;
        const float sum = wave_sum(e);
        p = sum > 0.0f ? e / sum : 0.0f;
    } else {
        p = expf(my_score - all_max) / all_total;
    }
    if (mine) {
        if (a.expert_scales) p *= a.expert_scales[my_id];
        const int64_t o = (int64_t)row * a.top_k + lane;
        a.ids[o] = my_id;
        a.weights[o] = p;
        if (a.token_of_route) a.token_of_route[o] = row;
    }
}

__global__ __launch_bounds__(256) void moe_combine_kernel(const MoeCombineArgs a) {
#pragma clang fp contract(off)  // the product is rounded before it is added, as the two reference kernels do
    const int64_t total = (int64_t)a.rows * a.n;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int row = (int)(i / a.n);
        const int col = (int)(i - (int64_t)row * a.n);
        float acc = 0.0f;
#pragma unroll 8
        for (int r = 0; r < a.top_k; r++) {
            const int64_t pair = (int64_t)row * a.top_k + r;
            const float y = a.in_f32 ? static_cast<const float*>(a.route_rows)[pair * a.n + col]
                                     : bf16_bits_to_f32(static_cast<const uint16_t*>(a.route_rows)[pair * a.n + col]);
            float w = a.weights[pair];
            if (a.bf16_steps) {
                w = bf16_bits_to_f32(f32_to_bf16_bits(w));
                const float scaled = bf16_bits_to_f32(f32_to_bf16_bits(y * w));
                acc = r == 0 ? scaled : bf16_bits_to_f32(f32_to_bf16_bits(acc + scaled));
            } else {
                const float scaled = y * w;
                acc = acc + scaled;
            }
        }
        if (a.out_f32) {
            static_cast<float*>(a.out)[i] = acc;
        } else {
            static_cast<uint16_t*>(a.out)[i] = f32_to_bf16_bits(acc);
        }
    }
}

hipError_t moe_route_launch(const MoeRouteArgs& a, hipStream_t stream) {
    if (a.rows <= 0) return hipSuccess;
    if (a.num_experts <= 0 || a.num_experts > kMoeMaxExperts || a.top_k <= 0 || a.top_k > kMoeMaxTopK ||
        a.top_k > a.num_experts)
        return hipErrorInvalidValue;
    const dim3 grid((unsigned)((a.rows + 3) / 4)), block(256);
    const int per = (a.num_experts + kWave - 1) / kWave;
    if (per <= 1) {
        hipLaunchKernelGGL(moe_route_kernel<1>, grid, block, 0, stream, a);
    } else if (per <= 2) {
        hipLaunchKernelGGL(moe_route_kernel<2>, grid, block, 0, stream, a);
    } else if (per <= 4) {
        hipLaunchKernelGGL(moe_route_kernel<4>, grid, block, 0, stream, a);
    } else if (per <= 8) {
        hipLaunchKernelGGL(moe_route_kernel<8>, grid, block, 0, stream, a);
    } else {
        hipLaunchKernelGGL(moe_route_kernel<16>, grid, block, 0, stream, a);
    }
    return hipGetLastError();
}

hipError_t moe_combine_launch(const MoeCombineArgs& a, hipStream_t stream) {
    const int64_t total = (int64_t)a.rows * a.n;
    if (total <= 0) return hipSuccess;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a);
    return hipGetLastError();
}

}  // namespace aq
