// MLX layout <-> tile-major layout (aq_tile.h) of a 4-bit group-64 affine tensor, on the device.  Load-time kernels:
// they run once per tensor and move every byte once (HBM-bound byte shuffling, no arithmetic).
#include "aq_kernels.h"
#include "aq_tile.h"

namespace aq {

namespace {

struct TileGeom {
    int64_t N;
    int K, cps, halves, groups;
    uint32_t set_units, step_units;  // 16-byte units per set of rows / per full step
    int64_t units;
};

// Where unit u of the tile-major tensor comes from: row (or -1: padding), and either the byte offset of 16 packed
// bytes inside the row (kind 1) or the first of four groups (kind 0; `count` of them exist).
struct TileUnit {
    int64_t row;
    int kind;
    uint32_t byte;
    int group, count;
};
__device__ __forceinline__ TileUnit locate(const TileGeom& g, int64_t u) {
    TileUnit t;
    const int64_t set = u / g.set_units;
    const uint32_t r = (uint32_t)(u - set * g.set_units);
    const uint32_t sp = r / g.step_units, q = r - sp * g.step_units;
    const uint32_t block = q >> 6, lane = q & 63, n = lane & 15, j = lane >> 4;
    t.row = set * kTileRows + n;
    if (t.row >= g.N) t.row = -1;
    if (block == 0) {
        t.kind = 0;
        t.byte = 0;
        t.group = 4 * ((int)sp * g.cps + (int)j);
        t.count = (int)j < g.cps ? min(4, g.groups - t.group) : 0;
        if (t.count < 0) t.count = 0;
    } else {
        const int h = 2 * (int)sp * g.cps + (int)block - 1;  // half of the row
        t.kind = 1;
        t.byte = (uint32_t)h * 64 + j * 16;
        t.group = 0;
        t.count = h < g.halves ? 1 : 0;
    }
    return t;
}

__global__ __launch_bounds__(256) void tile_repack_kernel(const uint8_t* __restrict__ w, const uint16_t* __restrict__ s,
                                                          const uint16_t* __restrict__ b, uint4* __restrict__ out, TileGeom g) {
    const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (u >= g.units) return;
    const TileUnit t = locate(g, u);
    uint4 v = make_uint4(0, 0, 0, 0);
    if (t.row >= 0 && t.count > 0) {
        if (t.kind == 1) {
            v = *reinterpret_cast<const uint4*>(w + t.row * (int64_t)(g.K >> 1) + t.byte);
        } else {
            uint32_t sv[4] = {0, 0, 0, 0}, bv[4] = {0, 0, 0, 0};
            for (int i = 0; i < t.count; i++) {
                sv[i] = s[t.row * g.groups + t.group + i];
                bv[i] = b[t.row * g.groups + t.group + i];
            }
            v = make_uint4(sv[0] | sv[1] << 16, sv[2] | sv[3] << 16, bv[0] | bv[1] << 16, bv[2] | bv[3] << 16);
        }
    }
    out[u] = v;
}

__global__ __launch_bounds__(256) void tile_unpack_kernel(const uint4* __restrict__ in, uint8_t* __restrict__ w,
                                                          uint16_t* __restrict__ s, uint16_t* __restrict__ b, TileGeom g) {
    const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (u >= g.units) return;
    const TileUnit t = locate(g, u);
    if (t.row < 0 || t.count <= 0) return;
    const uint4 v = in[u];
    if (t.kind == 1) {
        *reinterpret_cast<uint4*>(w + t.row * (int64_t)(g.K >> 1) + t.byte) = v;
    } else {
        const uint32_t sv[4] = {v.x & 0xffffu, v.x >> 16, v.y & 0xffffu, v.y >> 16};
        const uint32_t bv[4] = {v.z & 0xffffu, v.z >> 16, v.w & 0xffffu, v.w >> 16};
        for (int i = 0; i < t.count; i++) {
            s[t.row * g.groups + t.group + i] = (uint16_t)sv[i];
            b[t.row * g.groups + t.group + i] = (uint16_t)bv[i];
        }
    }
}

bool make_geom(int64_t N, int K, TileGeom* g) {
    const int64_t total = tile_total_bytes(N, K, 64, 4);
    if (total < 0) return false;
    g->N = N;
    g->K = K;
    g->cps = tile_cps_for(K);
    g->halves = K >> 7;
    g->groups = K >> 6;
    g->set_units = tile_set_bytes(K, g->cps) / 16;
    g->step_units = tile_step_bytes(g->cps) / 16;
    g->units = total / 16;
    return true;
}

}  // namespace

hipError_t tile_repack_launch(const void* w, const void* s, const void* b, void* tiled, int64_t N, int K, hipStream_t stream) {
    TileGeom g;
    if (!make_geom(N, K, &g) || (g.units + 255) / 256 > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(tile_repack_kernel, dim3((unsigned)((g.units + 255) / 256)), dim3(256), 0, stream,
                       static_cast<const uint8_t*>(w), static_cast<const uint16_t*>(s), static_cast<const uint16_t*>(b),
                       static_cast<uint4*>(tiled), g);
    return hipGetLastError();
}

hipError_t tile_unpack_launch(const void* tiled, void* w, void* s, void* b, int64_t N, int K, hipStream_t stream) {
    TileGeom g;
    if (!make_geom(N, K, &g) || (g.units + 255) / 256 > 0x7fffffff) return hipErrorInvalidValue;
    hipLaunchKernelGGL(tile_unpack_kernel, dim3((unsigned)((g.units + 255) / 256)), dim3(256), 0, stream,
                       static_cast<const uint4*>(tiled), static_cast<uint8_t*>(w), static_cast<uint16_t*>(s),
                       static_cast<uint16_t*>(b), g);
    return hipGetLastError();
}

}  // namespace aq
