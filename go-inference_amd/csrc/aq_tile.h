// Tile-major device layout of a 4-bit, group-64 affine tensor [N, K] (K a multiple of 128): what the diagonal-MFMA
// matvec kernels read fastest.  Made once at load time from the MLX layout (aq_tile_weights), inverted bit for bit
// by aq_untile_weights; the reference likewise synthesises its device layouts at load
// (go/engine/hip/hip_gguf_affine_adapter.go:199-218).
//
// The tensor is cut into sets of 16 rows (the last one padded with zero rows) and every set into steps of `cps`
// chunks of 256 codes (cps = tile_cps_for(K), the split of K the matvec kernels use; the last step may hold fewer
// chunks and the last chunk a single half of 128 codes).  One (set, step) pair is one contiguous tile:
//   1 KiB   scales and biases: 16 bytes per lane l = (n = l % 16, j = l / 16): the four bf16 scales of the groups
//           of chunk j of the step for row n, then the four biases (zeros where the row has no such group)
//   1 KiB   per half h of the step, in order: 16 bytes per lane l: bytes [64 h + 16 j, +16) of the step's codes
//           of row n (the MLX packed bytes, untouched)
// so that each load instruction of a wavefront takes 1 KiB of consecutive bytes and the 16 bytes a lane receives
// are its MFMA operand.  Every step of a set but the last has the full size, so a tile is found by multiplication.
// Size: sets * (steps * 1 KiB + halves * 1 KiB); 33 030 144 bytes for 14336 x 4096, as many as the MLX arrays.
#pragma once
#include <stdint.h>

namespace aq {

constexpr int kTileRows = 16;

// Chunks of 256 codes per step for this K: three where the even number of wavefronts that four would need holds
// them too (the heaviest wavefront then has three chunks instead of four).  A function of K alone, so that every
// launch form, and the tile-major layout, split a row the same way.
__host__ __device__ inline int tile_cps_for(int K) {
    const int chunks = (K + 255) / 256;
    const int nw4 = ((chunks + 3) / 4 + 1) & ~1;
    return (nw4 <= 4 && (chunks + 2) / 3 <= nw4) ? 3 : 4;
}
__host__ __device__ constexpr uint32_t tile_step_bytes(int cps) { return 1024u + (uint32_t)cps * 2048u; }
__host__ __device__ inline int tile_steps(int K, int cps) { return (((K >> 7) + 1) / 2 + cps - 1) / cps; }
__host__ __device__ inline uint32_t tile_set_bytes(int K, int cps) {
    return (uint32_t)tile_steps(K, cps) * 1024u + (uint32_t)(K >> 7) * 1024u;
}
// Bytes of the whole tensor in this layout, or -1 when the geometry has no tile-major form.
__host__ __device__ inline int64_t tile_total_bytes(int64_t N, int K, int group_size, int bits) {
    if (bits != 4 || group_size != 64 || K <= 0 || K % 128 != 0 || N <= 0) return -1;
    return ((N + kTileRows - 1) / kTileRows) * (int64_t)tile_set_bytes(K, tile_cps_for(K));
}

}  // namespace aq
