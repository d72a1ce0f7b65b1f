// Host side of the matmul path (affine_qmm and the many-row calls of affine_qmv): the context's workspace, the
// zero fill, and the choice among the tile kernel families.
//
// Replaces the selector of rocm_mlx_q4_projection_batch* (go/engine/hip/hip_projection_launch.go:5192-5287; kernels
// go/engine/hip/kernels/quant/affine_projection_tuned.hipinc:166-1109) with the semantics of MLX affine_qmm_t
// (go/engine/metal/quant_seam_backend.go:77-109, go/engine/metal/attention.go:731-751).  The kernels themselves are in
// aq_qmm_tile.hip (bf16 codes as MFMA operands, fp32 scaling of the partial products), aq_qmm_half.hip (4 bit:
// scale * (code - 8) as fp16 operands) and aq_qmm_few.hip (5..64 rows of x, K shared out over workgroups).
#include "aq_device.h"
#include "aq_kernels.h"
#include "aq_qmm.h"

#include <cstring>

#include "../../include/aq_mi355.h"

namespace aq {

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
    size_t partial = (M > 4 && M <= 64) ? qmmt_splitk_bytes(M, N, 16) : 0;
    if (M > 64 && (K / 64) % 8 == 0 && K >= 2048) {
        // 128 x 128 tiles that leave CUs idle share K out over up to 8 workgroups, at most two workgroups a CU in all
        // (qmm_dispatch): k partial tiles of M x N with (M / 128) (N / 128) k <= 2 CUs, bounded here for up to 512 CUs
        const size_t by_k = qmmt_splitk_bytes(M, N, 8), by_cus = (size_t)2 * 512 * 128 * 128 * 4 + ((size_t)M + N) * 128 * 8 * 4;
        partial = by_k < by_cus ? by_k : by_cus;
    }
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

bool qmm_takes_gate(const void* x, const void* packed, int K, int group_size, int bits) {
    return (bits == 4 || bits == 8) && (group_size == 64 || group_size == 128) && K % 64 == 0 &&
           (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(packed) & 15) == 0;
}

int qmm_dispatch(hipStream_t stream, Workspace* ws, int cu_count, int forced, const char** last_variant, const void* x,
                 const void* packed, const void* scales, const void* biases, void* y, int M, int K, int N,
                 int group_size, int bits, bool out_f32, FailFn fail, const float* gate, int act, int* x_state) {
    const bool mfma_ok = qmm_takes_gate(x, packed, K, group_size, bits);
    if (!mfma_ok) {
        if (gate) return fail(AQ_ERR_UNSUPPORTED, "aq_qmm: the gated epilogue needs the tile kernels (4 / 8 bit, groups of 64 / 128)");
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
        *last_variant = qmv_six_eligible(q, bits, group_size) ? "qmv_six" : "qmv_generic";
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
    a.gate = gate;
    a.act = act;
    const int idx = forced;
    int tile_idx = -1;
    if (idx >= 0) {
        tile_idx = idx;
        const QmmVariant* v = qmmt_variant(tile_idx);
        if (!v || v->bits != bits) return fail(AQ_ERR_ARG, "aq_qmm: forced variant %d does not fit bits=%d", idx, bits);
    } else if (idx < 0 && M >= 64) {
        // prefill sizes: the LDS-staged 128 x 128 tiles (four 64 x 64 wavefront tiles, two workgroups a CU);
        // the 128 x 64 wavefront tiles need more registers than two wavefronts a SIMD leave and measure slower
        tile_idx = find_qmmt(bits, 2, 2, 2, 2);
        // 4 bit: the kernels whose MFMA operand carries scale * (code - 8) as fp16 (half the vector instructions per
        // MFMA, no fp32 work on the accumulators) once their tiles cover enough of the chip.  A round of 256 x 256
        // tiles (eight wavefronts, twice the MFMAs per byte of x copied into LDS) takes 0.121 ms at K = 4096 however
        // few tiles it holds, a round of 256 x 128 tiles 0.094-0.107 ms, a round of up to 512 of the 128 x 128 tiles
        // 0.07-0.115 ms; measured on one box, 256 x 256 / 256 x 128 / 128 x 128 (ms): 2048 x 14336 0.277 / 0.305 / 0.32,
        // 1024 x 14336 0.139 / 0.150 / 0.196, 768 x 14336 0.125 / 0.135 / 0.158, 768 x 12288 0.122 / 0.129 / 0.148,
        // 768 x 10240 0.122 / 0.103 / 0.110, 2048 x 4096 0.126 / 0.107 / 0.117, 1536 x 4096 0.121 / 0.098 / 0.103,
        // 512 x 10240 0.121 / 0.094 / 0.094, 512 x 8192 0.121 / 0.095 / 0.071, 256 x 14336 0.120 / 0.094 / 0.067.
        // Hence: 256 x 256 from 9/16 of a tile per CU, else 256 x 128 above 5/8 of a tile per CU.
        const int cus = cu_count > 0 ? cu_count : 256;
        const int64_t mb = (M + 255) / 256;
        if (bits == 4 && mb * ((N + 255) / 256) * 16 >= (int64_t)cus * 9) {
            const int wide = find_qmmt_named("qmmh_b4_mb4_nb2_wm2_wn4");
            if (wide >= 0) tile_idx = wide;
            // 192 x 256 tiles where their rounds cost a tenth less than those of the 256 x 256 tiles (a round of them
            // takes 0.82 as long; 1536 x 14336: 0.224 against 0.256 ms, 768 x 14336: 0.117 against 0.126 ms)
            const int64_t strips = (N + 255) / 256;
            const int64_t rounds_large = (mb * strips + cus - 1) / cus, rounds_small = ((M + 191) / 192 * strips + cus - 1) / cus;
            const int narrow = find_qmmt_named("qmmh_b4_mb3_nb2_wm2_wn4");
            if (narrow >= 0 && rounds_small * 82 <= rounds_large * 90) tile_idx = narrow;
        } else if (bits == 4 && mb * ((N + 127) / 128) * 8 > (int64_t)cus * 5) {
            const int half = find_qmmt_named("qmmh_b4_mb4_nb2_wm2_wn2_s2c");
            if (half >= 0) tile_idx = half;
        }
    }
    // Few rows of x: M x N tiles alone would occupy a fraction of the chip (56 workgroups for 32 x 14336), so
    // K is shared out as well and a small kernel adds the partial tiles.
    int ksplit = 1;
    if (idx < 0 && M > 4 && M <= 64 && (K / 64) % 4 == 0) {
        // the kernels whose LDS stages hold four blocks of K: 32 or 64 rows by 256 (8 bit: 128) columns per workgroup, eight
        // (8 bit: four) wavefronts side by side
        const int bm = M <= 32 ? 32 : 64, bn = bits == 4 ? 256 : 128;
        const int want = find_qmmt_named(bits == 4 ? (M <= 32 ? "qmmf_b4_mb1_nb1_wm1_wn8" : "qmmf_b4_mb2_nb1_wm1_wn8")
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
    if (idx < 0 && M > 64 && tile_idx >= 0 && tile_idx == find_qmmt(bits, 2, 2, 2, 2) && (K / 64) % 4 == 0) {
        // 128 x 128 tiles that leave CUs idle and a long K: K shared out over up to eight workgroups per tile, two
        // workgroups a CU at most, 1024 codes of K each at least
        const int cus = cu_count > 0 ? cu_count : 256;
        const int64_t tiles = (int64_t)((M + 127) / 128) * ((N + 127) / 128);
        for (int k = 2; k <= 8; k++)
            if ((K / 64) % (4 * k) == 0 && tiles * k <= 2 * cus && (K / 64) / k >= 16) ksplit = k;
    }
    if (tile_idx < 0) {
        // fewer than 64 rows and a K that is no multiple of 256: 32 x 256 or 64 x 256 workgroup tiles
        tile_idx = M <= 32 ? find_qmmt(bits, 1, 2, 1, 4) : find_qmmt(bits, 2, 2, 1, 4);
        if (tile_idx < 0) return fail(AQ_ERR_UNSUPPORTED, "aq_qmm: no kernel variant for bits=%d", bits);
    }
    {
        const size_t xbytes = (qmmt_workspace_bytes(M, K) + 255) & ~(size_t)255;
        const uint64_t generation = ws->generation;
        if (int rc = grow_workspace(ws, xbytes + qmmt_splitk_bytes(M, N, ksplit), stream, fail)) return rc;
        // (a workspace that had to move no longer holds the earlier pass over x)
        a.x_ready = x_state && ws->generation == generation ? *x_state : kXReadyNone;
        *last_variant = qmmt_variant(tile_idx)->name;
        hipError_t rc = qmmt_launch_splitk(tile_idx, a, ws->ptr, ksplit, stream);
        if (rc != hipSuccess) return fail((int)rc, "rocm.hip.hipLaunchKernel: HIP returned %d (%s)", (int)rc, hipGetErrorString(rc));
        if (x_state) *x_state = qmmt_x_kind(tile_idx);
        return AQ_OK;
    }
}

}  // namespace aq
