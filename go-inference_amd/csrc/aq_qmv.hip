// affine_qmv / gather_qmv for gfx950, M = 1..4 activation rows.
//
// Replaces rocm_mlx_q4_projection* (go/engine/hip/kernels/quant/affine_projection.hipinc:3-266,
// row body affine_dot.hipinc:524-679) and rocm_moe_mlx_affine_routes
// (go/engine/hip/kernels/moe/routing.hipinc:160-399); semantics are those of
// MLX affine_qmv / affine_gather_qmv as driven by go/engine/metal/qmv.go:354-421
// and kernels/moe/lthn_gather_qmv.metal:54-66.
//
// Shape of the computation (HBM-bound; the packed weights are read exactly once):
//   * a wavefront owns R consecutive output rows; a row's packed codes are cut
//     into "slices" of 64 x 16 bytes, so every global_load_dwordx4 of a
//     wavefront is one fully coalesced 1 KiB read (32 codes per lane at 4 bit,
//     16 at 8 bit); `DEPTH` slices are kept in flight per wavefront;
//   * the activations are staged once per workgroup into LDS as bf16 pairs in
//     the order the unpacker produces codes, and read back 64 B per lane;
//   * codes become bf16 pairs with one v_and_or_b32 per pair (4 bit) or
//     cvt_f32_ubyte + v_perm (8 bit) and feed v_dot2c_f32_bf16 (fp32 sums);
//   * per 16-byte chunk: acc += scale * dot + (bias - off*scale) * sum(x),
//     the reference's own factorisation (affine_dot.hipinc:546-573);
//   * a DPP wave reduction, then lane 0 stores bf16 (RNE) or fp32.
#include "aq_qmv_body.h"

namespace aq {

template <int BITS, int M, int R, int NW, int DEPTH, bool GATHER>
__global__ __launch_bounds__(NW* kWave) void qmv_dot2_kernel(const QmvArgs a) {
    qmv_dot2_body<BITS, M, R, NW, DEPTH, GATHER>(a, blockIdx.x);
}

// Several weight matrices against the same activations in one launch (q|k|v, gate|up): the
// workgroups of all matrices form one grid, and each looks up which matrix it belongs to.
template <int BITS, int M, int R, int NW, int DEPTH>
__global__ __launch_bounds__(NW* kWave) void qmv_dot2_multi_kernel(const QmvMultiArgs ma) {
    int set = 0;
#pragma unroll
    for (int i = 1; i < kQmvMultiMax; i++)
        if (i < ma.count && (int)blockIdx.x >= ma.block_end[i - 1]) set = i;
    QmvArgs a = ma.common;
    a.w = ma.w[set];
    a.s = ma.s[set];
    a.b = ma.b[set];
    a.y = ma.y[set];
    a.N = ma.N[set];
    qmv_dot2_body<BITS, M, R, NW, DEPTH, false>(a, (int)blockIdx.x - (set ? ma.block_end[set - 1] : 0));
}

// ---- variant table --------------------------------------------------------

typedef void (*QmvKernel)(const QmvArgs);

struct QmvEntry {
    QmvVariant v;
    QmvKernel fn;
};

// (names keep the "_x0" of the staging mode they have always had: x through LDS)
#define AQ_QMV(BITS, M, R, NW, DEPTH, G)                                                                \
    {                                                                                                   \
        {"qmv_b" #BITS "_m" #M "_r" #R "_w" #NW "_d" #DEPTH "_g" #G "_x0", BITS, M, R, NW, DEPTH, G, 0}, \
            qmv_dot2_kernel<BITS, M, R, NW, DEPTH, (G != 0)>                                            \
    }
// four wavefronts a workgroup, two slices of K in flight, 1 / 2 / 4 rows per wavefront: what the selection picks from
#define AQ_QMV_SET(BITS, M, G) AQ_QMV(BITS, M, 1, 4, 2, G), AQ_QMV(BITS, M, 2, 4, 2, G), AQ_QMV(BITS, M, 4, 4, 2, G)

static const QmvEntry kQmvTable[] = {
    AQ_QMV_SET(4, 1, 0), AQ_QMV_SET(8, 1, 0), AQ_QMV_SET(4, 1, 1), AQ_QMV_SET(8, 1, 1),
    AQ_QMV_SET(4, 2, 0), AQ_QMV_SET(4, 3, 0), AQ_QMV_SET(4, 4, 0),
    AQ_QMV_SET(8, 2, 0), AQ_QMV_SET(8, 3, 0), AQ_QMV_SET(8, 4, 0),
    AQ_QMV(8, 1, 1, 4, 4, 0),  // one row of a large 8-bit matrix: every slice of a 4096-code row in flight (4096 x 14336: 12.1 against 12.5 us)
};

int qmv_variant_count() { return (int)(sizeof(kQmvTable) / sizeof(kQmvTable[0])); }

const QmvVariant* qmv_variant(int idx) {
    if (idx < 0 || idx >= qmv_variant_count()) return nullptr;
    return &kQmvTable[idx].v;
}

size_t qmv_lds_bytes(int idx, const QmvArgs& a) {
    const QmvVariant* v = qmv_variant(idx);
    if (!v) return 0;
    return (size_t)v->m * (size_t)a.K * 2;
}

hipError_t qmv_launch(int idx, const QmvArgs& a, hipStream_t stream) {
    if (idx < 0 || idx >= qmv_variant_count()) return hipErrorInvalidValue;
    const QmvEntry& e = kQmvTable[idx];
    const int rows_per_wg = e.v.rows * e.v.waves;
    dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), e.v.gather ? (unsigned)a.routes : 1u, 1u);
    dim3 block((unsigned)(e.v.waves * kWave), 1u, 1u);
    const size_t lds = qmv_lds_bytes(idx, a);
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e.fn), (size_t)lds)) return rc;
    hipLaunchKernelGGL(e.fn, grid, block, lds, stream, a);
    return hipGetLastError();
}

typedef void (*QmvMultiKernel)(const QmvMultiArgs);
struct QmvMultiEntry {
    int bits, m, rows;
    QmvMultiKernel fn;
};
#define AQ_QMV_MULTI(BITS, M, R) {BITS, M, R, qmv_dot2_multi_kernel<BITS, M, R, 4, 2>}
static const QmvMultiEntry kQmvMultiTable[] = {
    AQ_QMV_MULTI(4, 1, 1), AQ_QMV_MULTI(4, 1, 2), AQ_QMV_MULTI(4, 1, 4), AQ_QMV_MULTI(8, 1, 1), AQ_QMV_MULTI(8, 1, 2),
    AQ_QMV_MULTI(8, 1, 4), AQ_QMV_MULTI(4, 2, 2), AQ_QMV_MULTI(4, 3, 2), AQ_QMV_MULTI(4, 4, 2), AQ_QMV_MULTI(8, 2, 2),
    AQ_QMV_MULTI(8, 3, 2), AQ_QMV_MULTI(8, 4, 2),
};

bool qmv_multi_supported(int bits, int m, int rows) {
    for (const QmvMultiEntry& e : kQmvMultiTable)
        if (e.bits == bits && e.m == m && e.rows == rows) return true;
    return false;
}

hipError_t qmv_multi_launch(int bits, int m, int rows, QmvMultiArgs ma, hipStream_t stream) {
    const QmvMultiEntry* e = nullptr;
    for (const QmvMultiEntry& c : kQmvMultiTable)
        if (c.bits == bits && c.m == m && c.rows == rows) e = &c;
    if (!e || ma.count < 1 || ma.count > kQmvMultiMax) return hipErrorInvalidValue;
    const int rows_per_wg = rows * 4;
    int blocks = 0;
    for (int i = 0; i < ma.count; i++) {
        blocks += (ma.N[i] + rows_per_wg - 1) / rows_per_wg;
        ma.block_end[i] = blocks;
    }
    const size_t lds = (size_t)m * (size_t)ma.common.K * 2;
    if (hipError_t rc = ensure_dynamic_lds(reinterpret_cast<const void*>(e->fn), (size_t)lds)) return rc;
    hipLaunchKernelGGL(e->fn, dim3((unsigned)blocks), dim3(4 * kWave), lds, stream, ma);
    return hipGetLastError();
}

}  // namespace aq
