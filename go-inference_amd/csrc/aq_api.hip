// C-ABI layer of libaq_mi355.so: context, device memory, host-side argument
// validation, kernel selection and launch.  See include/aq_mi355.h for the
// contract of each entry point and the reference interface it replaces.
#include "../../include/aq_mi355.h"
#include "../../include/aq_mi355_host.h"

#include <hip/hip_runtime.h>

#include <climits>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "aq_kernels.h"
#include "aq_qmm.h"
#include "aq_tile.h"

namespace {

thread_local std::string g_last_error;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

int hip_fail(hipError_t rc, const char* what) {
    // Same wording as the reference's driver errors (go/engine/hip/hip_driver_cgo.go:1728-1730).
    return fail((int)rc, "rocm.hip.%s: HIP returned %d (%s)", what, (int)rc, hipGetErrorString(rc));
}

#define AQ_HIP(call, what)                              \
    do {                                                \
        hipError_t rc__ = (call);                       \
        if (rc__ != hipSuccess) return hip_fail(rc__, what); \
    } while (0)

bool is_pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
int ilog2(int v) {
    int s = 0;
    while ((1 << s) < v) s++;
    return s;
}
bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace

// Scratch of aq_qmv_greedy_static, the entry point that allocates nothing: the packed best of every 16 rows
// (or of every wavefront) of the projection, then the fold's tickets and slots.  Every GPU the library runs on
// holds its own copy until the process ends; host code uses the address hipGetSymbolAddress returns for the
// current device (kept in the context), never the array's name.
constexpr size_t kStaticPartialBytes = (size_t)2 << 20;
constexpr size_t kStaticScratchBytes = kStaticPartialBytes + 1024;
static_assert(aq::kHeadFoldBytes <= 1024, "the fold area sits behind the partials");
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

struct aq_ctx {
    int device = 0;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    std::mutex mu;
    int forced[2] = {-1, -1};
    unsigned families_off = 0;  // bit per kernel family that AQ_MI355_DISABLE names: the selection skips them
    const char* last_variant[2] = {"", ""};
    int cu_count = 0;
    aq::Workspace ws;       // scratch of the matmul path and of the unfused fallbacks (aq_qmm.h)
    aq::Workspace head_ws;         // per-wavefront maxima of aq_qmv_greedy; sized at creation for common vocabularies
    void* head_fold = nullptr;     // aq_qmv_greedy's fold tickets and slots (aq::kHeadFoldBytes, kept zeroed by the kernel)
    unsigned char* static_scratch = nullptr;  // this device's copy of `scratch` (hipGetSymbolAddress at creation)
    char name[256] = {0};
};

namespace {

// Widths every path accepts (MLX affine widths the reference dispatches,
// go/model/quant_weight.go:11-13); 1-bit packs are widened to 2-bit by the
// loader (go/model/linear.go:66-84) and are rejected here.
bool width_ok(int bits) { return bits == 2 || bits == 3 || bits == 4 || bits == 5 || bits == 6 || bits == 8; }

// Mirrors validateHIPMLXAffineProjectionShape (go/engine/hip/hip_projection_reference.go:122-144)
// and MatMulQuantF32NTInto's geometry checks (go/engine/metal/quant_seam_backend.go:41-49).
int check_geometry(const char* op, int K, int group_size, int bits) {
    if (!width_ok(bits)) return fail(AQ_ERR_UNSUPPORTED, "%s: unsupported affine width %d bits", op, bits);
    if (group_size <= 0) return fail(AQ_ERR_SHAPE, "%s: group size must be positive", op);
    if (K % group_size != 0) return fail(AQ_ERR_SHAPE, "%s: cols %d must be divisible by group size %d", op, K, group_size);
    if (((int64_t)K * bits) % 32 != 0)
        return fail(AQ_ERR_SHAPE, "%s: cols*bits must be divisible by 32 for MLX affine packing", op);
    return AQ_OK;
}

// The dot2 kernels need 16-byte chunks of a row to sit inside one group and
// 128-bit aligned rows.
bool dot2_eligible(int K, int group_size, int bits, const void* x, const void* w, size_t lds_bytes) {
    if (bits != 4 && bits != 8) return false;
    if (group_size != 32 && group_size != 64 && group_size != 128) return false;
    if (((int64_t)K * bits) % 128 != 0 || K % 8 != 0) return false;
    if (!aligned(x, 16) || !aligned(w, 16)) return false;
    return lds_bytes <= 160 * 1024;
}

// Pick a dot2 variant: rows per wavefront by how many wavefronts the matrix yields, 4 wavefronts per workgroup.
int pick_qmv_variant(const aq_ctx* ctx, int bits, int m, bool gather, int N, int K, int routes) {
    const int cus = ctx->cu_count > 0 ? ctx->cu_count : 256;
    const int64_t total_rows = (int64_t)N * (gather ? routes : 1);
    int want_rows = 1;
    const int chunks = K * bits / 128;
    const int slices = (chunks + 63) / 64;
    // measured on the 256-CU part: two rows per wavefront once that still gives 8 wavefronts a CU, four
    // only for much taller matrices, one below
    for (int r : {4, 2}) {
        if (total_rows / r >= (int64_t)cus * (r == 4 ? 16 : 8) && r * slices >= 2) {
            want_rows = r;
            break;
        }
    }
    if (m > 1 && want_rows > 4) want_rows = 4;
    // one row of a large 8-bit matrix: one row per wavefront with four slices of it in flight (4096 x 14336: 12.1 us
    // against 12.5 with two rows and two slices; the arithmetic of a row, and so its bytes, are the same)
    if (bits == 8 && m == 1 && !gather && slices >= 4 && (int64_t)N * K >= ((int64_t)40 << 20))
        for (int i = 0; i < aq::qmv_variant_count(); i++) {
            const aq::QmvVariant* v = aq::qmv_variant(i);
            if (v->bits == 8 && v->m == 1 && !v->gather && v->waves == 4 && v->depth == 4 && v->rows == 1 && v->xmode == 0) return i;
        }
    int best = -1;
    for (int i = 0; i < aq::qmv_variant_count(); i++) {
        const aq::QmvVariant* v = aq::qmv_variant(i);
        if (v->bits != bits || v->m != m || (v->gather != 0) != gather) continue;
        if (v->waves != 4 || v->depth != 2 || v->xmode != 0) continue;
        if (v->rows == want_rows) return i;
        if (best < 0 || (v->rows < want_rows && v->rows > aq::qmv_variant(best)->rows)) best = i;
    }
    return best;
}

// ---- the matvec kernel families and the one table that chooses among them ---------------------------------------

// Families with variants of their own.  aq_variant_name(0, i) and aq_force_variant(ctx, 0, i) index the
// concatenation of their tables, in this order.
enum { kFamDot2, kFamBlk, kFamDiag, kFamTok, kFamCount };
// Two more take part in the selection: the tile kernels of the matmul path (their variants are those of op 1)
// and the kernel that takes any geometry.
enum { kFamTiles = kFamCount, kFamTilesLarge, kFamGeneric };

// Route switches, the counterpart of the reference's GO_ROCM_DISABLE_* variables (hip_projection_launch.go:95-137):
// AQ_MI355_DISABLE=name[,name...] over dot2, blk, diag, tok, tiles, read when a context is created, takes those
// families out of the selection of aq_qmv, aq_gather_qmv and the calls built on them, which then fall through to the
// next family that takes the shape (the any-width kernel cannot be switched off).  The fused head, gate|up and
// multi-matrix calls honour `diag` only: with it off they run their dot2 kernels, which have no switch, because the
// unfused route behind them is the selection above.  There is no code-object override like
// GO_ROCM_KERNEL_HSACO (hip_kernel_module.go:14-35): the kernels are linked into this library.
unsigned families_off_from_env(const char* value) {
    static const struct { const char* name; unsigned bits; } kNames[] = {
        {"dot2", 1u << kFamDot2}, {"blk", 1u << kFamBlk}, {"diag", 1u << kFamDiag}, {"tok", 1u << kFamTok},
        {"tiles", (1u << kFamTiles) | (1u << kFamTilesLarge)}};
    unsigned off = 0;
    if (!value) return off;
    const char* p = value;
    while (*p) {
        const char* e = p;
        while (*e && *e != ',') e++;
        for (const auto& n : kNames)
            if (strlen(n.name) == (size_t)(e - p) && strncmp(n.name, p, (size_t)(e - p)) == 0) off |= n.bits;
        p = *e ? e + 1 : e;
    }
    return off;
}

struct QmvFamily {
    int (*count)();
    const aq::QmvVariant* (*variant)(int);
};
const QmvFamily kQmvFamilies[kFamCount] = {
    {aq::qmv_variant_count, aq::qmv_variant},      // VALU dot2 kernels (aq_qmv.hip)
    {aq::qmvb_variant_count, aq::qmvb_variant},    // block-MFMA kernels (aq_qmv_blk.hip)
    {aq::qmvd_variant_count, aq::qmvd_variant},    // diagonal-MFMA kernels (aq_qmv_diag.hip)
    {aq::qmvt_variant_count, aq::qmvt_variant},    // token-tile MFMA kernels (aq_qmv_tok.hip)
};

int qmv_total_variants() {
    int n = 0;
    for (const QmvFamily& f : kQmvFamilies) n += f.count();
    return n;
}
// Family and index inside it of entry idx of the concatenated table.
bool qmv_locate(int idx, int* family, int* local) {
    if (idx < 0) return false;
    for (int f = 0; f < kFamCount; f++) {
        const int n = kQmvFamilies[f].count();
        if (idx < n) {
            *family = f;
            *local = idx;
            return true;
        }
        idx -= n;
    }
    return false;
}
const aq::QmvVariant* qmv_any_variant(int idx) {
    int f, i;
    return qmv_locate(idx, &f, &i) ? kQmvFamilies[f].variant(i) : nullptr;
}

// Which family runs an unforced call.  The first rule whose key matches the call and whose family accepts the shape
// runs it; the key holds what the families differ in at first sight (code width, group size, rows of x, dense or
// gathered), and each family's own pick / fits / plan function narrows K, N and operand alignment and passes the call
// on when the shape is not its to run.  The last rule of each kind accepts everything.
struct QmvRule {
    int bits;        // 0: any
    int group_size;  // 0: any
    int gather;      // 1: gathered calls (one row of x per route), 0: dense calls
    int m_lo, m_hi;  // rows of x in the call
    int family;
};
const QmvRule kQmvRules[] = {
    // bits group gather rows         family
    {4, 64, 1, 1, 1, kFamDiag},             // K a multiple of 128 in 2..8 steps of 1024 codes
    {0, 0, 1, 1, 1, kFamDot2},              // 4 / 8 bit, groups of 32 / 64 / 128, 16-byte chunks inside one group
    {0, 0, 1, 1, 1, kFamGeneric},
    {4, 64, 0, 1, 8, kFamDiag},             // K from 1152 to 16384: up to 8 rows in one launch at 2..4 steps of 1024 codes,
                                            // up to 4 per launch at longer K; every row of such a call has the bytes of a
                                            // call with that row alone
    {4, 64, 0, 2, 8, kFamDot2},             // K the diagonal kernels do not take (up to 1024, no multiple of 128, beyond
                                            // 16384): the kernel a single row of such a K runs on, four rows a launch, so
                                            // that rows keep the bytes of single-row calls here too
    {4, 32, 0, 1, 2, kFamDiag},             // groups of 32: two tokens x eight groups as MFMA rows
    {8, 64, 0, 1, 4, kFamDiag},             // up to four rows of 8-bit codes, K of 2048, 4096 or 8192, up to 40 Mi codes (where
                                            // measured ahead of the next two rules, see qmvd_pick); a row of such a call
                                            // has the bytes of a call with that row alone
    {8, 0, 0, 1, 1, kFamDot2},              // one row of 8-bit codes: the dot2 kernel with its non-temporal loads, 12.4 us for
                                            // 4096 x 14336 (63 % of the HBM peak) against 14.2 us on the block-MFMA kernel
    {8, 64, 0, 2, 32, kFamTok},             // K a multiple of 256 up to 16384: one launch, weights streamed once, no scratch
                                            // (4 rows of 4096 x 14336: 14.3 us against 15.0 on the block-MFMA kernels, 21.5 on
                                            // the dot2 kernels; the reference states its rows-equal-single-rows contract for
                                            // 4-bit codes only, qmv_rows_test.go:36-41)
    {4, 64, 0, 5, 32, kFamTok},             // the same for 4-bit codes, up to 32 rows
                                            // (5..8 rows get here only when the two rules that keep the bytes of single-row
                                            // calls have passed, e.g. on operands that are not 16-byte aligned, or with the
                                            // diagonal and dot2 families switched off: this kernel is faster at long K,
                                            // 15.6 against 2 x 9 us at 8 rows of 14336 x 4096, but not row by row the same bytes)
    {0, 0, 0, 9, 64, kFamTilesLarge},       // 16 Mi codes and more: the 16-row block-MFMA kernel is bound by its 4x4x4 MFMAs
    {0, 0, 0, 2, 16, kFamBlk},              // the whole call in one launch of up to 16 rows (4 where K is long)
    {8, 0, 0, 1, 1, kFamBlk},               // (a single row of 4-bit codes is faster on the dot2 kernels)
    {0, 0, 0, 5, INT32_MAX, kFamTiles},     // K shared out over workgroups for few rows; any geometry
    {0, 0, 0, 1, 4, kFamDot2},
    {0, 0, 0, 1, INT32_MAX, kFamGeneric},   // beyond four rows only when the tile kernels are switched off
};

constexpr int kPass = INT32_MIN;  // a family's answer when the shape is not its to run

int run_dot2(aq_ctx* ctx, const aq::QmvArgs& a, int group_size, int bits, bool gather, int forced) {
    const int M = a.M;
    if (!dot2_eligible(a.K, group_size, bits, a.x, a.w, (size_t)(M < 4 ? M : 4) * a.K * 2)) return kPass;
    const size_t esize = a.out_f32 ? 4 : 2;
    for (int m0 = 0; m0 < M;) {
        int m = M - m0 < 4 ? M - m0 : 4;
        int idx = forced;
        if (idx >= 0) {
            const aq::QmvVariant* v = aq::qmv_variant(idx);
            if (!v || v->bits != bits || (v->gather != 0) != gather || v->m > M - m0) return kPass;
            m = v->m;
        } else {
            idx = pick_qmv_variant(ctx, bits, m, gather, a.N, a.K, a.routes);
            if (idx < 0) return kPass;
        }
        aq::QmvArgs c = a;
        c.M = m;
        c.x = a.x + (size_t)m0 * a.K;
        c.y = static_cast<char*>(a.y) + (size_t)m0 * a.N * esize;
        ctx->last_variant[0] = aq::qmv_variant(idx)->name;
        AQ_HIP(aq::qmv_launch(idx, c, ctx->stream), "hipLaunchKernel");
        m0 += m;
    }
    return AQ_OK;
}

int run_blk(aq_ctx* ctx, const aq::QmvArgs& a, int group_size, int bits, bool gather, int forced) {
    aq::BlkPlan plan;
    if (!aq::qmvb_plan(a, bits, group_size, gather, ctx->cu_count, forced, &plan)) return kPass;
    ctx->last_variant[0] = aq::qmvb_variant(plan.idx)->name;
    AQ_HIP(aq::qmvb_launch(plan, a, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int run_diag(aq_ctx* ctx, const aq::QmvArgs& a, int group_size, int bits, bool gather, int forced) {
    const int di = forced >= 0        ? forced
                   : gather           ? aq::qmvd_pick_gather(a.K)
                   : group_size == 32 ? aq::qmvd_pick_g32(a.M, a.K, a.N)
                                      : aq::qmvd_pick(a.M, a.K, a.N, bits);
    if (di >= 0 && aq::qmvd_fits(a, bits, group_size, gather, di)) {
        ctx->last_variant[0] = aq::qmvd_variant(di)->name;
        AQ_HIP(aq::qmvd_launch(di, a, ctx->stream), "hipLaunchKernel");
        return AQ_OK;
    }
    // Five to eight rows of a K that one launch takes for up to four: two launches.  Every row of a call has the bytes
    // of a call with that row alone (go/engine/metal/qmv_rows.go:14-24), which the other families do not give.
    if (forced < 0 && !gather && group_size == 64 && bits == 4 && a.M > 4 && a.M <= 8) {
        const int d4 = aq::qmvd_pick(4, a.K, a.N);
        aq::QmvArgs part = a;
        part.M = 4;
        if (d4 >= 0 && aq::qmvd_fits(part, bits, group_size, false, d4)) {
            const size_t esize = a.out_f32 ? 4 : 2;
            for (int m0 = 0; m0 < a.M; m0 += 4) {
                part.M = a.M - m0 < 4 ? a.M - m0 : 4;
                part.x = a.x + (size_t)m0 * a.K;
                part.y = static_cast<char*>(a.y) + (size_t)m0 * a.N * esize;
                const int dp = aq::qmvd_pick(part.M, a.K, a.N);
                if (dp < 0 || !aq::qmvd_fits(part, bits, group_size, false, dp)) return kPass;
                ctx->last_variant[0] = aq::qmvd_variant(dp)->name;
                AQ_HIP(aq::qmvd_launch(dp, part, ctx->stream), "hipLaunchKernel");
            }
            return AQ_OK;
        }
    }
    return kPass;
}

int run_tok(aq_ctx* ctx, const aq::QmvArgs& a, int group_size, int bits, bool gather, int forced) {
    const int ti = forced >= 0 ? forced : aq::qmvt_pick(bits, a.M, a.K, a.N, ctx->cu_count);
    if (gather || ti < 0 || !aq::qmvt_fits(a, bits, group_size, ti)) return kPass;
    ctx->last_variant[0] = aq::qmvt_variant(ti)->name;
    AQ_HIP(aq::qmvt_launch(ti, a, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int run_tiles(aq_ctx* ctx, const aq::QmvArgs& a, int group_size, int bits, bool large_only) {
    if (large_only && ((a.K / 64) % 4 != 0 || (int64_t)a.N * a.K < (int64_t)16 << 20)) return kPass;
    const int rc = aq::qmm_dispatch(ctx->stream, &ctx->ws, ctx->cu_count, ctx->forced[1], &ctx->last_variant[1], a.x, a.w,
                                    a.s, a.b, a.y, a.M, a.K, a.N, group_size, bits, a.out_f32 != 0, fail);
    if (rc == AQ_OK) ctx->last_variant[0] = ctx->last_variant[1];  // the kernel this matvec call ran
    return rc;
}

int run_generic(aq_ctx* ctx, const aq::QmvArgs& a, int group_size, int bits, bool gather) {
    ctx->last_variant[0] = aq::qmv_six_eligible(a, bits, group_size) ? "qmv_six" : "qmv_generic";
    AQ_HIP(aq::qmv_generic_launch(a, bits, group_size, gather, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int run_family(int family, aq_ctx* ctx, const aq::QmvArgs& a, int group_size, int bits, bool gather, int forced) {
    switch (family) {
        case kFamDot2: return run_dot2(ctx, a, group_size, bits, gather, forced);
        case kFamBlk: return run_blk(ctx, a, group_size, bits, gather, forced);
        case kFamDiag: return run_diag(ctx, a, group_size, bits, gather, forced);
        case kFamTok: return run_tok(ctx, a, group_size, bits, gather, forced);
        case kFamTiles: return run_tiles(ctx, a, group_size, bits, false);
        case kFamTilesLarge: return run_tiles(ctx, a, group_size, bits, true);
        default: return run_generic(ctx, a, group_size, bits, gather);
    }
}

// One matvec call, dense (a.M rows of x) or gathered (one row per route): the forced variant, or the rule table.
int launch_qmv_rows(aq_ctx* ctx, aq::QmvArgs a, int group_size, int bits, bool gather) {
    a.gs_shift = is_pow2(group_size) ? ilog2(group_size) : 0;
    const int forced = ctx->forced[0];
    if (forced >= 0) {
        int family = 0, local = 0;
        const int rc = qmv_locate(forced, &family, &local) ? run_family(family, ctx, a, group_size, bits, gather, local) : kPass;
        if (rc == kPass)
            return fail(AQ_ERR_ARG, "aq_qmv: forced variant %d does not fit bits=%d group=%d gather=%d rows=%d K=%d N=%d",
                        forced, bits, group_size, (int)gather, a.M, a.K, a.N);
        return rc;
    }
    for (const QmvRule& r : kQmvRules) {
        if ((r.bits && r.bits != bits) || (r.group_size && r.group_size != group_size) || (r.gather != 0) != gather ||
            a.M < r.m_lo || a.M > r.m_hi || (ctx->families_off >> r.family & 1))
            continue;
        const int rc = run_family(r.family, ctx, a, group_size, bits, gather, -1);
        if (rc != kPass) return rc;
    }
    return fail(AQ_ERR_UNSUPPORTED, "aq_qmv: no kernel for bits=%d group=%d rows=%d K=%d N=%d", bits, group_size, a.M, a.K, a.N);
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// The MLX arrays of a tile-major tensor, written into the context's workspace at byte offset `base` (which the
// caller has reserved up to base + untiled_bytes(N, K)): the route of calls that no tile-major kernel takes.
size_t untiled_bytes(int64_t N, int K) { return align256((size_t)N * (K / 2)) + 2 * align256((size_t)N * (K / 64) * 2); }
int untile_into_ws(aq_ctx* ctx, size_t base, const void* tiled, int64_t N, int K, const uint32_t** w, const uint16_t** s,
                   const uint16_t** b) {
    char* p = static_cast<char*>(ctx->ws.ptr) + base;
    char* ps = p + align256((size_t)N * (K / 2));
    char* pb = ps + align256((size_t)N * (K / 64) * 2);
    AQ_HIP(aq::tile_unpack_launch(tiled, p, ps, pb, N, K, ctx->stream), "hipLaunchKernel");
    *w = reinterpret_cast<const uint32_t*>(p);
    *s = reinterpret_cast<const uint16_t*>(ps);
    *b = reinterpret_cast<const uint16_t*>(pb);
    return AQ_OK;
}

// A dense matvec call whose weights are in the tile-major layout (a.w; a.s and a.b unset): the diagonal-MFMA
// kernels read it as it lies; any other kernel gets the MLX arrays rebuilt in the workspace first.
int launch_qmv_tiled(aq_ctx* ctx, aq::QmvArgs a, int group_size, int bits) {
    a.gs_shift = ilog2(group_size);
    a.tiled = 1;
    int family = -1, local = -1;
    const int forced = ctx->forced[0];
    if (forced >= 0 && !qmv_locate(forced, &family, &local)) return fail(AQ_ERR_ARG, "aq_qmv: forced variant %d does not exist", forced);
    if (forced >= 0 ? family == kFamDiag : !(ctx->families_off >> kFamDiag & 1)) {
        const int rc = run_diag(ctx, a, group_size, bits, false, forced >= 0 ? local : -1);
        if (rc != kPass) return rc;
        if (forced >= 0)
            return fail(AQ_ERR_ARG, "aq_qmv: forced variant %d does not fit tile-major weights with rows=%d K=%d N=%d", forced, a.M,
                        a.K, a.N);
    }
    const size_t region = aq::qmm_scratch_bytes(a.M, a.K, a.N);
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, region + untiled_bytes(a.N, a.K), fail)) return rc;
    if (int rc = untile_into_ws(ctx, region, a.w, a.N, a.K, &a.w, &a.s, &a.b)) return rc;
    a.tiled = 0;
    return launch_qmv_rows(ctx, a, group_size, bits, false);
}

}  // namespace

namespace {
// Scoped device allocations for the host-slice entry points.
struct DevBuf {
    void* p = nullptr;
    ~DevBuf() {
        if (p) (void)hipFree(p);
    }
    hipError_t alloc(size_t n) { return hipMalloc(&p, n ? n : 1); }
};
}  // namespace

extern "C" {

const char* aq_version(void) { return "aq_mi355 0.1 (gfx950)"; }
const char* aq_last_error(void) { return g_last_error.c_str(); }

int aq_create(int device, aq_ctx** out) {
    if (!out) return fail(AQ_ERR_ARG, "aq_create: out is null");
    *out = nullptr;
    int count = 0;
    hipError_t rc = hipGetDeviceCount(&count);
    if (rc != hipSuccess || count <= 0) return fail(AQ_ERR_NODEVICE, "aq_create: no HIP device available");
    if (device < 0 || device >= count) return fail(AQ_ERR_ARG, "aq_create: device %d out of range (have %d)", device, count);
    AQ_HIP(hipSetDevice(device), "hipSetDevice");
    hipDeviceProp_t prop;
    AQ_HIP(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties");
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(AQ_ERR_NODEVICE, "aq_create: device %d is %s; this library carries gfx950 code only", device,
                    prop.gcnArchName);
    aq_ctx* ctx = new (std::nothrow) aq_ctx();
    if (!ctx) return fail(AQ_ERR_NOMEM, "aq_create: out of host memory");
    ctx->device = device;
    ctx->cu_count = prop.multiProcessorCount;
    ctx->families_off = families_off_from_env(getenv("AQ_MI355_DISABLE"));
    // what the runtime reports, unchanged; a host that reports no marketing name shows the architecture instead
    char arch_only[80];
    snprintf(arch_only, sizeof arch_only, "%.*s device (no name reported)", (int)strcspn(prop.gcnArchName, ":"), prop.gcnArchName);
    snprintf(ctx->name, sizeof ctx->name, "%s (%s, %d CUs, %d MHz)", prop.name[0] ? prop.name : arch_only, prop.gcnArchName,
             prop.multiProcessorCount, prop.clockRate / 1000);
    rc = hipStreamCreateWithFlags(&ctx->own_stream, hipStreamNonBlocking);
    if (rc == hipSuccess) rc = hipEventCreate(&ctx->ev0);
    if (rc == hipSuccess) rc = hipEventCreate(&ctx->ev1);
    if (rc == hipSuccess) rc = hipMalloc(&ctx->head_fold, aq::kHeadFoldBytes);
    if (rc == hipSuccess) rc = hipMemset(ctx->head_fold, 0, aq::kHeadFoldBytes);
    if (rc == hipSuccess) {
        // room for the argmax partials of a 1M-row vocabulary at two rows per wavefront
        rc = hipMalloc(&ctx->head_ws.ptr, (size_t)4 << 20);
        if (rc == hipSuccess) ctx->head_ws.bytes = (size_t)4 << 20;
    }
    if (rc != hipSuccess) {
        aq_destroy(ctx);
        return hip_fail(rc, "hipStreamCreate");
    }
    // the device is current (hipSetDevice above): this is its own copy of the array
    rc = hipGetSymbolAddress(reinterpret_cast<void**>(&ctx->static_scratch), HIP_SYMBOL(scratch));
    if (rc != hipSuccess || !ctx->static_scratch) {
        aq_destroy(ctx);
        return hip_fail(rc != hipSuccess ? rc : hipErrorInvalidSymbol, "hipGetSymbolAddress");
    }
    ctx->stream = ctx->own_stream;
    *out = ctx;
    return AQ_OK;
}

void aq_destroy(aq_ctx* ctx) {
    if (!ctx) return;
    if (ctx->own_stream) {
        (void)hipStreamSynchronize(ctx->own_stream);
        (void)hipStreamDestroy(ctx->own_stream);
    }
    if (ctx->ws.ptr) (void)hipFree(ctx->ws.ptr);
    if (ctx->head_ws.ptr) (void)hipFree(ctx->head_ws.ptr);
    if (ctx->head_fold) (void)hipFree(ctx->head_fold);
    if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
    if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
    delete ctx;
}

int aq_use_stream(aq_ctx* ctx, void* hip_stream) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_use_stream: ctx is null");
    std::lock_guard<std::mutex> lk(ctx->mu);
    ctx->stream = static_cast<hipStream_t>(hip_stream);
    return AQ_OK;
}

int aq_use_own_stream(aq_ctx* ctx) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_use_own_stream: ctx is null");
    std::lock_guard<std::mutex> lk(ctx->mu);
    ctx->stream = ctx->own_stream;
    return AQ_OK;
}

int aq_device_name(aq_ctx* ctx, char* buf, size_t buf_len) {
    if (!ctx || !buf || buf_len == 0) return fail(AQ_ERR_ARG, "aq_device_name: bad argument");
    snprintf(buf, buf_len, "%s", ctx->name);
    return AQ_OK;
}

int aq_malloc(aq_ctx* ctx, size_t bytes, void** dptr) {
    if (!ctx || !dptr) return fail(AQ_ERR_ARG, "aq_malloc: bad argument");
    *dptr = nullptr;
    if (bytes == 0) return AQ_OK;
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    AQ_HIP(hipMalloc(dptr, bytes), "hipMalloc");
    return AQ_OK;
}

int aq_free(aq_ctx* ctx, void* dptr) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_free: ctx is null");
    if (!dptr) return AQ_OK;
    AQ_HIP(hipFree(dptr), "hipFree");
    return AQ_OK;
}

int aq_h2d(aq_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes) {
    if (!ctx || (bytes && (!dst_dev || !src_host))) return fail(AQ_ERR_ARG, "aq_h2d: bad argument");
    if (!bytes) return AQ_OK;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream), "hipMemcpyHtoD");
    AQ_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    return AQ_OK;
}

int aq_d2h(aq_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes) {
    if (!ctx || (bytes && (!dst_host || !src_dev))) return fail(AQ_ERR_ARG, "aq_d2h: bad argument");
    if (!bytes) return AQ_OK;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream), "hipMemcpyDtoH");
    AQ_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    return AQ_OK;
}

int aq_d2d(aq_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes) {
    if (!ctx || (bytes && (!dst_dev || !src_dev))) return fail(AQ_ERR_ARG, "aq_d2d: bad argument");
    if (!bytes) return AQ_OK;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream), "hipMemcpyDtoD");
    return AQ_OK;
}

int aq_fill_zero(aq_ctx* ctx, void* dptr, size_t bytes) {
    if (!ctx || (bytes && !dptr)) return fail(AQ_ERR_ARG, "aq_fill_zero: bad argument");
    if (!bytes) return AQ_OK;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::fill_zero_launch(dptr, bytes, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int aq_sync(aq_ctx* ctx) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_sync: ctx is null");
    AQ_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    return AQ_OK;
}

int aq_timer_start(aq_ctx* ctx) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_timer_start: ctx is null");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipEventRecord(ctx->ev0, ctx->stream), "hipEventRecord");
    return AQ_OK;
}

int aq_timer_stop(aq_ctx* ctx, float* elapsed_ms) {
    if (!ctx || !elapsed_ms) return fail(AQ_ERR_ARG, "aq_timer_stop: bad argument");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipEventRecord(ctx->ev1, ctx->stream), "hipEventRecord");
    AQ_HIP(hipEventSynchronize(ctx->ev1), "hipEventSynchronize");
    AQ_HIP(hipEventElapsedTime(elapsed_ms, ctx->ev0, ctx->ev1), "hipEventElapsedTime");
    return AQ_OK;
}

struct aq_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    // the context workspaces whose addresses the captured kernels carry, and the generation they were captured under
    bool uses_ws = false, uses_head_ws = false;
    uint64_t ws_generation = 0, head_ws_generation = 0;
};

int aq_capture_begin(aq_ctx* ctx) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_capture_begin: ctx is null");
    std::lock_guard<std::mutex> lk(ctx->mu);
    if (ctx->stream == nullptr) return fail(AQ_ERR_UNSUPPORTED, "aq_capture_begin: the legacy default stream cannot be captured");
    AQ_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
    ctx->ws.touched = ctx->head_ws.touched = false;
    return AQ_OK;
}

int aq_capture_end(aq_ctx* ctx, aq_graph** out) {
    if (!ctx || !out) return fail(AQ_ERR_ARG, "aq_capture_end: bad argument");
    *out = nullptr;
    std::lock_guard<std::mutex> lk(ctx->mu);
    hipGraph_t g = nullptr;
    AQ_HIP(hipStreamEndCapture(ctx->stream, &g), "hipStreamEndCapture");
    aq_graph* ag = new (std::nothrow) aq_graph();
    if (!ag) {
        (void)hipGraphDestroy(g);
        return fail(AQ_ERR_NOMEM, "aq_capture_end: out of host memory");
    }
    ag->graph = g;
    ag->uses_ws = ctx->ws.touched;
    ag->uses_head_ws = ctx->head_ws.touched;
    ag->ws_generation = ctx->ws.generation;
    ag->head_ws_generation = ctx->head_ws.generation;
    hipError_t rc = hipGraphInstantiate(&ag->exec, g, nullptr, nullptr, 0);
    if (rc != hipSuccess) {
        aq_graph_destroy(ag);
        return hip_fail(rc, "hipGraphInstantiate");
    }
    *out = ag;
    return AQ_OK;
}

int aq_graph_launch(aq_ctx* ctx, aq_graph* graph) {
    if (!ctx || !graph || !graph->exec) return fail(AQ_ERR_ARG, "aq_graph_launch: bad argument");
    std::lock_guard<std::mutex> lk(ctx->mu);
    if ((graph->uses_ws && graph->ws_generation != ctx->ws.generation) ||
        (graph->uses_head_ws && graph->head_ws_generation != ctx->head_ws.generation))
        return fail(AQ_ERR_UNSUPPORTED,
                    "aq_graph_launch: the context's workspace was reallocated after this graph was captured (a later call "
                    "needed more room); the graph's kernels still point at the freed block: capture it again, and reserve "
                    "the largest workspace first (aq_reserve_workspace / aq_reserve_workspace_bytes)");
    AQ_HIP(hipGraphLaunch(graph->exec, ctx->stream), "hipGraphLaunch");
    return AQ_OK;
}

void aq_graph_destroy(aq_graph* graph) {
    if (!graph) return;
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
}

int aq_probe_read(aq_ctx* ctx, const void* packed, const void* scales, const void* biases, int K, int N, int mode) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_probe_read: ctx is null");
    if (K <= 0 || N <= 0 || K % 1024 != 0) return fail(AQ_ERR_SHAPE, "aq_probe_read: K must be a positive multiple of 1024, N positive");
    if (mode < 0 || mode > 3) return fail(AQ_ERR_ARG, "aq_probe_read: mode is 0..3");
    if (!packed || (mode != 2 && (!scales || !biases))) return fail(AQ_ERR_ARG, "aq_probe_read: null operand");
    if (!aligned(packed, 16) || !aligned(scales, 8) || !aligned(biases, 8))
        return fail(AQ_ERR_ARG, "aq_probe_read: packed must be 16-byte, scales and biases 8-byte aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::read_probe_launch(packed, scales, biases, N, K / 2, K / 32, mode, nullptr, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int aq_qmv(aq_ctx* ctx, const void* x, const void* packed, const void* scales, const void* biases, void* y, int M,
           int K, int N, int group_size, int bits, unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_qmv: ctx is null");
    if (M < 0 || K < 0 || N < 0) return fail(AQ_ERR_SHAPE, "aq_qmv: M, K, N must be non-negative");
    if (M == 0 || N == 0 || K == 0) return AQ_OK;
    if (int rc = check_geometry("aq_qmv", K, group_size, bits)) return rc;
    const bool tiled = (flags & AQ_W_TILED) != 0;
    if (tiled) {
        if (aq::tile_total_bytes(N, K, group_size, bits) < 0)
            return fail(AQ_ERR_UNSUPPORTED, "aq_qmv: no tile-major layout for bits=%d group=%d K=%d", bits, group_size, K);
        if (!aligned(packed, 16)) return fail(AQ_ERR_ARG, "aq_qmv: a tile-major tensor is 16-byte aligned");
        scales = biases = nullptr;
    }
    if (!x || !packed || (!tiled && (!scales || !biases)) || !y) return fail(AQ_ERR_ARG, "aq_qmv: null operand");
    if (!aligned(x, 2) || !aligned(packed, 4) || !aligned(scales, 2) || !aligned(biases, 2) || !aligned(y, 2))
        return fail(AQ_ERR_ARG, "aq_qmv: operand pointer is not element-aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    aq::QmvArgs a{};
    a.x = static_cast<const uint16_t*>(x);
    a.w = static_cast<const uint32_t*>(packed);
    a.s = static_cast<const uint16_t*>(scales);
    a.b = static_cast<const uint16_t*>(biases);
    a.y = y;
    a.K = K;
    a.N = N;
    a.M = M;
    a.out_f32 = (flags & AQ_OUT_F32) ? 1 : 0;
    a.routes = 1;
    if (tiled) return launch_qmv_tiled(ctx, a, group_size, bits);
    return launch_qmv_rows(ctx, a, group_size, bits, false);
}

int aq_qmv_multi(aq_ctx* ctx, const void* x, int count, const void* const* packed, const void* const* scales,
                 const void* const* biases, void* const* y, const int* N, int M, int K, int group_size, int bits,
                 unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_qmv_multi: ctx is null");
    if (count < 0 || count > aq::kQmvMultiMax) return fail(AQ_ERR_ARG, "aq_qmv_multi: count must be 0..%d", aq::kQmvMultiMax);
    if (count == 0) return AQ_OK;
    if (!packed || !y || !N) return fail(AQ_ERR_ARG, "aq_qmv_multi: null array");
    if (M < 0 || K < 0) return fail(AQ_ERR_SHAPE, "aq_qmv_multi: M, K must be non-negative");
    bool fused = M >= 1 && M <= 4 && K > 0 && bits == 4 && ctx->forced[0] < 0;
    const bool tiled = (flags & AQ_W_TILED) != 0;  // every member is a tile-major tensor; scales and biases are not read
    if (!tiled && (!scales || !biases)) return fail(AQ_ERR_ARG, "aq_qmv_multi: null array");
    const void* const kNoArrays[aq::kQmvMultiMax] = {nullptr, nullptr, nullptr, nullptr};
    if (tiled) scales = biases = kNoArrays;
    for (int i = 0; i < count; i++) {
        if (N[i] < 0) return fail(AQ_ERR_SHAPE, "aq_qmv_multi: N[%d] must be non-negative", i);
        if (N[i] == 0) fused = false;  // an empty member: leave the bookkeeping to aq_qmv
        if (N[i] > 0 && K > 0 && M > 0 && (!packed[i] || (!tiled && (!scales[i] || !biases[i])) || !y[i]))
            return fail(AQ_ERR_ARG, "aq_qmv_multi: null operand in member %d", i);
        if (tiled && N[i] > 0 && K > 0 && M > 0 && (aq::tile_total_bytes(N[i], K, group_size, bits) < 0 || !aligned(packed[i], 16)))
            fused = false;  // aq_qmv names the problem
    }
    if (fused) {
        if (int rc = check_geometry("aq_qmv_multi", K, group_size, bits)) return rc;
        if (!x) return fail(AQ_ERR_ARG, "aq_qmv_multi: null operand");
        int64_t total = 0;
        for (int i = 0; i < count; i++) {
            total += N[i];
            fused = fused && dot2_eligible(K, group_size, bits, x, packed[i], (size_t)K * 2) && aligned(scales[i], 2) &&
                    aligned(biases[i], 2) && aligned(y[i], 2);
        }
        fused = fused && total < (int64_t)1 << 30;
        if (fused) {
            std::lock_guard<std::mutex> lk(ctx->mu);
            // the kernels aq_qmv would pick for each member, in one grid
            // (every variant with the same split of K computes the same bytes, whatever the rows per workgroup)
            const int di = (ctx->families_off >> kFamDiag & 1) ? -1 : aq::qmvd_pick(M, K, (int)total);
            if (di >= 0 && aq::qmvd_multi_supported(di)) {
                bool fits = true;
                aq::QmvMultiArgs ma{};
                ma.common.x = static_cast<const uint16_t*>(x);
                ma.common.K = K;
                ma.common.M = M;
                ma.common.gs_shift = ilog2(group_size);
                ma.common.out_f32 = (flags & AQ_OUT_F32) ? 1 : 0;
                ma.common.routes = 1;
                ma.common.tiled = tiled ? 1 : 0;
                ma.count = count;
                for (int i = 0; i < count; i++) {
                    ma.w[i] = static_cast<const uint32_t*>(packed[i]);
                    ma.s[i] = static_cast<const uint16_t*>(scales[i]);
                    ma.b[i] = static_cast<const uint16_t*>(biases[i]);
                    ma.y[i] = y[i];
                    ma.N[i] = N[i];
                    aq::QmvArgs one = ma.common;
                    one.w = ma.w[i];
                    one.s = ma.s[i];
                    one.b = ma.b[i];
                    one.y = y[i];
                    one.N = N[i];
                    fits = fits && aq::qmvd_fits(one, bits, group_size, false, di);
                }
                if (fits) {
                    ctx->last_variant[0] = "qmv_multi_diag";
                    AQ_HIP(aq::qmvd_multi_launch(di, ma, ctx->stream), "hipLaunchKernel");
                    return AQ_OK;
                }
            }
            const int idx = M == 1 && !tiled ? pick_qmv_variant(ctx, bits, 1, false, (int)total, K, 1) : -1;
            const int rows = idx >= 0 ? aq::qmv_variant(idx)->rows : 0;
            if (rows > 0 && aq::qmv_multi_supported(bits, 1, rows)) {
                aq::QmvMultiArgs ma{};
                ma.common.x = static_cast<const uint16_t*>(x);
                ma.common.K = K;
                ma.common.M = 1;
                ma.common.gs_shift = ilog2(group_size);
                ma.common.out_f32 = (flags & AQ_OUT_F32) ? 1 : 0;
                ma.common.routes = 1;
                ma.count = count;
                for (int i = 0; i < count; i++) {
                    ma.w[i] = static_cast<const uint32_t*>(packed[i]);
                    ma.s[i] = static_cast<const uint16_t*>(scales[i]);
                    ma.b[i] = static_cast<const uint16_t*>(biases[i]);
                    ma.y[i] = y[i];
                    ma.N[i] = N[i];
                }
                ctx->last_variant[0] = "qmv_multi_dot2";
                AQ_HIP(aq::qmv_multi_launch(bits, 1, rows, ma, ctx->stream), "hipLaunchKernel");
                return AQ_OK;
            }
        }
    }
    for (int i = 0; i < count; i++)
        if (int rc = aq_qmv(ctx, x, packed[i], scales[i], biases[i], y[i], M, K, N[i], group_size, bits, flags)) return rc;
    return AQ_OK;
}

int aq_qmm(aq_ctx* ctx, const void* x, const void* packed, const void* scales, const void* biases, void* y, int M,
           int K, int N, int group_size, int bits, unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_qmm: ctx is null");
    // go/engine/metal/quant_seam_backend.go:41-43: the matmul seam rejects non-positive dims.
    if (M <= 0 || K <= 0 || N <= 0) return fail(AQ_ERR_SHAPE, "aq_qmm: M, N, K must be positive");
    if (int rc = check_geometry("aq_qmm", K, group_size, bits)) return rc;
    if (!x || !packed || !scales || !biases || !y) return fail(AQ_ERR_ARG, "aq_qmm: null operand");
    if (!aligned(x, 2) || !aligned(packed, 4) || !aligned(scales, 2) || !aligned(biases, 2) || !aligned(y, 2))
        return fail(AQ_ERR_ARG, "aq_qmm: operand pointer is not element-aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    if (M <= aq::kQmvMaxRows && ctx->forced[1] < 0) {
        // a matmul of up to four rows is a matvec: the matvec selection runs it (no pass over x, no workspace)
        aq::QmvArgs a{};
        a.x = static_cast<const uint16_t*>(x);
        a.w = static_cast<const uint32_t*>(packed);
        a.s = static_cast<const uint16_t*>(scales);
        a.b = static_cast<const uint16_t*>(biases);
        a.y = y;
        a.K = K;
        a.N = N;
        a.M = M;
        a.out_f32 = (flags & AQ_OUT_F32) ? 1 : 0;
        a.routes = 1;
        const int rc = launch_qmv_rows(ctx, a, group_size, bits, false);
        if (rc == AQ_OK) ctx->last_variant[1] = ctx->last_variant[0];
        return rc;
    }
    return aq::qmm_dispatch(ctx->stream, &ctx->ws, ctx->cu_count, ctx->forced[1], &ctx->last_variant[1], x, packed, scales,
                            biases, y, M, K, N, group_size, bits, (flags & AQ_OUT_F32) != 0, fail);
}

int aq_qmm_multi(aq_ctx* ctx, const void* x, int count, const void* const* packed, const void* const* scales,
                 const void* const* biases, void* const* y, const int* N, int M, int K, int group_size, int bits,
                 unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_qmm_multi: ctx is null");
    if (count < 1 || count > 8) return fail(AQ_ERR_ARG, "aq_qmm_multi: count must be 1..8");
    if (!packed || !scales || !biases || !y || !N) return fail(AQ_ERR_ARG, "aq_qmm_multi: null array");
    if (M <= 0 || K <= 0) return fail(AQ_ERR_SHAPE, "aq_qmm_multi: M, N, K must be positive");
    if (int rc = check_geometry("aq_qmm_multi", K, group_size, bits)) return rc;
    if (!x || !aligned(x, 2)) return fail(AQ_ERR_ARG, "aq_qmm_multi: null or misaligned x");
    size_t need = 0;
    for (int i = 0; i < count; i++) {
        if (N[i] <= 0) return fail(AQ_ERR_SHAPE, "aq_qmm_multi: M, N, K must be positive");
        if (!packed[i] || !scales[i] || !biases[i] || !y[i]) return fail(AQ_ERR_ARG, "aq_qmm_multi: null operand");
        if (!aligned(packed[i], 4) || !aligned(scales[i], 2) || !aligned(biases[i], 2) || !aligned(y[i], 2))
            return fail(AQ_ERR_ARG, "aq_qmm_multi: operand pointer is not element-aligned");
        const size_t n = aq::qmm_scratch_bytes(M, K, N[i]);
        need = n > need ? n : need;
    }
    if (M <= aq::kQmvMaxRows && ctx->forced[1] < 0) {
        // up to four rows: matvec calls (one launch per four members where the fused kernels take the shape)
        for (int i = 0; i < count; i += aq::kQmvMultiMax) {
            const int n = count - i < aq::kQmvMultiMax ? count - i : aq::kQmvMultiMax;
            if (int rc = aq_qmv_multi(ctx, x, n, packed + i, scales + i, biases + i, y + i, N + i, M, K, group_size, bits, flags)) return rc;
        }
        ctx->last_variant[1] = ctx->last_variant[0];
        return AQ_OK;
    }
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    // the largest member's scratch first, so that no member makes the workspace move under the pass over x
    if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, need, fail)) return rc;
    int x_state = aq::kXReadyNone;
    for (int i = 0; i < count; i++)
        if (int rc = aq::qmm_dispatch(ctx->stream, &ctx->ws, ctx->cu_count, ctx->forced[1], &ctx->last_variant[1], x, packed[i],
                                      scales[i], biases[i], y[i], M, K, N[i], group_size, bits, (flags & AQ_OUT_F32) != 0, fail,
                                      nullptr, 0, &x_state))
            return rc;
    return AQ_OK;
}

int aq_reserve_workspace(aq_ctx* ctx, int M, int K) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_reserve_workspace: ctx is null");
    if (M < 0 || K < 0) return fail(AQ_ERR_SHAPE, "aq_reserve_workspace: M and K must be non-negative");
    if (M == 0 || K == 0) return AQ_OK;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    return aq::qmm_reserve(ctx->stream, &ctx->ws, M, K, fail);
}

int aq_reserve_workspace_bytes(aq_ctx* ctx, size_t bytes) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_reserve_workspace_bytes: ctx is null");
    if (bytes == 0) return AQ_OK;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    return aq::workspace_reserve(ctx->stream, &ctx->ws, bytes, fail);
}

size_t aq_workspace_bytes(aq_ctx* ctx) {
    if (!ctx) return 0;
    std::lock_guard<std::mutex> lk(ctx->mu);
    return ctx->ws.bytes + ctx->head_ws.bytes;
}

int aq_gather_qmv(aq_ctx* ctx, const void* x, const void* packed, const void* scales, const void* biases,
                  const int32_t* lhs, const int32_t* rhs, void* y, int routes, int x_rows, int K, int N,
                  int num_experts, int expert_rows, int row_base, int group_size, int bits, unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_gather_qmv: ctx is null");
    if (routes < 0 || K < 0 || N < 0) return fail(AQ_ERR_SHAPE, "aq_gather_qmv: routes, K, N must be non-negative");
    if (routes == 0 || N == 0 || K == 0) return AQ_OK;  // qmv_gather.go:422-424
    if (num_experts <= 0 || expert_rows <= 0 || x_rows <= 0)
        return fail(AQ_ERR_SHAPE, "aq_gather_qmv: num_experts, expert_rows and x_rows must be positive");
    if (row_base < 0 || (int64_t)row_base + N > expert_rows)
        return fail(AQ_ERR_SHAPE, "aq_gather_qmv: rows [%d, %d) fall outside an expert slab of %d rows", row_base,
                    row_base + N, expert_rows);
    if (int rc = check_geometry("aq_gather_qmv", K, group_size, bits)) return rc;
    if (!x || !packed || !scales || !biases || !rhs || !y) return fail(AQ_ERR_ARG, "aq_gather_qmv: null operand");
    if (!aligned(x, 2) || !aligned(packed, 4) || !aligned(scales, 2) || !aligned(biases, 2) || !aligned(y, 2) ||
        !aligned(rhs, 4) || (lhs && !aligned(lhs, 4)))
        return fail(AQ_ERR_ARG, "aq_gather_qmv: operand pointer is not element-aligned");
    if (routes > 65535) return fail(AQ_ERR_UNSUPPORTED, "aq_gather_qmv: at most 65535 routes per call");
    std::lock_guard<std::mutex> lk(ctx->mu);
    aq::QmvArgs a{};
    a.x = static_cast<const uint16_t*>(x);
    a.w = static_cast<const uint32_t*>(packed);
    a.s = static_cast<const uint16_t*>(scales);
    a.b = static_cast<const uint16_t*>(biases);
    a.y = y;
    a.lhs = lhs;
    a.rhs = rhs;
    a.K = K;
    a.N = N;
    a.M = 1;
    a.out_f32 = (flags & AQ_OUT_F32) ? 1 : 0;
    a.num_experts = num_experts;
    a.expert_rows = expert_rows;
    a.row_base = row_base;
    a.x_rows = x_rows;
    a.routes = routes;
    // every expert slab must keep 16-byte row alignment for the dot2 kernels
    return launch_qmv_rows(ctx, a, group_size, bits, true);
}

namespace {

bool act_ok(int act) { return act == AQ_ACT_GELU_TANH || act == AQ_ACT_SILU; }

// Bytes of the workspace the matmul path may claim for an M x K by N call (activations in fragment order,
// partial tiles of a K split), 256-byte aligned: the unfused fallbacks keep their intermediates behind it.
size_t qmm_region(int M, int K, int N) { return aq::qmm_scratch_bytes(M, K, N); }

// Rows per wavefront for the activation-fused dot2 kernels: `slots` row streams a wavefront of the
// plain kernel would take for this much work, shared between the two matrices of a pair.
int act_rows(const aq_ctx* ctx, int bits, int fuse, bool gather, int64_t N, int K, int routes) {
    const int64_t streams = fuse == 1 ? 2 * N : N;
    const int idx = pick_qmv_variant(ctx, bits, 1, gather, (int)(streams < INT32_MAX ? streams : INT32_MAX), K, routes);
    int rows = idx >= 0 ? aq::qmv_variant(idx)->rows : 1;
    if (fuse == 1) rows = rows >= 4 ? 2 : 1;
    while (rows > 1 && !aq::qmv_act_supported(bits, fuse, rows, gather)) rows >>= 1;
    return rows;
}

}  // namespace

int aq_act_mul(aq_ctx* ctx, const void* gate, const void* up, void* y, int64_t n, int act) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_act_mul: ctx is null");
    if (n < 0) return fail(AQ_ERR_SHAPE, "aq_act_mul: n must be non-negative");
    if (!act_ok(act)) return fail(AQ_ERR_UNSUPPORTED, "aq_act_mul: unknown activation %d", act);
    if (n == 0) return AQ_OK;
    if (!gate || !up || !y) return fail(AQ_ERR_ARG, "aq_act_mul: null operand");
    if (!aligned(gate, 2) || !aligned(up, 2) || !aligned(y, 2))
        return fail(AQ_ERR_ARG, "aq_act_mul: operand pointer is not element-aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::act_mul_launch(static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up),
                              static_cast<uint16_t*>(y), n, act, ctx->stream),
           "hipLaunchKernel");
    return AQ_OK;
}

int aq_qmv_gate_up(aq_ctx* ctx, const void* x, const void* gate_packed, const void* gate_scales, const void* gate_biases,
                   const void* up_packed, const void* up_scales, const void* up_biases, void* y, int M, int K, int N,
                   int group_size, int bits, int act, unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_qmv_gate_up: ctx is null");
    if (M < 0 || K < 0 || N < 0) return fail(AQ_ERR_SHAPE, "aq_qmv_gate_up: M, K, N must be non-negative");
    if (!act_ok(act)) return fail(AQ_ERR_UNSUPPORTED, "aq_qmv_gate_up: unknown activation %d", act);
    if (M == 0 || N == 0) return AQ_OK;
    if (K == 0) return fail(AQ_ERR_SHAPE, "aq_qmv_gate_up: K must be positive when there is output to write");
    if (int rc = check_geometry("aq_qmv_gate_up", K, group_size, bits)) return rc;
    const bool tiled = (flags & AQ_W_TILED) != 0;  // gate_packed and up_packed are tile-major tensors
    if (tiled) {
        if (aq::tile_total_bytes(N, K, group_size, bits) < 0)
            return fail(AQ_ERR_UNSUPPORTED, "aq_qmv_gate_up: no tile-major layout for bits=%d group=%d K=%d", bits, group_size, K);
        if (!aligned(gate_packed, 16) || !aligned(up_packed, 16))
            return fail(AQ_ERR_ARG, "aq_qmv_gate_up: a tile-major tensor is 16-byte aligned");
        gate_scales = gate_biases = up_scales = up_biases = nullptr;
    }
    if (!x || !gate_packed || !up_packed || !y || (!tiled && (!gate_scales || !gate_biases || !up_scales || !up_biases)))
        return fail(AQ_ERR_ARG, "aq_qmv_gate_up: null operand");
    if (!aligned(x, 2) || !aligned(gate_packed, 4) || !aligned(up_packed, 4) || !aligned(gate_scales, 2) ||
        !aligned(gate_biases, 2) || !aligned(up_scales, 2) || !aligned(up_biases, 2) || !aligned(y, 2))
        return fail(AQ_ERR_ARG, "aq_qmv_gate_up: operand pointer is not element-aligned");
    const bool out_f32 = (flags & AQ_OUT_F32) != 0;
    if (M <= 4 && ctx->forced[0] < 0) {
        // the diagonal-MFMA kernels with one set of wavefronts per matrix
        // the split of K that a single row gets; any row count shares its bytes
        const int di = (ctx->families_off >> kFamDiag & 1) ? -1 : aq::qmvd_pick(1, K, 1 << 20);
        aq::QmvArgs a{};
        a.x = static_cast<const uint16_t*>(x);
        a.w = static_cast<const uint32_t*>(gate_packed);
        a.s = static_cast<const uint16_t*>(gate_scales);
        a.b = static_cast<const uint16_t*>(gate_biases);
        a.w2 = static_cast<const uint32_t*>(up_packed);
        a.s2 = static_cast<const uint16_t*>(up_scales);
        a.b2 = static_cast<const uint16_t*>(up_biases);
        a.y = y;
        a.K = K;
        a.N = N;
        a.M = M;
        a.gs_shift = is_pow2(group_size) ? ilog2(group_size) : 0;
        a.out_f32 = out_f32 ? 1 : 0;
        a.routes = 1;
        a.act = act;
        a.tiled = tiled ? 1 : 0;
        aq::QmvArgs up = a;
        up.w = a.w2;
        up.s = a.s2;
        up.b = a.b2;
        if (di >= 0 && aq::qmvd_pair_supported(di) && aq::qmvd_fits(a, bits, group_size, false, di) &&
            aq::qmvd_fits(up, bits, group_size, false, di) &&
            (size_t)M * K * 2 + (size_t)M * ((K + 255) / 256) * 48 + 128 + (size_t)2 * aq::qmvd_variant(di)->waves * 256 <= 96 * 1024) {
            std::lock_guard<std::mutex> lk(ctx->mu);
            ctx->last_variant[0] = "qmv_gate_up_diag";
            AQ_HIP(aq::qmvd_pair_launch(di, a, false, ctx->stream), "hipLaunchKernel");
            return AQ_OK;
        }
    }
    if (tiled) {
        // no fused tile-major kernel for this call: the MLX arrays of both matrices are rebuilt behind the scratch
        // of the unfused route, which then runs as for any other call
        const size_t region = qmm_region(M, K, N) + 2 * align256((size_t)M * N * 4);
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
        if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, region + 2 * untiled_bytes(N, K), fail)) return rc;
        const uint32_t* w[2];
        const uint16_t *sc[2], *bi[2];
        if (int rc = untile_into_ws(ctx, region, gate_packed, N, K, &w[0], &sc[0], &bi[0])) return rc;
        if (int rc = untile_into_ws(ctx, region + untiled_bytes(N, K), up_packed, N, K, &w[1], &sc[1], &bi[1])) return rc;
        gate_packed = w[0], gate_scales = sc[0], gate_biases = bi[0];
        up_packed = w[1], up_scales = sc[1], up_biases = bi[1];
    }
    if (M == 1 && ctx->forced[0] < 0 && dot2_eligible(K, group_size, bits, x, gate_packed, (size_t)K * 2) &&
        aligned(up_packed, 16)) {
        std::lock_guard<std::mutex> lk(ctx->mu);
        const int rows = act_rows(ctx, bits, 1, false, N, K, 1);
        if (aq::qmv_act_supported(bits, 1, rows, false)) {
            aq::QmvArgs a{};
            a.x = static_cast<const uint16_t*>(x);
            a.w = static_cast<const uint32_t*>(gate_packed);
            a.s = static_cast<const uint16_t*>(gate_scales);
            a.b = static_cast<const uint16_t*>(gate_biases);
            a.w2 = static_cast<const uint32_t*>(up_packed);
            a.s2 = static_cast<const uint16_t*>(up_scales);
            a.b2 = static_cast<const uint16_t*>(up_biases);
            a.y = y;
            a.K = K;
            a.N = N;
            a.M = 1;
            a.gs_shift = ilog2(group_size);
            a.out_f32 = out_f32 ? 1 : 0;
            a.routes = 1;
            a.act = act;
            ctx->last_variant[0] = "qmv_gate_up_dot2";
            AQ_HIP(aq::qmv_act_launch(bits, 1, rows, false, a, ctx->stream), "hipLaunchKernel");
            return AQ_OK;
        }
    }
    // two projections into fp32 scratch, then the element-wise step
    const size_t region = qmm_region(M, K, N);
    const size_t each = (((size_t)M * N * 4) + 255) & ~(size_t)255;
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
        if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, region + 2 * each, fail)) return rc;
    }
    float* g = reinterpret_cast<float*>(static_cast<char*>(ctx->ws.ptr) + region);
    float* u = reinterpret_cast<float*>(static_cast<char*>(ctx->ws.ptr) + region + each);
    if (M > 32 && ctx->forced[0] < 0 && !(ctx->families_off >> kFamTiles & 1) &&
        aq::qmm_takes_gate(x, up_packed, K, group_size, bits) && aq::qmm_takes_gate(x, gate_packed, K, group_size, bits)) {
        // prefill sizes: both projections run on the matmul tiles (where aq_qmv sends this many rows anyway), the second
        // pass over x is skipped, and the stores of the `up` projection apply act(gate) * up on the way out
        // (rocm_mlx_q4_gelu_tanh_multiply_batch, go/engine/hip/kernels/quant/affine_gelu_tanh.hipinc:921-1109): one
        // [M, N] fp32 matrix is written and read instead of two written and two read.  Same bytes as the route below.
        std::lock_guard<std::mutex> lk(ctx->mu);
        int x_state = aq::kXReadyNone;
        if (int rc = aq::qmm_dispatch(ctx->stream, &ctx->ws, ctx->cu_count, ctx->forced[1], &ctx->last_variant[1], x, gate_packed,
                                      gate_scales, gate_biases, g, M, K, N, group_size, bits, true, fail, nullptr, 0, &x_state))
            return rc;
        const int rc = aq::qmm_dispatch(ctx->stream, &ctx->ws, ctx->cu_count, ctx->forced[1], &ctx->last_variant[1], x, up_packed,
                                        up_scales, up_biases, y, M, K, N, group_size, bits, out_f32, fail, g, act, &x_state);
        if (rc == AQ_OK) ctx->last_variant[0] = "qmv_gate_up_tiles";
        return rc;
    }
    if (int rc = aq_qmv(ctx, x, gate_packed, gate_scales, gate_biases, g, M, K, N, group_size, bits, AQ_OUT_F32)) return rc;
    if (int rc = aq_qmv(ctx, x, up_packed, up_scales, up_biases, u, M, K, N, group_size, bits, AQ_OUT_F32)) return rc;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::act_mul_f32_launch(g, u, y, (int64_t)M * N, act, out_f32 ? 1 : 0, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int aq_gather_qmv_gate_up(aq_ctx* ctx, const void* x, const void* packed, const void* scales, const void* biases,
                          const int32_t* lhs, const int32_t* rhs, void* y, int routes, int x_rows, int K, int N,
                          int num_experts, int expert_rows, int gate_row_base, int up_row_base, int group_size,
                          int bits, int act, unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_gather_qmv_gate_up: ctx is null");
    if (routes < 0 || K < 0 || N < 0) return fail(AQ_ERR_SHAPE, "aq_gather_qmv_gate_up: routes, K, N must be non-negative");
    if (!act_ok(act)) return fail(AQ_ERR_UNSUPPORTED, "aq_gather_qmv_gate_up: unknown activation %d", act);
    if (routes == 0 || N == 0) return AQ_OK;
    if (K == 0) return fail(AQ_ERR_SHAPE, "aq_gather_qmv_gate_up: K must be positive when there is output to write");
    if (num_experts <= 0 || expert_rows <= 0 || x_rows <= 0)
        return fail(AQ_ERR_SHAPE, "aq_gather_qmv_gate_up: num_experts, expert_rows and x_rows must be positive");
    for (int base : {gate_row_base, up_row_base})
        if (base < 0 || (int64_t)base + N > expert_rows)
            return fail(AQ_ERR_SHAPE, "aq_gather_qmv_gate_up: rows [%d, %d) fall outside an expert slab of %d rows", base,
                        base + N, expert_rows);
    if (int rc = check_geometry("aq_gather_qmv_gate_up", K, group_size, bits)) return rc;
    if (!x || !packed || !scales || !biases || !rhs || !y) return fail(AQ_ERR_ARG, "aq_gather_qmv_gate_up: null operand");
    if (!aligned(x, 2) || !aligned(packed, 4) || !aligned(scales, 2) || !aligned(biases, 2) || !aligned(y, 2) ||
        !aligned(rhs, 4) || (lhs && !aligned(lhs, 4)))
        return fail(AQ_ERR_ARG, "aq_gather_qmv_gate_up: operand pointer is not element-aligned");
    if (routes > 65535) return fail(AQ_ERR_UNSUPPORTED, "aq_gather_qmv_gate_up: at most 65535 routes per call");
    const bool out_f32 = (flags & AQ_OUT_F32) != 0;
    if (ctx->forced[0] < 0) {
        // the gathered diagonal-MFMA pair kernel: one set of wavefronts on the gate rows, one on the up rows
        const int di = (ctx->families_off >> kFamDiag & 1) ? -1 : aq::qmvd_pick_gather(K);
        aq::QmvArgs a{};
        a.x = static_cast<const uint16_t*>(x);
        a.w = a.w2 = static_cast<const uint32_t*>(packed);
        a.s = a.s2 = static_cast<const uint16_t*>(scales);
        a.b = a.b2 = static_cast<const uint16_t*>(biases);
        a.y = y;
        a.lhs = lhs;
        a.rhs = rhs;
        a.K = K;
        a.N = N;
        a.M = 1;
        a.gs_shift = is_pow2(group_size) ? ilog2(group_size) : 0;
        a.out_f32 = out_f32 ? 1 : 0;
        a.num_experts = num_experts;
        a.expert_rows = expert_rows;
        a.row_base = gate_row_base;
        a.row_base2 = up_row_base;
        a.x_rows = x_rows;
        a.routes = routes;
        a.act = act;
        if (di >= 0 && aq::qmvd_pair_supported(di) && aq::qmvd_fits(a, bits, group_size, true, di)) {
            std::lock_guard<std::mutex> lk(ctx->mu);
            ctx->last_variant[0] = "gather_gate_up_diag";
            AQ_HIP(aq::qmvd_pair_launch(di, a, true, ctx->stream), "hipLaunchKernel");
            return AQ_OK;
        }
    }
    if (ctx->forced[0] < 0 && dot2_eligible(K, group_size, bits, x, packed, (size_t)K * 2)) {
        std::lock_guard<std::mutex> lk(ctx->mu);
        const int rows = act_rows(ctx, bits, 1, true, N, K, routes);
        if (aq::qmv_act_supported(bits, 1, rows, true)) {
            aq::QmvArgs a{};
            a.x = static_cast<const uint16_t*>(x);
            a.w = a.w2 = static_cast<const uint32_t*>(packed);
            a.s = a.s2 = static_cast<const uint16_t*>(scales);
            a.b = a.b2 = static_cast<const uint16_t*>(biases);
            a.y = y;
            a.lhs = lhs;
            a.rhs = rhs;
            a.K = K;
            a.N = N;
            a.M = 1;
            a.gs_shift = ilog2(group_size);
            a.out_f32 = out_f32 ? 1 : 0;
            a.num_experts = num_experts;
            a.expert_rows = expert_rows;
            a.row_base = gate_row_base;
            a.row_base2 = up_row_base;
            a.x_rows = x_rows;
            a.routes = routes;
            a.act = act;
            ctx->last_variant[0] = "gather_gate_up_dot2";
            AQ_HIP(aq::qmv_act_launch(bits, 1, rows, true, a, ctx->stream), "hipLaunchKernel");
            return AQ_OK;
        }
    }
    const size_t each = (((size_t)routes * N * 4) + 255) & ~(size_t)255;
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
        if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, 2 * each, fail)) return rc;
    }
    float* g = static_cast<float*>(ctx->ws.ptr);
    float* u = reinterpret_cast<float*>(static_cast<char*>(ctx->ws.ptr) + each);
    if (int rc = aq_gather_qmv(ctx, x, packed, scales, biases, lhs, rhs, g, routes, x_rows, K, N, num_experts, expert_rows,
                               gate_row_base, group_size, bits, AQ_OUT_F32))
        return rc;
    if (int rc = aq_gather_qmv(ctx, x, packed, scales, biases, lhs, rhs, u, routes, x_rows, K, N, num_experts, expert_rows,
                               up_row_base, group_size, bits, AQ_OUT_F32))
        return rc;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::act_mul_f32_launch(g, u, y, (int64_t)routes * N, act, out_f32 ? 1 : 0, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int aq_qmv_act(aq_ctx* ctx, const void* gate_x, const void* up_x, const void* packed, const void* scales,
               const void* biases, void* y, int M, int K, int N, int group_size, int bits, int act, unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_qmv_act: ctx is null");
    if (M < 0 || K < 0 || N < 0) return fail(AQ_ERR_SHAPE, "aq_qmv_act: M, K, N must be non-negative");
    if (!act_ok(act)) return fail(AQ_ERR_UNSUPPORTED, "aq_qmv_act: unknown activation %d", act);
    if (M == 0 || N == 0 || K == 0) return AQ_OK;
    if (int rc = check_geometry("aq_qmv_act", K, group_size, bits)) return rc;
    if (!gate_x || !up_x || !packed || !scales || !biases || !y) return fail(AQ_ERR_ARG, "aq_qmv_act: null operand");
    if (!aligned(gate_x, 2) || !aligned(up_x, 2) || !aligned(packed, 4) || !aligned(scales, 2) || !aligned(biases, 2) ||
        !aligned(y, 2))
        return fail(AQ_ERR_ARG, "aq_qmv_act: operand pointer is not element-aligned");
    if (M == 1 && ctx->forced[0] < 0 && dot2_eligible(K, group_size, bits, gate_x, packed, (size_t)K * 2) &&
        aligned(up_x, 16)) {
        std::lock_guard<std::mutex> lk(ctx->mu);
        const int rows = act_rows(ctx, bits, 2, false, N, K, 1);
        if (aq::qmv_act_supported(bits, 2, rows, false)) {
            aq::QmvArgs a{};
            a.x = static_cast<const uint16_t*>(gate_x);
            a.x2 = static_cast<const uint16_t*>(up_x);
            a.w = static_cast<const uint32_t*>(packed);
            a.s = static_cast<const uint16_t*>(scales);
            a.b = static_cast<const uint16_t*>(biases);
            a.y = y;
            a.K = K;
            a.N = N;
            a.M = 1;
            a.gs_shift = ilog2(group_size);
            a.out_f32 = (flags & AQ_OUT_F32) ? 1 : 0;
            a.routes = 1;
            a.act = act;
            ctx->last_variant[0] = "qmv_act_dot2";
            AQ_HIP(aq::qmv_act_launch(bits, 2, rows, false, a, ctx->stream), "hipLaunchKernel");
            return AQ_OK;
        }
    }
    const size_t region = qmm_region(M, K, N);
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
        if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, region + (size_t)M * K * 2, fail)) return rc;
    }
    void* gated = static_cast<char*>(ctx->ws.ptr) + region;
    if (int rc = aq_act_mul(ctx, gate_x, up_x, gated, (int64_t)M * K, act)) return rc;
    return aq_qmv(ctx, gated, packed, scales, biases, y, M, K, N, group_size, bits, flags);
}

int aq_gather_qmv_act(aq_ctx* ctx, const void* gate_x, const void* up_x, const void* packed, const void* scales,
                      const void* biases, const int32_t* lhs, const int32_t* rhs, void* y, int routes, int x_rows, int K,
                      int N, int num_experts, int expert_rows, int row_base, int group_size, int bits, int act,
                      unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_gather_qmv_act: ctx is null");
    if (routes < 0 || K < 0 || N < 0) return fail(AQ_ERR_SHAPE, "aq_gather_qmv_act: routes, K, N must be non-negative");
    if (!act_ok(act)) return fail(AQ_ERR_UNSUPPORTED, "aq_gather_qmv_act: unknown activation %d", act);
    if (routes == 0 || N == 0 || K == 0) return AQ_OK;
    if (num_experts <= 0 || expert_rows <= 0 || x_rows <= 0)
        return fail(AQ_ERR_SHAPE, "aq_gather_qmv_act: num_experts, expert_rows and x_rows must be positive");
    if (row_base < 0 || (int64_t)row_base + N > expert_rows)
        return fail(AQ_ERR_SHAPE, "aq_gather_qmv_act: rows [%d, %d) fall outside an expert slab of %d rows", row_base,
                    row_base + N, expert_rows);
    if (int rc = check_geometry("aq_gather_qmv_act", K, group_size, bits)) return rc;
    if (!gate_x || !up_x || !packed || !scales || !biases || !rhs || !y)
        return fail(AQ_ERR_ARG, "aq_gather_qmv_act: null operand");
    if (!aligned(gate_x, 2) || !aligned(up_x, 2) || !aligned(packed, 4) || !aligned(scales, 2) || !aligned(biases, 2) ||
        !aligned(y, 2) || !aligned(rhs, 4) || (lhs && !aligned(lhs, 4)))
        return fail(AQ_ERR_ARG, "aq_gather_qmv_act: operand pointer is not element-aligned");
    if (routes > 65535) return fail(AQ_ERR_UNSUPPORTED, "aq_gather_qmv_act: at most 65535 routes per call");
    if (ctx->forced[0] < 0 && dot2_eligible(K, group_size, bits, gate_x, packed, (size_t)K * 2) && aligned(up_x, 16)) {
        std::lock_guard<std::mutex> lk(ctx->mu);
        const int rows = act_rows(ctx, bits, 2, true, N, K, routes);
        if (aq::qmv_act_supported(bits, 2, rows, true)) {
            aq::QmvArgs a{};
            a.x = static_cast<const uint16_t*>(gate_x);
            a.x2 = static_cast<const uint16_t*>(up_x);
            a.w = static_cast<const uint32_t*>(packed);
            a.s = static_cast<const uint16_t*>(scales);
            a.b = static_cast<const uint16_t*>(biases);
            a.y = y;
            a.lhs = lhs;
            a.rhs = rhs;
            a.K = K;
            a.N = N;
            a.M = 1;
            a.gs_shift = ilog2(group_size);
            a.out_f32 = (flags & AQ_OUT_F32) ? 1 : 0;
            a.num_experts = num_experts;
            a.expert_rows = expert_rows;
            a.row_base = row_base;
            a.x_rows = x_rows;
            a.routes = routes;
            a.act = act;
            ctx->last_variant[0] = "gather_act_dot2";
            AQ_HIP(aq::qmv_act_launch(bits, 2, rows, true, a, ctx->stream), "hipLaunchKernel");
            return AQ_OK;
        }
    }
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
        if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, (size_t)x_rows * K * 2, fail)) return rc;
    }
    if (int rc = aq_act_mul(ctx, gate_x, up_x, ctx->ws.ptr, (int64_t)x_rows * K, act)) return rc;
    return aq_gather_qmv(ctx, ctx->ws.ptr, packed, scales, biases, lhs, rhs, y, routes, x_rows, K, N, num_experts,
                         expert_rows, row_base, group_size, bits, flags);
}

int aq_moe_route(aq_ctx* ctx, const void* logits, int rows, int num_experts, int top_k, const float* expert_scales,
                 int normalise_top_k, int32_t* ids, float* weights, int32_t* token_of_route, unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_moe_route: ctx is null");
    if (rows < 0) return fail(AQ_ERR_SHAPE, "aq_moe_route: rows must be non-negative");
    // rocmReferenceRouteExperts (moe_quant_reference.go:28-33): logits required, 0 < top-k <= experts
    if (num_experts <= 0) return fail(AQ_ERR_SHAPE, "aq_moe_route: router logits are required");
    if (top_k <= 0 || top_k > num_experts) return fail(AQ_ERR_SHAPE, "aq_moe_route: top-k must be within the expert count");
    if (num_experts > aq::kMoeMaxExperts || top_k > aq::kMoeMaxTopK)
        return fail(AQ_ERR_UNSUPPORTED, "aq_moe_route: at most %d experts and top-%d", aq::kMoeMaxExperts, aq::kMoeMaxTopK);
    if (rows == 0) return AQ_OK;
    if (!logits || !ids || !weights) return fail(AQ_ERR_ARG, "aq_moe_route: null operand");
    const bool lb = (flags & AQ_LOGITS_BF16) != 0;
    if (!aligned(logits, lb ? 2 : 4) || !aligned(ids, 4) || !aligned(weights, 4) ||
        (expert_scales && !aligned(expert_scales, 4)) || (token_of_route && !aligned(token_of_route, 4)))
        return fail(AQ_ERR_ARG, "aq_moe_route: operand pointer is not element-aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    aq::MoeRouteArgs a{};
    a.logits = logits;
    a.expert_scales = expert_scales;
    a.ids = ids;
    a.weights = weights;
    a.token_of_route = token_of_route;
    a.rows = rows;
    a.num_experts = num_experts;
    a.top_k = top_k;
    a.normalise = normalise_top_k ? 1 : 0;
    a.logits_bf16 = lb ? 1 : 0;
    AQ_HIP(aq::moe_route_launch(a, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int aq_moe_combine(aq_ctx* ctx, const void* route_rows, const float* weights, void* out, int rows, int top_k, int n,
                   unsigned flags) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_moe_combine: ctx is null");
    if (rows < 0 || n < 0) return fail(AQ_ERR_SHAPE, "aq_moe_combine: rows and n must be non-negative");
    if (top_k <= 0) return fail(AQ_ERR_SHAPE, "aq_moe_combine: top-k must be positive");
    if (rows == 0 || n == 0) return AQ_OK;
    if (!route_rows || !weights || !out) return fail(AQ_ERR_ARG, "aq_moe_combine: null operand");
    const bool in_f32 = (flags & AQ_IN_F32) != 0, out_f32 = (flags & AQ_OUT_F32) != 0;
    if (!aligned(route_rows, in_f32 ? 4 : 2) || !aligned(weights, 4) || !aligned(out, out_f32 ? 4 : 2))
        return fail(AQ_ERR_ARG, "aq_moe_combine: operand pointer is not element-aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    aq::MoeCombineArgs a{};
    a.route_rows = route_rows;
    a.weights = weights;
    a.out = out;
    a.rows = rows;
    a.top_k = top_k;
    a.n = n;
    a.in_f32 = in_f32 ? 1 : 0;
    a.out_f32 = out_f32 ? 1 : 0;
    a.bf16_steps = (flags & AQ_BF16_STEPS) ? 1 : 0;
    AQ_HIP(aq::moe_combine_launch(a, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

namespace {

// The static scratch array of the context's device as (partial maxima, fold area) for `slots` maxima; the fold
// area's tickets must start at zero whatever an earlier call left there, so they are cleared by a fill kernel
// ahead of the projection on the same stream (a kernel, not a memset node: the call may be under capture).
int static_head_scratch(aq_ctx* ctx, const char* op, size_t slots, unsigned long long** partial, unsigned long long** fold) {
    if (slots * 8 > kStaticPartialBytes)
        return fail(AQ_ERR_SIZE, "%s: %zu partial maxima need %zu bytes, the static scratch holds %zu; use aq_qmv_greedy", op,
                    slots, slots * 8, kStaticPartialBytes);
    if (!ctx->static_scratch) return fail(AQ_ERR_NODEVICE, "%s: the device's scratch array was not resolved", op);
    *partial = reinterpret_cast<unsigned long long*>(ctx->static_scratch);
    *fold = reinterpret_cast<unsigned long long*>(ctx->static_scratch + kStaticPartialBytes);
    AQ_HIP(aq::fill_zero_launch(*fold, aq::kHeadFoldBytes, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

// Shared front of aq_qmv_greedy / aq_qmv_scores.  fuse 3: best[M]; fuse 4: scores[M, N].
// no_alloc (fuse 3 only): the partial maxima and the fold area live in the device's static scratch array instead of
// the context's workspaces, and a shape the fused kernels do not take is refused instead of going through scratch
// that would have to be allocated.
int head_call(aq_ctx* ctx, const char* op, int fuse, const void* x, const void* packed, const void* scales,
              const void* biases, const int32_t* suppress, int suppress_count, uint64_t* out, int M, int K, int N,
              int group_size, int bits, bool no_alloc = false) {
    if (!ctx) return fail(AQ_ERR_ARG, "%s: ctx is null", op);
    if (M < 0 || K < 0 || N < 0 || suppress_count < 0) return fail(AQ_ERR_SHAPE, "%s: M, K, N, suppress_count must be non-negative", op);
    if (M == 0) return AQ_OK;
    if (!out) return fail(AQ_ERR_ARG, "%s: null output", op);
    if (!aligned(out, 8)) return fail(AQ_ERR_ARG, "%s: output pointer is not 8-byte aligned", op);
    if (suppress_count > 0 && !suppress) return fail(AQ_ERR_ARG, "%s: suppress_count without a suppress list", op);
    if (suppress && !aligned(suppress, 4)) return fail(AQ_ERR_ARG, "%s: operand pointer is not element-aligned", op);
    // (a forced matvec variant sends the other head calls through aq_qmv and scratch memory; the entry point that
    // allocates nothing has no such route and keeps to the fused kernels)
    const bool fused = M == 1 && N > 0 && K > 0 && (ctx->forced[0] < 0 || no_alloc) && (bits == 4 || bits == 8) && x && packed &&
                       dot2_eligible(K, group_size, bits, x, packed, (size_t)K * 2);
    if (no_alloc && !fused && M > 0 && N > 0 && K > 0)
        return fail(AQ_ERR_UNSUPPORTED,
                    "%s: takes one activation row of 4- or 8-bit codes with 16-byte aligned rows (the fused kernels); "
                    "other shapes need scratch memory: use aq_qmv_greedy", op);
    if (fuse == 3 && !fused) {
        // the unfused reduction accumulates with atomics and starts from "no result"
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(aq::fill_zero_launch(out, (size_t)M * 8, ctx->stream), "hipLaunchKernel");
    }
    if (N == 0) return AQ_OK;
    if (K == 0) return fail(AQ_ERR_SHAPE, "%s: K must be positive when there are rows to score", op);
    if (int rc = check_geometry(op, K, group_size, bits)) return rc;
    if (!x || !packed || !scales || !biases) return fail(AQ_ERR_ARG, "%s: null operand", op);
    if (!aligned(x, 2) || !aligned(packed, 4) || !aligned(scales, 2) || !aligned(biases, 2))
        return fail(AQ_ERR_ARG, "%s: operand pointer is not element-aligned", op);
    if (fused) {
        std::lock_guard<std::mutex> lk(ctx->mu);
        {
            // the diagonal-MFMA kernel aq_qmv would pick for this projection, with the head epilogue
            const int di = bits != 4 || (ctx->families_off >> kFamDiag & 1) ? -1
                           : group_size == 32 ? aq::qmvd_pick_g32(1, K, N) : group_size == 64 ? aq::qmvd_pick(1, K, N) : -1;
            aq::QmvArgs a{};
            a.x = static_cast<const uint16_t*>(x);
            a.w = static_cast<const uint32_t*>(packed);
            a.s = static_cast<const uint16_t*>(scales);
            a.b = static_cast<const uint16_t*>(biases);
            a.y = out;
            a.K = K;
            a.N = N;
            a.M = 1;
            a.gs_shift = ilog2(group_size);
            a.routes = 1;
            a.suppress = suppress;
            a.suppress_count = suppress_count;
            if (di >= 0 && aq::qmvd_head_supported(di, fuse) && aq::qmvd_fits(a, bits, group_size, false, di)) {
                const size_t slots = aq::qmvd_head_partials(di, N);
                unsigned long long* fold = static_cast<unsigned long long*>(ctx->head_fold);
                if (fuse == 3 && no_alloc) {
                    if (int rc = static_head_scratch(ctx, op, slots, &a.partial, &fold)) return rc;
                } else if (fuse == 3) {
                    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
                    if (int rc = aq::workspace_reserve(ctx->stream, &ctx->head_ws, slots * 8, fail)) return rc;
                    a.partial = static_cast<unsigned long long*>(ctx->head_ws.ptr);
                }
                ctx->last_variant[0] = fuse == 3 ? "qmv_greedy_diag" : "qmv_scores_diag";
                AQ_HIP(aq::qmvd_head_launch(di, fuse, a, ctx->stream), "hipLaunchKernel");
                if (fuse == 3)
                    AQ_HIP(aq::head_fold_launch(a.partial, (int)slots, fold, reinterpret_cast<unsigned long long*>(out),
                                                ctx->stream),
                           "hipLaunchKernel");
                return AQ_OK;
            }
        }
        const int idx = pick_qmv_variant(ctx, bits, 1, false, N, K, 1);
        int rows = idx >= 0 ? aq::qmv_variant(idx)->rows : 1;
        while (rows > 1 && !aq::qmv_head_supported(bits, fuse, rows)) rows >>= 1;
        if (!aq::qmv_head_supported(bits, fuse, rows)) return fail(AQ_ERR_UNSUPPORTED, "%s: no kernel for bits=%d", op, bits);
        unsigned long long* partial = nullptr;
        unsigned long long* fold = static_cast<unsigned long long*>(ctx->head_fold);
        if (fuse == 3 && no_alloc) {
            if (int rc = static_head_scratch(ctx, op, aq::qmv_head_partials(N, rows), &partial, &fold)) return rc;
        } else if (fuse == 3) {
            AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
            if (int rc = aq::workspace_reserve(ctx->stream, &ctx->head_ws, aq::qmv_head_partials(N, rows) * 8, fail)) return rc;
            partial = static_cast<unsigned long long*>(ctx->head_ws.ptr);
        }
        {
            aq::QmvArgs a{};
            a.x = static_cast<const uint16_t*>(x);
            a.w = static_cast<const uint32_t*>(packed);
            a.s = static_cast<const uint16_t*>(scales);
            a.b = static_cast<const uint16_t*>(biases);
            a.y = out;
            a.K = K;
            a.N = N;
            a.M = 1;
            a.gs_shift = ilog2(group_size);
            a.routes = 1;
            a.suppress = suppress;
            a.suppress_count = suppress_count;
            a.partial = partial;
            a.fold = fold;
            ctx->last_variant[0] = fuse == 3 ? "qmv_greedy_dot2" : "qmv_scores_dot2";
            AQ_HIP(aq::qmv_head_launch(bits, fuse, rows, a, ctx->stream), "hipLaunchKernel");
            return AQ_OK;
        }
    }
    // the projection as fp32 into scratch, then the same epilogue over it
    const size_t region = qmm_region(M, K, N);
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
        if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, region + (size_t)M * N * 4, fail)) return rc;
    }
    float* logits = reinterpret_cast<float*>(static_cast<char*>(ctx->ws.ptr) + region);
    if (int rc = aq_qmv(ctx, x, packed, scales, biases, logits, M, K, N, group_size, bits, AQ_OUT_F32)) return rc;
    std::lock_guard<std::mutex> lk(ctx->mu);
    unsigned long long* o = reinterpret_cast<unsigned long long*>(out);
    AQ_HIP(aq::pack_scores_launch(logits, M, N, suppress, suppress_count, fuse == 3 ? o : nullptr, fuse == 4 ? o : nullptr,
                                  ctx->stream),
           "hipLaunchKernel");
    return AQ_OK;
}

uint32_t ordered_key_host(float v) {
    uint32_t bits;
    memcpy(&bits, &v, 4);
    return (bits & 0x80000000u) ? ~bits : (bits ^ 0x80000000u);
}

}  // namespace

int aq_qmv_greedy(aq_ctx* ctx, const void* x, const void* packed, const void* scales, const void* biases,
                  const int32_t* suppress, int suppress_count, uint64_t* best, int M, int K, int N, int group_size,
                  int bits) {
    return head_call(ctx, "aq_qmv_greedy", 3, x, packed, scales, biases, suppress, suppress_count, best, M, K, N,
                     group_size, bits);
}

int aq_qmv_greedy_selected(aq_ctx* ctx, const void* x, const void* packed, const void* scales, const void* biases,
                           const int32_t* rows, int count, uint64_t* best, int K, int N, int group_size, int bits) {
    const char* op = "aq_qmv_greedy_selected";
    if (!ctx) return fail(AQ_ERR_ARG, "%s: ctx is null", op);
    if (K < 0 || N < 0 || count < 0) return fail(AQ_ERR_SHAPE, "%s: K, N, count must be non-negative", op);
    if (!best) return fail(AQ_ERR_ARG, "%s: null output", op);
    if (!aligned(best, 8)) return fail(AQ_ERR_ARG, "%s: output pointer is not 8-byte aligned", op);
    if (count > 0 && !rows) return fail(AQ_ERR_ARG, "%s: count without a list of rows", op);
    if (rows && !aligned(rows, 4)) return fail(AQ_ERR_ARG, "%s: operand pointer is not element-aligned", op);
    if (count == 0 || N == 0) {  // nothing to choose from: "no result"
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(aq::fill_zero_launch(best, 8, ctx->stream), "hipLaunchKernel");
        return AQ_OK;
    }
    if (K == 0) return fail(AQ_ERR_SHAPE, "%s: K must be positive when there are rows to score", op);
    if (int rc = check_geometry(op, K, group_size, bits)) return rc;
    if (!x || !packed || !scales || !biases) return fail(AQ_ERR_ARG, "%s: null operand", op);
    if (!aligned(x, 2) || !aligned(packed, 4) || !aligned(scales, 2) || !aligned(biases, 2))
        return fail(AQ_ERR_ARG, "%s: operand pointer is not element-aligned", op);
    if (count > 65535) return fail(AQ_ERR_UNSUPPORTED, "%s: at most 65535 candidates per call", op);
    const int width = N < 16 ? N : 16;
    const size_t start_bytes = align256((size_t)count * 4), need = start_bytes + (size_t)count * width * 4;
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, need, fail)) return rc;
    int32_t* start = static_cast<int32_t*>(ctx->ws.ptr);
    float* scores = reinterpret_cast<float*>(static_cast<char*>(ctx->ws.ptr) + start_bytes);
    AQ_HIP(aq::selected_windows_launch(rows, count, N, width, start, ctx->stream), "hipLaunchKernel");
    aq::QmvArgs a{};
    a.x = static_cast<const uint16_t*>(x);
    a.w = static_cast<const uint32_t*>(packed);
    a.s = static_cast<const uint16_t*>(scales);
    a.b = static_cast<const uint16_t*>(biases);
    a.y = scores;
    a.rhs = start;  // the "expert" of candidate z is the row its window starts at: a slab of experts one row apart
    a.K = K;
    a.N = width;
    a.M = 1;
    a.out_f32 = 1;
    a.num_experts = N - width + 1;
    a.expert_rows = 1;
    a.x_rows = 1;
    a.routes = count;
    if (int rc = launch_qmv_rows(ctx, a, group_size, bits, true)) return rc;
    AQ_HIP(aq::selected_pick_launch(scores, rows, start, count, width, reinterpret_cast<unsigned long long*>(best), ctx->stream),
           "hipLaunchKernel");
    return AQ_OK;
}

int aq_qmv_greedy_static(aq_ctx* ctx, const void* x, const void* packed, const void* scales, const void* biases,
                         const int32_t* suppress, int suppress_count, uint64_t* best, int K, int N, int group_size, int bits) {
    return head_call(ctx, "aq_qmv_greedy_static", 3, x, packed, scales, biases, suppress, suppress_count, best, 1, K, N,
                     group_size, bits, true);
}

int aq_qmv_scores(aq_ctx* ctx, const void* x, const void* packed, const void* scales, const void* biases,
                  const int32_t* suppress, int suppress_count, uint64_t* scores, int M, int K, int N, int group_size,
                  int bits) {
    return head_call(ctx, "aq_qmv_scores", 4, x, packed, scales, biases, suppress, suppress_count, scores, M, K, N,
                     group_size, bits);
}

int aq_packed_topk(aq_ctx* ctx, const uint64_t* scores, int64_t count, int top_k, uint64_t* out) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_packed_topk: ctx is null");
    if (count < 0) return fail(AQ_ERR_SHAPE, "aq_packed_topk: count must be non-negative");
    if (top_k <= 0) return fail(AQ_ERR_SHAPE, "aq_packed_topk: top-k must be positive");
    if (top_k > aq::kTopKMax) return fail(AQ_ERR_UNSUPPORTED, "aq_packed_topk: top-k is at most %d", aq::kTopKMax);
    if (!out || (count > 0 && !scores)) return fail(AQ_ERR_ARG, "aq_packed_topk: null operand");
    if (!aligned(out, 8) || !aligned(scores, 8)) return fail(AQ_ERR_ARG, "aq_packed_topk: operand pointer is not 8-byte aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    if (count == 0) {
        AQ_HIP(aq::fill_zero_launch(out, (size_t)top_k * 8, ctx->stream), "hipLaunchKernel");
        return AQ_OK;
    }
    const size_t need = aq::packed_topk_scratch_entries(count, top_k) * 8;
    if (need) {
        AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
        if (int rc = aq::workspace_reserve(ctx->stream, &ctx->ws, need, fail)) return rc;
    }
    AQ_HIP(aq::packed_topk_launch(reinterpret_cast<const unsigned long long*>(scores), count, top_k,
                                  reinterpret_cast<unsigned long long*>(out),
                                  static_cast<unsigned long long*>(ctx->ws.ptr), ctx->stream),
           "hipLaunchKernel");
    return AQ_OK;
}

int aq_packed_topk_sample(aq_ctx* ctx, const uint64_t* top, int top_k, float temperature, float top_p, float softcap,
                          double draw, uint64_t* out) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_packed_topk_sample: ctx is null");
    if (top_k <= 0) return fail(AQ_ERR_SHAPE, "aq_packed_topk_sample: top-k must be positive");
    if (top_k > aq::kSampleTopKMax)
        return fail(AQ_ERR_UNSUPPORTED, "aq_packed_topk_sample: top-k is at most %d", aq::kSampleTopKMax);
    if (!top || !out) return fail(AQ_ERR_ARG, "aq_packed_topk_sample: null operand");
    if (!aligned(top, 8) || !aligned(out, 8)) return fail(AQ_ERR_ARG, "aq_packed_topk_sample: operand pointer is not 8-byte aligned");
    // rocm_valid_packed_topk_sample_args, kernels/sampling/topk_validate.hipinc:53-77
    if (!(temperature >= 0.0f) || !std::isfinite(temperature))
        return fail(AQ_ERR_ARG, "aq_packed_topk_sample: temperature must be non-negative and finite");
    if (!(top_p >= 0.0f) || !(top_p <= 1.0f)) return fail(AQ_ERR_ARG, "aq_packed_topk_sample: top-p must be in [0, 1]");
    if (!(softcap >= 0.0f) || !std::isfinite(softcap))
        return fail(AQ_ERR_ARG, "aq_packed_topk_sample: softcap must be non-negative and finite");
    if (!std::isfinite(draw)) return fail(AQ_ERR_ARG, "aq_packed_topk_sample: draw must be finite");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::packed_topk_sample_launch(reinterpret_cast<const unsigned long long*>(top), top_k, temperature, top_p, softcap,
                                         draw, reinterpret_cast<unsigned long long*>(out), ctx->stream),
           "hipLaunchKernel");
    return AQ_OK;
}

uint64_t aq_pack_best(float score, int token) {
    return ((uint64_t)ordered_key_host(score) << 32) | (uint64_t)(~(uint32_t)token);
}

int aq_unpack_best(uint64_t packed, float softcap, int vocab_size, int* token, float* score) {
    // order and wording of hipUnpackGreedyBest (hip_projection_launch.go:2397-2416)
    if (vocab_size <= 0) return fail(AQ_ERR_SHAPE, "aq_unpack_best: vocab size must be positive");
    if (packed == 0) return fail(AQ_ERR_INDEX, "aq_unpack_best: greedy projection did not produce a result");
    if (softcap < 0 || softcap != softcap || softcap - softcap != 0)
        return fail(AQ_ERR_ARG, "aq_unpack_best: softcap must be non-negative and finite");
    const uint32_t low = (uint32_t)packed;
    const int64_t id = (int64_t)(int32_t)(~low);
    if (id < 0 || id >= vocab_size) return fail(AQ_ERR_INDEX, "aq_unpack_best: greedy projection token is out of range");
    const uint32_t key = (uint32_t)(packed >> 32);
    const uint32_t bits = (key & 0x80000000u) ? (key ^ 0x80000000u) : ~key;
    float s;
    memcpy(&s, &bits, 4);
    if (softcap > 0) s = (float)tanh((double)(s / softcap)) * softcap;
    if (token) *token = (int)id;
    if (score) *score = s;
    return AQ_OK;
}

namespace {

// Geometry a loaded weight must satisfy before it may be handed to the kernels.
int check_linear(const char* op, const aqh_linear* l) {
    if (!l) return fail(AQ_ERR_ARG, "%s: null weight", op);
    if (!l->quantised || !l->scales || !l->biases || !l->weight)
        return fail(AQ_ERR_UNSUPPORTED, "%s: only affine-quantised weights (with scales and biases) are uploaded", op);
    if (l->expert_rows <= 0 || l->experts < 0 || l->in_dim <= 0) return fail(AQ_ERR_SHAPE, "%s: invalid dimensions", op);
    if (int rc = check_geometry(op, l->in_dim, l->group_size, l->bits)) return rc;
    const size_t e = l->experts > 0 ? (size_t)l->experts : 1;
    const size_t want_w = e * (size_t)l->expert_rows * ((size_t)l->in_dim * l->bits / 32) * 4;
    const size_t want_sb = e * (size_t)l->expert_rows * (size_t)(l->in_dim / l->group_size) * 2;
    if (l->weight_len != want_w || l->scales_len != want_sb || l->biases_len != want_sb)
        return fail(AQ_ERR_SIZE, "%s: packed/scales/biases size mismatch", op);
    return AQ_OK;
}

}  // namespace

int aq_upload_linear(aq_ctx* ctx, const struct aqh_linear* lin, aq_device_linear* out) {
    if (!ctx || !out) return fail(AQ_ERR_ARG, "aq_upload_linear: bad argument");
    memset(out, 0, sizeof *out);
    if (int rc = check_linear("aq_upload_linear", lin)) return rc;
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    DevBuf w, s, b;
    AQ_HIP(w.alloc(lin->weight_len), "hipMalloc");
    AQ_HIP(s.alloc(lin->scales_len), "hipMalloc");
    AQ_HIP(b.alloc(lin->biases_len), "hipMalloc");
    if (int rc = aq_h2d(ctx, w.p, lin->weight, lin->weight_len)) return rc;
    if (int rc = aq_h2d(ctx, s.p, lin->scales, lin->scales_len)) return rc;
    if (int rc = aq_h2d(ctx, b.p, lin->biases, lin->biases_len)) return rc;
    out->weight = w.p, out->scales = s.p, out->biases = b.p;
    w.p = s.p = b.p = nullptr;
    out->rows = lin->expert_rows;
    out->in_dim = lin->in_dim;
    out->group_size = lin->group_size;
    out->bits = lin->bits;
    out->experts = lin->experts;
    return AQ_OK;
}

int aq_upload_fused_gate_up(aq_ctx* ctx, const struct aqh_linear* gate, const struct aqh_linear* up, aq_device_linear* out) {
    if (!ctx || !out) return fail(AQ_ERR_ARG, "aq_upload_fused_gate_up: bad argument");
    memset(out, 0, sizeof *out);
    if (int rc = check_linear("aq_upload_fused_gate_up", gate)) return rc;
    if (int rc = check_linear("aq_upload_fused_gate_up", up)) return rc;
    // model.ConcatQuantRows' conditions (quant_weight.go:46-48), plus equal row and expert counts
    if (gate->in_dim != up->in_dim || gate->bits != up->bits || gate->group_size != up->group_size ||
        gate->expert_rows != up->expert_rows || gate->experts != up->experts)
        return fail(AQ_ERR_SHAPE, "aq_upload_fused_gate_up: gate and up differ in geometry");
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    const size_t experts = gate->experts > 0 ? (size_t)gate->experts : 1;
    const size_t w_part = gate->weight_len / experts, sb_part = gate->scales_len / experts;
    DevBuf w, s, b;
    AQ_HIP(w.alloc(2 * gate->weight_len), "hipMalloc");
    AQ_HIP(s.alloc(2 * gate->scales_len), "hipMalloc");
    AQ_HIP(b.alloc(2 * gate->biases_len), "hipMalloc");
    std::lock_guard<std::mutex> lk(ctx->mu);
    // one strided copy per part and array: expert e's rows go to [e][part]
    struct Job {
        void* dst;
        const uint8_t* src;
        size_t part;
    } jobs[6] = {{w.p, gate->weight, w_part},  {static_cast<char*>(w.p) + w_part, up->weight, w_part},
                 {s.p, gate->scales, sb_part}, {static_cast<char*>(s.p) + sb_part, up->scales, sb_part},
                 {b.p, gate->biases, sb_part}, {static_cast<char*>(b.p) + sb_part, up->biases, sb_part}};
    for (const Job& j : jobs)
        AQ_HIP(hipMemcpy2DAsync(j.dst, 2 * j.part, j.src, j.part, j.part, experts, hipMemcpyHostToDevice, ctx->stream),
               "hipMemcpy2D");
    AQ_HIP(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize");
    out->weight = w.p, out->scales = s.p, out->biases = b.p;
    w.p = s.p = b.p = nullptr;
    out->rows = 2 * gate->expert_rows;
    out->in_dim = gate->in_dim;
    out->group_size = gate->group_size;
    out->bits = gate->bits;
    out->experts = gate->experts;
    return AQ_OK;
}

int aq_free_device_linear(aq_ctx* ctx, aq_device_linear* lin) {
    if (!ctx || !lin) return fail(AQ_ERR_ARG, "aq_free_device_linear: bad argument");
    for (void* p : {lin->weight, lin->scales, lin->biases})
        if (p) AQ_HIP(hipFree(p), "hipFree");
    memset(lin, 0, sizeof *lin);
    return AQ_OK;
}

int64_t aq_tiled_bytes(int64_t N, int K, int group_size, int bits) { return aq::tile_total_bytes(N, K, group_size, bits); }

int aq_tile_weights(aq_ctx* ctx, const void* packed, const void* scales, const void* biases, int64_t N, int K, int group_size,
                    int bits, void* tiled) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_tile_weights: ctx is null");
    if (N <= 0 || K <= 0) return fail(AQ_ERR_SHAPE, "aq_tile_weights: N and K must be positive");
    if (int rc = check_geometry("aq_tile_weights", K, group_size, bits)) return rc;
    if (aq::tile_total_bytes(N, K, group_size, bits) < 0)
        return fail(AQ_ERR_UNSUPPORTED, "aq_tile_weights: no tile-major layout for bits=%d group=%d K=%d (4-bit codes in groups of 64, K a multiple of 128)",
                    bits, group_size, K);
    if (!packed || !scales || !biases || !tiled) return fail(AQ_ERR_ARG, "aq_tile_weights: null operand");
    if (!aligned(packed, 16) || !aligned(tiled, 16) || !aligned(scales, 2) || !aligned(biases, 2))
        return fail(AQ_ERR_ARG, "aq_tile_weights: packed and tiled must be 16-byte aligned, scales and biases 2-byte aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::tile_repack_launch(packed, scales, biases, tiled, N, K, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int aq_tile_device_linear(aq_ctx* ctx, aq_device_linear* lin) {
    if (!ctx || !lin) return fail(AQ_ERR_ARG, "aq_tile_device_linear: bad argument");
    if (!lin->weight || !lin->scales || !lin->biases)
        return fail(AQ_ERR_ARG, "aq_tile_device_linear: the weight is not resident as MLX arrays (already tile-major?)");
    // (an expert slab is read by the gathers, which take MLX arrays)
    if (lin->experts > 0) return fail(AQ_ERR_UNSUPPORTED, "aq_tile_device_linear: expert slabs stay MLX arrays (the gathers read them)");
    const int64_t bytes = aq::tile_total_bytes(lin->rows, lin->in_dim, lin->group_size, lin->bits);
    if (bytes < 0 || bytes >= ((int64_t)1 << 32))
        return fail(AQ_ERR_UNSUPPORTED, "aq_tile_device_linear: no tile-major layout for bits=%d group=%d K=%d rows=%d", lin->bits,
                    lin->group_size, lin->in_dim, lin->rows);
    void* tiled = nullptr;
    {
        std::lock_guard<std::mutex> lk(ctx->mu);
        AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
        AQ_HIP(hipMalloc(&tiled, (size_t)bytes), "hipMalloc");
    }
    int rc = aq_tile_weights(ctx, lin->weight, lin->scales, lin->biases, lin->rows, lin->in_dim, lin->group_size, lin->bits, tiled);
    if (rc == AQ_OK) rc = aq_sync(ctx);  // the arrays are freed next
    if (rc != AQ_OK) {
        (void)hipFree(tiled);
        return rc;
    }
    for (void* p : {lin->weight, lin->scales, lin->biases}) AQ_HIP(hipFree(p), "hipFree");
    lin->weight = tiled;
    lin->scales = lin->biases = nullptr;
    return AQ_OK;
}

int aq_untile_weights(aq_ctx* ctx, const void* tiled, int64_t N, int K, int group_size, int bits, void* packed, void* scales,
                      void* biases) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_untile_weights: ctx is null");
    if (N <= 0 || K <= 0) return fail(AQ_ERR_SHAPE, "aq_untile_weights: N and K must be positive");
    if (int rc = check_geometry("aq_untile_weights", K, group_size, bits)) return rc;
    if (aq::tile_total_bytes(N, K, group_size, bits) < 0)
        return fail(AQ_ERR_UNSUPPORTED, "aq_untile_weights: no tile-major layout for bits=%d group=%d K=%d", bits, group_size, K);
    if (!packed || !scales || !biases || !tiled) return fail(AQ_ERR_ARG, "aq_untile_weights: null operand");
    if (!aligned(packed, 16) || !aligned(tiled, 16) || !aligned(scales, 2) || !aligned(biases, 2))
        return fail(AQ_ERR_ARG, "aq_untile_weights: packed and tiled must be 16-byte aligned, scales and biases 2-byte aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::tile_unpack_launch(tiled, packed, scales, biases, N, K, ctx->stream), "hipLaunchKernel");
    return AQ_OK;
}

int aq_dequant_f32(aq_ctx* ctx, const void* packed, const void* scales, const void* biases, float* out_f32, int64_t N,
                   int K, int group_size, int bits) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_dequant_f32: ctx is null");
    // mlxaffine.go:182-184: non-positive dims are invalid for the dequantizer.
    if (N <= 0 || K <= 0 || group_size <= 0 || K % group_size != 0)
        return fail(AQ_ERR_SHAPE, "aq_dequant_f32: invalid dimensions");
    if (!(bits == 1 || width_ok(bits))) return fail(AQ_ERR_UNSUPPORTED, "aq_dequant_f32: unsupported bits %d", bits);
    if (((int64_t)K * bits) % 32 != 0) return fail(AQ_ERR_SHAPE, "aq_dequant_f32: cols*bits must be divisible by 32");
    if (!packed || !scales || !biases || !out_f32) return fail(AQ_ERR_ARG, "aq_dequant_f32: null operand");
    if (N * (int64_t)K / 8 > 0x7fffffffLL * 32) return fail(AQ_ERR_UNSUPPORTED, "aq_dequant_f32: tensor too large");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::dequant_launch(static_cast<const uint32_t*>(packed), static_cast<const uint16_t*>(scales),
                              static_cast<const uint16_t*>(biases), out_f32, N, K, group_size, bits, ctx->stream),
           "hipLaunchKernel");
    return AQ_OK;
}

int aq_gguf_affine_layout_of(int gguf_type, int64_t rows, int64_t cols, aq_gguf_affine_layout* out) {
    if (!out) return fail(AQ_ERR_ARG, "aq_gguf_affine_layout_of: out is null");
    aq::GgufFormat f;
    if (!aq::gguf_format(gguf_type, &f))
        return fail(AQ_ERR_UNSUPPORTED, "aq_gguf_affine_layout_of: tensor must be GGUF affine-compatible (type %d)", gguf_type);
    if (rows <= 0 || cols <= 0 || cols % f.block_cols != 0)
        return fail(AQ_ERR_SHAPE, "aq_gguf_affine_layout_of: tensor shape must align to %d-column blocks", f.block_cols);
    if (rows > (int64_t)0x7fffffff * 32 / cols * 256)
        return fail(AQ_ERR_UNSUPPORTED, "aq_gguf_affine_layout_of: tensor too large");
    out->bits = f.bits;
    out->group_size = f.group_size;
    out->packed_cols = cols * f.bits / 32;
    out->groups = cols / f.group_size;
    out->src_bytes = (uint64_t)rows * (uint64_t)(cols / f.block_cols) * (uint64_t)f.block_bytes;
    out->packed_bytes = (uint64_t)rows * (uint64_t)out->packed_cols * 4;
    out->scales_bytes = (uint64_t)rows * (uint64_t)out->groups * 2;
    return AQ_OK;
}

int aq_gguf_to_affine(aq_ctx* ctx, int gguf_type, const void* src, uint64_t src_bytes, int64_t rows, int64_t cols,
                      void* packed, void* scales, void* biases) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_gguf_to_affine: ctx is null");
    aq_gguf_affine_layout lay;
    if (int rc = aq_gguf_affine_layout_of(gguf_type, rows, cols, &lay)) return rc;
    if (src_bytes != lay.src_bytes)
        return fail(AQ_ERR_SHAPE, "aq_gguf_to_affine: tensor byte count %llu does not match dimensions (%llu)",
                    (unsigned long long)src_bytes, (unsigned long long)lay.src_bytes);
    if (!src || !packed || !scales || !biases) return fail(AQ_ERR_ARG, "aq_gguf_to_affine: null operand");
    if (!aligned(packed, 16) || !aligned(scales, 2) || !aligned(biases, 2) || (gguf_type == aq::kGgufF32 && !aligned(src, 4)))
        return fail(AQ_ERR_ARG, "aq_gguf_to_affine: packed must be 16-byte, scales/biases 2-byte, F32 input 4-byte aligned");
    std::lock_guard<std::mutex> lk(ctx->mu);
    AQ_HIP(aq::gguf_repack_launch(gguf_type, static_cast<const uint8_t*>(src), static_cast<uint32_t*>(packed),
                                  static_cast<uint16_t*>(scales), static_cast<uint16_t*>(biases), rows * (cols / 32),
                                  ctx->stream),
           "hipLaunchKernel");
    return AQ_OK;
}

int aq_matvec_host(aq_ctx* ctx, const uint8_t* x, size_t x_len, const uint8_t* packed, size_t packed_len,
                   const uint8_t* scales, size_t scales_len, const uint8_t* biases, size_t biases_len, int out_dim,
                   int in_dim, int group_size, int bits, uint8_t* out, size_t out_len) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_matvec_host: ctx is null");
    // Order and conditions of enginetest.ReferenceAffineMatVec (quant_reference.go:79-106).
    if (out_dim < 0 || in_dim < 0) return fail(AQ_ERR_SHAPE, "aq_matvec_host: outDim/inDim must be non-negative");
    if (out_dim == 0 || in_dim == 0) return AQ_OK;
    if (bits <= 0 || bits > 8) return fail(AQ_ERR_UNSUPPORTED, "aq_matvec_host: bits must be in 1..8");
    if (group_size <= 0 || in_dim % group_size != 0)
        return fail(AQ_ERR_SHAPE, "aq_matvec_host: groupSize must be > 0 and divide inDim");
    if (((int64_t)in_dim * bits) % 8 != 0) return fail(AQ_ERR_SHAPE, "aq_matvec_host: inDim*bits must be byte-aligned");
    if (x_len != (size_t)in_dim * 2) return fail(AQ_ERR_SIZE, "aq_matvec_host: len(x) must equal inDim bf16 bytes");
    const size_t row_packed = (size_t)in_dim * bits / 8;
    const size_t row_sb = (size_t)(in_dim / group_size) * 2;
    if (packed_len != (size_t)out_dim * row_packed || scales_len != (size_t)out_dim * row_sb ||
        biases_len != (size_t)out_dim * row_sb)
        return fail(AQ_ERR_SIZE, "aq_matvec_host: packed/scales/biases size mismatch");
    if (out_len < (size_t)out_dim * 2) return fail(AQ_ERR_SIZE, "aq_matvec_host: out holds fewer than outDim bf16 values");
    if (!x || !packed || !scales || !biases || !out) return fail(AQ_ERR_ARG, "aq_matvec_host: null operand");
    if (int rc = check_geometry("aq_matvec_host", in_dim, group_size, bits)) return rc;
    DevBuf dx, dw, ds, db, dy;
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    AQ_HIP(dx.alloc(x_len), "hipMalloc");
    AQ_HIP(dw.alloc(packed_len), "hipMalloc");
    AQ_HIP(ds.alloc(scales_len), "hipMalloc");
    AQ_HIP(db.alloc(biases_len), "hipMalloc");
    AQ_HIP(dy.alloc((size_t)out_dim * 2), "hipMalloc");
    if (int rc = aq_h2d(ctx, dx.p, x, x_len)) return rc;
    if (int rc = aq_h2d(ctx, dw.p, packed, packed_len)) return rc;
    if (int rc = aq_h2d(ctx, ds.p, scales, scales_len)) return rc;
    if (int rc = aq_h2d(ctx, db.p, biases, biases_len)) return rc;
    if (int rc = aq_qmv(ctx, dx.p, dw.p, ds.p, db.p, dy.p, 1, in_dim, out_dim, group_size, bits, 0)) return rc;
    return aq_d2h(ctx, out, dy.p, (size_t)out_dim * 2);
}

int aq_proj_quant_matmul_host(aq_ctx* ctx, float* out, const float* x, size_t x_len, const uint8_t* packed,
                              size_t packed_len, const uint8_t* scales, size_t scales_len, const uint8_t* biases,
                              size_t biases_len, int M, int K, int N, int group_size, int bits) {
    if (!ctx) return fail(AQ_ERR_ARG, "aq_proj_quant_matmul_host: ctx is null");
    // quant_seam_backend.go:41-49
    if (M <= 0 || N <= 0 || K <= 0) return fail(AQ_ERR_SHAPE, "aq_proj_quant_matmul_host: M, N, K must be positive");
    if (x_len != (size_t)M * K) return fail(AQ_ERR_SIZE, "aq_proj_quant_matmul_host: len(x) must equal M*K");
    if (group_size <= 0 || bits <= 0 || K % group_size != 0)
        return fail(AQ_ERR_SHAPE, "aq_proj_quant_matmul_host: invalid quant geometry");
    if (int rc = check_geometry("aq_proj_quant_matmul_host", K, group_size, bits)) return rc;
    const size_t want_packed = (size_t)N * ((size_t)K * bits / 32) * 4;
    const size_t want_sb = (size_t)N * (K / group_size) * 2;
    if (packed_len != want_packed || scales_len != want_sb || biases_len != want_sb)
        return fail(AQ_ERR_SIZE, "aq_proj_quant_matmul_host: packed/scales/biases size mismatch");
    if (!out || !x || !packed || !scales || !biases) return fail(AQ_ERR_ARG, "aq_proj_quant_matmul_host: null operand");
    // f32 -> bf16 RNE at the seam (quant_seam_backend.go:50,66-74; codec mlxaffine.go:229-237)
    std::vector<uint16_t> xb((size_t)M * K);
    for (size_t i = 0; i < xb.size(); i++) {
        uint32_t u;
        memcpy(&u, &x[i], 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) {
            xb[i] = (uint16_t)((u >> 16) | 0x0040u);
        } else {
            u += 0x7fffu + ((u >> 16) & 1u);
            xb[i] = (uint16_t)(u >> 16);
        }
    }
    DevBuf dx, dw, ds, db, dy;
    AQ_HIP(hipSetDevice(ctx->device), "hipSetDevice");
    AQ_HIP(dx.alloc(xb.size() * 2), "hipMalloc");
    AQ_HIP(dw.alloc(packed_len), "hipMalloc");
    AQ_HIP(ds.alloc(scales_len), "hipMalloc");
    AQ_HIP(db.alloc(biases_len), "hipMalloc");
    AQ_HIP(dy.alloc((size_t)M * N * 2), "hipMalloc");
    if (int rc = aq_h2d(ctx, dx.p, xb.data(), xb.size() * 2)) return rc;
    if (int rc = aq_h2d(ctx, dw.p, packed, packed_len)) return rc;
    if (int rc = aq_h2d(ctx, ds.p, scales, scales_len)) return rc;
    if (int rc = aq_h2d(ctx, db.p, biases, biases_len)) return rc;
    int rc = (M == 1) ? aq_qmv(ctx, dx.p, dw.p, ds.p, db.p, dy.p, 1, K, N, group_size, bits, 0)
                      : aq_qmm(ctx, dx.p, dw.p, ds.p, db.p, dy.p, M, K, N, group_size, bits, 0);
    if (rc) return rc;
    std::vector<uint16_t> yb((size_t)M * N);
    if (int rc2 = aq_d2h(ctx, yb.data(), dy.p, yb.size() * 2)) return rc2;
    for (size_t i = 0; i < yb.size(); i++) {
        uint32_t u = (uint32_t)yb[i] << 16;
        memcpy(&out[i], &u, 4);
    }
    return AQ_OK;
}

int aq_variant_count(int op) {
    if (op == 0) return qmv_total_variants();
    if (op == 1) return aq::qmmt_variant_count();
    return 0;
}

const char* aq_variant_name(int op, int variant) {
    if (op == 0) {
        const aq::QmvVariant* v = (variant >= 0 && variant < qmv_total_variants()) ? qmv_any_variant(variant) : nullptr;
        return v ? v->name : "";
    }
    if (op == 1) {
        const aq::QmmVariant* v = aq::qmmt_variant(variant);
        return v ? v->name : "";
    }
    return "";
}

int aq_force_variant(aq_ctx* ctx, int op, int variant) {
    if (!ctx || op < 0 || op > 1) return fail(AQ_ERR_ARG, "aq_force_variant: bad argument");
    if (variant >= aq_variant_count(op)) return fail(AQ_ERR_ARG, "aq_force_variant: variant %d out of range", variant);
    std::lock_guard<std::mutex> lk(ctx->mu);
    ctx->forced[op] = variant < 0 ? -1 : variant;
    return AQ_OK;
}

const char* aq_last_variant(aq_ctx* ctx, int op) {
    if (!ctx || op < 0 || op > 1) return "";
    return ctx->last_variant[op];
}

}  // extern "C"
