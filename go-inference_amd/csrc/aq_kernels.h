// Launch-side declarations shared between the kernel translation units and the
// C-ABI layer.  Plain structs and ints only; nothing here touches the public
// header's types.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aq {

// Operands of one affine matvec / gathered matvec launch.  Layouts follow the
// MLX group-affine format (go/model/quant/mlxaffine/mlxaffine.go:14-20):
//   w [rows, K*bits/32] u32, s/b [rows, K/group] bf16, x [x_rows, K] bf16.
struct QmvArgs {
    // (What a kernel needs before it can request its weights sits in the first 64 bytes of the kernel arguments: one
    // scalar load and one wait at the start of a wavefront instead of one per cache line.)
    const uint16_t* x;
    const uint32_t* w;
    void* y;          // [M, N] (plain) or [routes, N] (gather); bf16 or f32
    int K;
    int N;
    int M;            // activation rows (plain); 1 for gather
    int early_wgs;    // diagonal-MFMA kernels: workgroups (by index) that request their weights before they stage x
    const uint16_t* s;
    const uint16_t* b;
    int gs_shift;     // log2(group size)
    int out_f32;      // 0: bf16 stores, 1: f32 stores
    const int32_t* lhs;  // gather only: route -> x row, nullptr = row 0 for all
    const int32_t* rhs;  // gather only: route -> expert id
    int num_experts;  // gather only
    int expert_rows;  // gather only: rows per expert in the slab
    int row_base;     // gather only: first row of the slab used
    int x_rows;       // gather only: rows in x (bounds for lhs)
    int routes;       // gather only
    int stream_w;     // diagonal-MFMA kernels: load the weights with the non-temporal hint (set by the launch functions)
    int tiled;        // diagonal-MFMA kernels, dense: w (and w2) hold the tile-major layout of aq_tile.h; s, b are not read
    // activation-fused kernels only (aq_qmv_act.hip)
    const uint16_t* x2;  // x-load fusion: the `up` activations, same shape and row indexing as x (the `gate` ones)
    const uint32_t* w2;  // pair fusion: the `up` matrix (w, s, b are the `gate` one)
    const uint16_t* s2;
    const uint16_t* b2;
    int row_base2;       // pair fusion + gather: first `up` row inside an expert's slab
    int act;             // kActGeluTanh or kActSilu
    // head kernels only (aq_qmv_head.hip): y is uint64 best[M] (argmax) or uint64 scores[M, N]
    const int32_t* suppress;  // token ids that may not win, or nullptr
    int suppress_count;
    unsigned long long* partial;  // argmax: one slot per wavefront of the grid (qmv_head_partials)
    unsigned long long* fold;     // argmax: kHeadFoldBytes of zeroed device memory that the fold leaves zeroed
};

constexpr int kActGeluTanh = 1;
constexpr int kActSilu = 2;

// Activation-fused dot2 kernels (aq_qmv_act.hip), one activation row.
//   fuse 1: y[n] = act(gate[n,:] . x) * (up[n,:] . x)          (two matrices, one output)
//   fuse 2: y[n] = w[n,:] . bf16(act(x[k]) * x2[k])            (activation applied while x is staged)
// rows: output rows per wavefront (fuse 1: of each matrix).  False / error when no kernel fits.
bool qmv_act_supported(int bits, int fuse, int rows, bool gather);
hipError_t qmv_act_launch(int bits, int fuse, int rows, bool gather, const QmvArgs& a, hipStream_t stream);
// y[i] = bf16(act(gate[i]) * up[i]) over n bf16 values.
hipError_t act_mul_launch(const uint16_t* gate, const uint16_t* up, uint16_t* y, int64_t n, int act, hipStream_t stream);
// y[i] = act(gate[i]) * up[i] over n fp32 values, stored as bf16 or fp32.
hipError_t act_mul_f32_launch(const float* gate, const float* up, void* y, int64_t n, int act, int out_f32,
                              hipStream_t stream);

// Up to kQmvMultiMax weight matrices that share x, K, group size and width: one launch.
constexpr int kQmvMultiMax = 4;
struct QmvMultiArgs {
    QmvArgs common;  // x, K, M, gs_shift, out_f32 (w, s, b, y, N are taken from the arrays below)
    int count;
    const uint32_t* w[kQmvMultiMax];
    const uint16_t* s[kQmvMultiMax];
    const uint16_t* b[kQmvMultiMax];
    void* y[kQmvMultiMax];
    int N[kQmvMultiMax];
    int block_end[kQmvMultiMax];  // filled by the launcher: first workgroup past matrix i
};
// dot2 kernels only: 4 wavefronts a workgroup, `rows` output rows per wavefront, m = 1..4 activation rows.
bool qmv_multi_supported(int bits, int m, int rows);
hipError_t qmv_multi_launch(int bits, int m, int rows, QmvMultiArgs ma, hipStream_t stream);

struct QmvVariant {
    const char* name;
    int bits;
    int m;       // activation rows handled per pass (1..4)
    int rows;    // output rows per wavefront
    int waves;   // wavefronts per workgroup
    int depth;   // K slices in flight per wavefront
    int gather;  // 1: reads rhs/lhs on device, grid.y = routes
    int xmode;   // family-specific (dot2: 0; diagonal: chunks per step when not 4; token tile: runs held per pass)
    int kind;    // 0: VALU dot2 kernel (aq_qmv.hip),
                 // 2: block-MFMA kernel (aq_qmv_blk.hip; m = most rows, depth = K pieces per wavefront),
                 // 4: diagonal-MFMA kernel (aq_qmv_diag.hip; m = most rows, rows = sets of 16 rows per workgroup,
                 //    xmode = chunks per step when not 4), 5: the same for quantisation groups of 32 codes
                 // 6: token-tile MFMA kernel (aq_qmv_tok.hip; m = most rows, rows = sets of 16 weight rows per workgroup)
};

int qmv_variant_count();
const QmvVariant* qmv_variant(int idx);
// Launch variant `idx` (from the table) on `stream`.  Shapes must already be
// validated by the caller.
hipError_t qmv_launch(int idx, const QmvArgs& a, hipStream_t stream);
// LDS bytes variant idx needs for these args (x staging).
size_t qmv_lds_bytes(int idx, const QmvArgs& a);

// Block-MFMA matvec kernels (aq_qmv_blk.hip; M <= 16, persistent workgroups that split K among their
// wavefronts).  A launch needs a plan: which kernel, how many wavefronts and workgroups, LDS bytes.
struct BlkGeom {
    uint32_t row_bytes;     // packed bytes per weight row
    uint32_t sb_row_bytes;  // bytes per row of scales (= biases)
    uint32_t wstep;         // bytes between a wavefront's consecutive K pieces
    int gpw;                // groups in one wavefront K piece
    int hh_shift;           // log2(gpw / 4): 8-byte scale pieces per K piece
    int rpp;                // row groups one 64-lane staging pass covers
    int stage_bufs;         // 1, or 2 when a workgroup walks more than one batch
    int total_rg;           // row groups (4 rows each)
    int batch;              // row groups whose scales are staged and whose partial sums meet in LDS at once
};
struct BlkPlan {
    int idx;  // variant
    int nw;   // wavefronts per workgroup
    int nwg;  // workgroups along x
    size_t lds;
    BlkGeom geom;
};
int qmvb_variant_count();
const QmvVariant* qmvb_variant(int idx);
// False when the shape does not fit these kernels (the caller then uses another family).
// forced_idx < 0: choose the variant; otherwise plan for exactly that one.
bool qmvb_plan(const QmvArgs& a, int bits, int group_size, bool gather, int cu_count, int forced_idx, BlkPlan* out);
hipError_t qmvb_launch(const BlkPlan& p, const QmvArgs& a, hipStream_t stream);

// Diagonal-MFMA matvec kernels (aq_qmv_diag.hip; 4-bit group-64 codes, M <= 8, K a multiple of 128 in 2..16 steps of 1024;
// 8-bit group-64 codes, M <= 4, in steps of 512).
int qmvd_variant_count();
const QmvVariant* qmvd_variant(int idx);
bool qmvd_fits(const QmvArgs& a, int bits, int group_size, bool gather, int idx);
hipError_t qmvd_launch(int idx, const QmvArgs& a, hipStream_t stream);
// The variant the library picks for M rows and this K, or -1 when another family takes the shape.
int qmvd_pick(int M, int K, int N, int bits = 4);  // (8-bit codes: up to four rows)
// The same for quantisation groups of 32 codes (up to two rows, K a multiple of 256).
int qmvd_pick_g32(int M, int K, int N);
// y = act(gate . x) * (up . x) with variant idx's split of K (a.w2, a.s2, a.b2: the `up` matrix; a.act); the two
// dot products are the bytes qmvd_launch computes for each matrix.
bool qmvd_pair_supported(int idx);
hipError_t qmvd_pair_launch(int idx, const QmvArgs& a, bool gather, hipStream_t stream);
// The gathered variant (one activation row per route, grid.y = routes) for this K, or -1.
int qmvd_pick_gather(int K);
// lm_head epilogues on variant idx (fuse 3: best packed value per 16 rows into a.partial, qmvd_head_partials(idx, N)
// slots, to be folded by head_fold_launch; fuse 4: packed scores into a.y).
bool qmvd_head_supported(int idx, int fuse);
size_t qmvd_head_partials(int idx, int N);
hipError_t qmvd_head_launch(int idx, int fuse, const QmvArgs& a, hipStream_t stream);
// Folds `count` partial maxima into best[0] (aq_qmv_head.hip).
hipError_t head_fold_launch(const unsigned long long* partial, int count, unsigned long long* fold, unsigned long long* best,
                            hipStream_t stream);
bool qmvd_multi_supported(int idx);
hipError_t qmvd_multi_launch(int idx, QmvMultiArgs ma, hipStream_t stream);

// Token-tile MFMA matvec kernels (aq_qmv_tok.hip; group-64 codes of 4 or 8 bits, up to 32 activation rows as
// the rows of 16x16x32 MFMAs, K a multiple of 256 up to 16384; one launch, no scratch memory).  kind 6 in QmvVariant.
int qmvt_variant_count();
const QmvVariant* qmvt_variant(int idx);
bool qmvt_fits(const QmvArgs& a, int bits, int group_size, int idx);
hipError_t qmvt_launch(int idx, const QmvArgs& a, hipStream_t stream);
int qmvt_pick(int bits, int M, int K, int N, int cu_count);

// lm_head kernels (aq_qmv_head.hip), one activation row: the projection with its epilogue replaced by
//   fuse 3: best[0] = max over rows of pack(score, row): every wavefront stores its own maximum into
//           a.partial (no contention); a second kernel of kHeadFoldGroups workgroups folds the partials,
//           and the last of those to finish (a ticket in a.fold) writes a.y[0]
//   fuse 4: scores[row] = pack(score, row)
// Non-finite scores and suppressed rows pack to 0.
constexpr int kHeadFoldGroups = 64;
constexpr size_t kHeadFoldBytes = 128 + (size_t)kHeadFoldGroups * 8;  // ticket counter on its own line, then the group maxima
bool qmv_head_supported(int bits, int fuse, int rows);
// Slots a.partial must hold for the argmax of N rows at `rows` rows per wavefront.
size_t qmv_head_partials(int N, int rows);
hipError_t qmv_head_launch(int bits, int fuse, int rows, const QmvArgs& a, hipStream_t stream);
// Greedy over a candidate list (aq_qmv_head.hip): the window of `width` rows each candidate is scored in (-1: id out of
// range), and the maximum of pack(score, row) over the candidates' own rows of the gathered scores [count, width].
hipError_t selected_windows_launch(const int32_t* rows, int count, int N, int width, int32_t* start, hipStream_t stream);
hipError_t selected_pick_launch(const float* scores, const int32_t* rows, const int32_t* start, int count, int width,
                                unsigned long long* best, hipStream_t stream);
// The same two epilogues over fp32 scores that are already in memory: scores [M, N] -> best[M] / packed[M, N].
hipError_t pack_scores_launch(const float* scores, int M, int N, const int32_t* suppress, int suppress_count,
                              unsigned long long* best_or_null, unsigned long long* packed_or_null, hipStream_t stream);
// Largest top_k (<= kTopKMax) of `count` packed values, sorted descending, into out[top_k]; scratch holds
// packed_topk_scratch_entries(count, top_k) values.
constexpr int kTopKMax = 64;
constexpr int kTopKPerLane = 16;                    // values a lane sorts in registers
constexpr int kTopKSegment = 64 * kTopKPerLane;     // values one wavefront reduces to top_k
constexpr int kTopKCandidates = 1024;               // entries the threshold path orders in one workgroup
constexpr int kTopKThresholdSegments = 1024;        // most segments whose maxima a wavefront holds in registers
size_t packed_topk_scratch_entries(int64_t count, int top_k);
hipError_t packed_topk_launch(const unsigned long long* in, int64_t count, int top_k, unsigned long long* out,
                              unsigned long long* scratch, hipStream_t stream);

// MoE router and combine (aq_moe.hip).
constexpr int kMoeMaxExperts = 1024;
constexpr int kMoeMaxTopK = 64;
struct MoeRouteArgs {
    const void* logits;           // [rows, num_experts] f32 or bf16
    const float* expert_scales;   // [num_experts] or nullptr
    int32_t* ids;                 // [rows, top_k]
    float* weights;               // [rows, top_k]
    int32_t* token_of_route;      // [rows, top_k] or nullptr
    int rows, num_experts, top_k;
    int normalise;                // 1: softmax over the selected scores; 0: softmax over all, gathered
    int logits_bf16;
};
struct MoeCombineArgs {
    const void* route_rows;  // [rows * top_k, n] bf16 or f32
    const float* weights;    // [rows * top_k]
    void* out;               // [rows, n] bf16 or f32
    int rows, top_k, n;
    int in_f32, out_f32, bf16_steps;
};
hipError_t moe_route_launch(const MoeRouteArgs& a, hipStream_t stream);
hipError_t moe_combine_launch(const MoeCombineArgs& a, hipStream_t stream);

// Any-width (2..8 bit, codes may straddle words), any-group fallback.
hipError_t qmv_generic_launch(const QmvArgs& a, int bits, int group_size, bool gather, hipStream_t stream);
// Six-bit codes in groups of 16 or 32 with K a multiple of 16 take a kernel of their own inside that launch.
bool qmv_six_eligible(const QmvArgs& a, int bits, int group_size);

// Allows `lds` bytes of dynamic LDS for kernel function fn when that is beyond the 48 KiB every kernel may use: one
// hipFuncSetAttribute per device and function (for the largest size asked so far) instead of one per launch.
hipError_t ensure_dynamic_lds(const void* fn, size_t lds);

// Measurement aid (aq_misc.hip): reads the codes, scales and biases of a 4-bit group-64 tensor once with no arithmetic,
// in the access shape of the diagonal-MFMA matvec (mode 0) or as contiguous 1 KiB pieces (mode 1).
hipError_t read_probe_launch(const void* w, const void* s, const void* b, int64_t rows, int row_bytes, int sb_bytes, int mode,
                             uint32_t* out, hipStream_t stream);

// MLX layout <-> tile-major layout of a 4-bit group-64 tensor (aq_tile.hip, layout in aq_tile.h).  w 16-byte aligned.
hipError_t tile_repack_launch(const void* w, const void* s, const void* b, void* tiled, int64_t N, int K, hipStream_t stream);
hipError_t tile_unpack_launch(const void* tiled, void* w, void* s, void* b, int64_t N, int K, hipStream_t stream);

// fp32 dequantisation of a whole tensor, bits in {1,2,4,8} (word-clean widths)
// or {3,5,6} through the straddling path.
hipError_t dequant_launch(const uint32_t* w, const uint16_t* s, const uint16_t* b, float* out, int64_t N, int K,
                          int group_size, int bits, hipStream_t stream);

// Temperature / top-p sampling over a descending packed list of at most kSampleTopKMax entries (aq_qmv_head.hip).
constexpr int kSampleTopKMax = 128;
hipError_t packed_topk_sample_launch(const unsigned long long* in, int top_k, float temperature, float top_p, float softcap,
                                     double draw, unsigned long long* out, hipStream_t stream);

// GGUF block formats -> affine layout (aq_gguf.hip).  Type ids are GGUF's own
// (go/engine/hip/hip_gguf_affine_adapter.go:19-25, :56).
constexpr int kGgufF32 = 0, kGgufQ4_0 = 2, kGgufQ4_1 = 3, kGgufQ8_0 = 8, kGgufQ4_K = 12, kGgufQ5_K = 13, kGgufQ6_K = 14;
struct GgufFormat {
    int block_cols, block_bytes, bits, group_size;
};
bool gguf_format(int type, GgufFormat* f);
// spans = rows * cols / 32.  w 16-byte aligned, s and b 2-byte aligned, src 4-byte aligned for F32.
hipError_t gguf_repack_launch(int type, const uint8_t* src, uint32_t* w, uint16_t* s, uint16_t* b, int64_t spans,
                              hipStream_t stream);

}  // namespace aq
