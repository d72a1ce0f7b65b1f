// MFMA matmul path (affine_qmm and the many-row calls of affine_qmv).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aq {

// Largest M the dot2 matvec kernels take in one pass; a matmul call of up to this many rows runs as a matvec.
constexpr int kQmvMaxRows = 4;

struct QmmArgs {
    const uint16_t* x;  // [M, K] bf16
    const uint32_t* w;  // [N, K*bits/32]
    const uint16_t* s;  // [N, K/group]
    const uint16_t* b;  // [N, K/group]
    void* y;            // [M, N] bf16 or f32
    int M, K, N;
    int gs_blocks;  // 64-code blocks per quantisation group (1 for group 64, 2 for 128)
    int out_f32;
    const float* gate;  // not null: y = act(gate[m, n]) * (x . w^T)[m, n], gate being fp32 [M, N] (a gated MLP's other projection)
    int act;            // kActGeluTanh or kActSilu
    int x_ready;        // kXReady*: the workspace already holds this x as that pass over x leaves it (a call of several
                        // weight matrices against one x): the pass is skipped
};

// Which pass over x the workspace holds (QmmArgs.x_ready, and what a launch reports back through qmm_dispatch).
enum { kXReadyNone = 0, kXReadyTile4 = 1, kXReadyTile8 = 2, kXReadyHalf = 3 };

struct QmmVariant {
    const char* name;
    int bits;
    int mb, nb;  // 32x32 MFMA blocks per wavefront along M and N
    int wm, wn;  // wavefronts per workgroup along M and N
};

// Operands of the LDS-staged tile kernels (aq_qmm_tile.hip): x has been rewritten by their pass over x.
struct QmmTileArgs {
    const uint16_t* xf;  // activations in A-fragment order, rows padded to a multiple of 32
    const uint16_t* xs;  // per 64-code block sums of x as (hi, lo) bf16, four blocks per 16 bytes
    const float* rs;     // fp16-operand kernels: per row of x, the inverse of the power of two it was scaled by
    const uint32_t* w;
    const uint16_t* s;
    const uint16_t* b;
    void* y;
    int M, K, N;
    int gs_blocks;
    int out_f32;
    int mblks;             // ceil(M / 32)
    int tiles_m, tiles_n;  // workgroup tiles along M and N
    int ksplit;            // workgroups that share a tile along K (1: none)
    int gsplit;            // 64-code blocks of K per workgroup (a multiple of 4)
    float* partial;        // ksplit > 1: fp32 partial tiles [ksplit][M][N]
    const float* gate;     // as in QmmArgs (applied where the final value is stored)
    int act;
};

// (the variants of the fp16-operand kernels, aq_qmm_half.hip, are listed behind those of the tile kernels)
int qmmt_variant_count();
const QmmVariant* qmmt_variant(int idx);
// Device bytes the tile kernels need beside their operands for an M x K activation matrix.
size_t qmmt_workspace_bytes(int M, int K);
// Pass over x + tile kernel `idx`; `workspace` holds at least qmmt_workspace_bytes(M, K).
hipError_t qmmt_launch(int idx, const QmmArgs& a, void* workspace, hipStream_t stream);
// The pass over x variant idx needs (kXReady*).
int qmmt_x_kind(int idx);
// The same with K shared out over ksplit workgroups per tile and a second kernel that adds the partial
// tiles: for few rows of x, where M x N tiles alone leave most of the chip idle.
size_t qmmt_splitk_bytes(int M, int N, int ksplit);
hipError_t qmmt_launch_splitk(int idx, const QmmArgs& a, void* workspace, int ksplit, hipStream_t stream);

// Kernels for 5..64 rows of x whose LDS stages hold four blocks of K (aq_qmm_few.hip): listed behind the
// fp16-operand variants; they take the operands the tile kernels take and are launched through qmmt_launch_splitk.
int qmmf_variant_count();
const QmmVariant* qmmf_variant(int idx);
hipError_t qmmf_launch_kernel(int idx, const QmmTileArgs& a, hipStream_t stream);

// 4-bit kernels whose matrix-core operand carries scale * (code - 8) as fp16 (aq_qmm_half.hip); same workspace.
int qmmh_variant_count();
const QmmVariant* qmmh_variant(int idx);
hipError_t qmmh_launch(int idx, const QmmArgs& a, void* workspace, hipStream_t stream);

// Scratch memory a context lends to the matmul path; grown on demand, never while a capture is open.
// `generation` counts reallocations: a captured graph has the block's address in its kernel arguments and is
// only valid while the generation it was captured under stands.  `touched` is set by every reserve call, so
// that the owner can tell whether a capture used the block.
struct Workspace {
    void* ptr = nullptr;
    size_t bytes = 0;
    uint64_t generation = 0;
    bool touched = false;
};

hipError_t fill_zero_launch(void* p, size_t bytes, hipStream_t stream);

typedef int (*FailFn)(int code, const char* fmt, ...);

// Makes ws hold at least `need` bytes (drains the stream and reallocates when it must grow; refused
// while the stream is being captured).
int workspace_reserve(hipStream_t stream, Workspace* ws, size_t need, FailFn fail);

// Upper bound (256-byte aligned) of the workspace bytes qmm_dispatch may use for an M x K by N call: the
// rewritten activations and, for few rows, the fp32 partial tiles of the K split.  Callers that keep their
// own data in the same workspace place it behind this.
size_t qmm_scratch_bytes(int M, int K, int N);

// Sizes ws for activations of M x K ahead of time (not during capture).
int qmm_reserve(hipStream_t stream, Workspace* ws, int M, int K, FailFn fail);

// Validated-shape dispatch used by aq_qmm and by aq_qmv for calls the matvec families pass on.
// Returns an AQ_* / hipError_t code through `fail`.
// `forced` indexes the tile variants (qmmt_variant), or is negative.
// gate (fp32 [M, N], or null) and act: the gated-MLP epilogue, see QmmArgs; only where qmm_takes_gate says so.
// x_state (or null): in, which pass over this x the workspace already holds (kXReady*); out, which it holds now.
int qmm_dispatch(hipStream_t stream, Workspace* ws, int cu_count, int forced, const char** last_variant, const void* x,
                 const void* packed, const void* scales, const void* biases, void* y, int M, int K, int N,
                 int group_size, int bits, bool out_f32, FailFn fail, const float* gate = nullptr, int act = 0,
                 int* x_state = nullptr);
// Whether qmm_dispatch runs this call on the tile kernels, whose stores can carry the gated-MLP epilogue.
bool qmm_takes_gate(const void* x, const void* packed, int K, int group_size, int bits);

}  // namespace aq
