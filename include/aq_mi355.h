/*
 * aq_mi355.h -- C ABI of libaq_mi355.so: MLX group-affine quantized matvec /
 * matmul / expert-gathered matvec for AMD MI355X (gfx950).
 *
 * This is the boundary a go-inference backend binds (cgo or dlopen) in place
 * of its own HIP module + launch-packet path.  Every entry point names the
 * reference interface it stands in for (paths relative to the go-inference
 * checkout).  Plain pointers and sizes only.
 *
 * Tensor layout (go/model/quant/mlxaffine/mlxaffine.go:14-20):
 *   packed  uint32 little-endian [N, K*bits/32]; code p of a word occupies bits
 *           [p*bits, p*bits+bits), LSB first, along K
 *   scales  bf16 [N, K/group]     biases  bf16 [N, K/group]
 *   w[n,k] = scale[n,k/group] * code[n,k] + bias[n,k/group]
 * Activations and results are bf16 row-major unless AQ_OUT_F32 is given.
 *
 * Return value: 0 = ok; < 0 = argument rejected on the host before any launch
 * (AQ_ERR_*), > 0 = a hipError_t from the runtime.  aq_last_error() describes
 * the last failure of the calling thread.  The reference reports the same
 * conditions as Go errors ("HIP returned <rc>", go/engine/hip/hip_driver_cgo.go:1728-1730;
 * shape errors, go/engine/hip/hip_projection_reference.go:122-144).
 *
 * Threading: calls on one aq_ctx are serialised by an internal mutex; kernels
 * are enqueued on the context's stream and are asynchronous with respect to
 * the host unless the entry point says otherwise.
 */
#ifndef AQ_MI355_H
#define AQ_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AQ_OK 0
#define AQ_ERR_ARG (-1)         /* null pointer, negative size, misaligned pointer       */
#define AQ_ERR_SHAPE (-2)       /* dims do not describe a valid affine tensor            */
#define AQ_ERR_UNSUPPORTED (-3) /* valid, but no kernel for this width / group           */
#define AQ_ERR_INDEX (-4)       /* expert / row index out of range (host-visible ids)    */
#define AQ_ERR_NOMEM (-5)       /* host allocation failed                                */
#define AQ_ERR_NODEVICE (-6)    /* no usable gfx950 device                               */
#define AQ_ERR_SIZE (-7)        /* a host buffer length disagrees with the dims          */

#define AQ_OUT_F32 0x1u     /* y is float32 instead of bf16 (validation of the fp32 accumulator) */
#define AQ_IN_F32 0x2u      /* aq_moe_combine: the route rows are float32 instead of bf16           */
#define AQ_LOGITS_BF16 0x4u /* aq_moe_route: the router scores are bf16 instead of float32          */
#define AQ_BF16_STEPS 0x8u  /* aq_moe_combine: round every product and partial sum to bf16          */
#define AQ_W_TILED 0x10u    /* aq_qmv, aq_qmv_multi, aq_qmv_gate_up: the packed pointers are tile-major tensors
                               made by aq_tile_weights; they hold scales and biases too, so the scale and bias
                               arguments are not read (NULL will do)                                          */

typedef struct aq_ctx aq_ctx;

/* Library / error plumbing.  No reference counterpart beyond core.E strings. */
const char *aq_version(void);
const char *aq_last_error(void);

/* Context: device selection, one stream, timing events.
 * Replaces hipRuntime/cgoHIPDriver set-up (go/engine/hip/hip_runtime.go:21-50,
 * go/engine/hip/hip_driver_cgo.go:1667-1726: hipSetDevice, module load, function cache). */
int aq_create(int device, aq_ctx **out);
void aq_destroy(aq_ctx *ctx);
/* Enqueue on a caller-owned hipStream_t instead of the context's own stream
 * (pass NULL for the legacy default stream the reference launches on,
 * go/engine/hip/hip_driver_cgo.go:452-478).  aq_use_own_stream() goes back. */
int aq_use_stream(aq_ctx *ctx, void *hip_stream);
int aq_use_own_stream(aq_ctx *ctx);
int aq_device_name(aq_ctx *ctx, char *buf, size_t buf_len);

/* Device memory: nativeHIPDriver.Malloc / Free / CopyHostToDevice / CopyDeviceToHost
 * (go/engine/hip/hip_runtime.go:23-30).  Pointers are ordinary HIP device
 * pointers and may equally come from the caller's own hipMalloc. */
int aq_malloc(aq_ctx *ctx, size_t bytes, void **dptr);
int aq_free(aq_ctx *ctx, void *dptr);
int aq_h2d(aq_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);  /* synchronous */
int aq_d2h(aq_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);  /* synchronous */
int aq_d2d(aq_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes);   /* stream-ordered */
int aq_fill_zero(aq_ctx *ctx, void *dptr, size_t bytes);                     /* stream-ordered */
int aq_sync(aq_ctx *ctx);                                                    /* DeviceSynchronize, hip_launch.go:393-407 */

/* hipEvent pair on the context's stream: the per-kernel timing the reference
 * takes with a device synchronise per launch (go/engine/hip/hip_decode_route_metrics.go:17-52). */
int aq_timer_start(aq_ctx *ctx);
int aq_timer_stop(aq_ctx *ctx, float *elapsed_ms); /* records, waits, reports */

/* Launch batching: everything enqueued on the context between aq_capture_begin and
 * aq_capture_end is recorded into a HIP graph instead of being executed; aq_graph_launch
 * replays the whole batch with one submission.  Counterpart of the reference's per-step
 * launch batch (hipLaunchKernelContext batching, go/engine/hip/hip_launch.go:240-273,
 * cgoHIPDriver.LaunchKernelBatch go/engine/hip/hip_driver_cgo.go:1137-1190).  Only the
 * kernel entry points (aq_qmv*, aq_qmm, aq_gather_qmv*, aq_act_mul, aq_moe_*, aq_dequant_f32, aq_fill_zero, aq_d2d)
 * may be called while capturing; the pointers they were given must stay valid for replays.
 * Calls that go through the context's workspace (aq_qmm, aq_qmv with many rows, aq_packed_topk, aq_qmv_greedy,
 * the unfused fallbacks) record the workspace's address: the workspace cannot grow during a capture (the call
 * fails with a message), and when a later call makes it grow, every graph captured over the old block is
 * refused by aq_graph_launch with AQ_ERR_UNSUPPORTED - reserve the largest workspace first
 * (aq_reserve_workspace / aq_reserve_workspace_bytes), or capture again. */
typedef struct aq_graph aq_graph;
int aq_capture_begin(aq_ctx *ctx);
int aq_capture_end(aq_ctx *ctx, aq_graph **out);
int aq_graph_launch(aq_ctx *ctx, aq_graph *graph);
void aq_graph_destroy(aq_graph *graph);

/* Measurement aid with no counterpart in the reference: streams the codes, scales and biases of a 4-bit group-64
 * tensor [N, K] once through the load instructions of the single-row matvec and does nothing with them (no
 * activations, no arithmetic, no store).  Its time is what a launch that only reads that tensor costs on this device;
 * the benchmark reports the matvec beside the mode whose loads it issues.
 *   mode 0: MLX arrays, 64 contiguous bytes of each of 16 rows per instruction, plain loads (the matvec's loads on
 *           matrices under 16 MB)
 *   mode 1: MLX arrays, whole 128-byte lines of 8 rows per instruction with the non-temporal hint (its loads on
 *           larger matrices)
 *   mode 2: `packed` is a tile-major tensor (aq_tile_weights), read as 1 KiB of consecutive bytes per instruction with
 *           the hint (its loads on tile-major weights); scales and biases are not read and may be NULL
 *   mode 3: MLX arrays as consecutive 1 KiB pieces, plain loads
 * K a multiple of 1024.  Stream-ordered; writes nothing. */
int aq_probe_read(aq_ctx *ctx, const void *packed, const void *scales, const void *biases, int K, int N, int mode);

/* affine_qmv: y[M,N] = x[M,K] . dequant(w[N,K])^T, all operands device-resident.
 * Stands in for rocm_mlx_q4_projection / _batch launches
 * (go/engine/hip/hip_projection_launch.go:1306-1406, 2671-2720, 4907-5287) with the bf16
 * semantics of MLX affine_qmv (go/engine/metal/qmv.go:354-421) and the M-row
 * form (go/engine/metal/qmv_rows.go:14-60).  M >= 1; rows of x are contiguous.
 * N == 0 or K == 0 is a no-op returning AQ_OK (qmv.go:365-371). */
int aq_qmv(aq_ctx *ctx, const void *x, const void *packed, const void *scales, const void *biases, void *y, int M,
           int K, int N, int group_size, int bits, unsigned flags);

/* `count` (1..4) independent aq_qmv calls that share x, M, K, group size and width, in ONE launch:
 * y[i][M, N[i]] = x . dequant(packed[i], scales[i], biases[i])^T.  The arrays are host arrays of device
 * pointers.  Results are byte-identical to `count` separate aq_qmv calls.  This is the no-copy form of
 * running q|k|v or gate|up over model.ConcatQuantRows (go/model/quant_weight.go:32-62): at batch 1 the
 * narrow projections are bound by launch latency, not bandwidth, and one grid over all of them fills
 * the machine.  One launch for one activation row (up to four when K is a multiple of 128 between 1152 and 16384);
 * shapes the fused kernels do not take are run as separate launches. */
int aq_qmv_multi(aq_ctx *ctx, const void *x, int count, const void *const *packed, const void *const *scales,
                 const void *const *biases, void *const *y, const int *N, int M, int K, int group_size, int bits,
                 unsigned flags);

/* affine_qmm: same contract as aq_qmv, tuned for prefill-sized M
 * (go/engine/metal/quant_seam_backend.go:77-109 qmmTBF16Into; reference HIP
 * batch kernels go/engine/hip/kernels/quant/affine_projection_tuned.hipinc:166-1109).
 * Every element of y[M,N] is written, ragged N included. */
int aq_qmm(aq_ctx *ctx, const void *x, const void *packed, const void *scales, const void *biases, void *y, int M,
           int K, int N, int group_size, int bits, unsigned flags);

/* `count` (1..8) aq_qmm calls that share x, M, K, group size and width (q|k|v, gate|up at prefill; the no-copy form of
 * one matmul over model.ConcatQuantRows, go/model/quant_weight.go:32-62): y[i][M, N[i]] = x . dequant(packed[i], ...)^T.
 * The pass that rewrites x into MFMA operand order runs once for the members that need the same form of it instead of
 * once per member (10 us of a 290 us call at M = 2048, K = 4096); every y[i] is byte-identical to the separate
 * aq_qmm call.  Host arrays of device pointers, as in aq_qmv_multi.  Up to four rows run as aq_qmv_multi. */
int aq_qmm_multi(aq_ctx *ctx, const void *x, int count, const void *const *packed, const void *const *scales,
                 const void *const *biases, void *const *y, const int *N, int M, int K, int group_size, int bits,
                 unsigned flags);

/* Prefill-sized aq_qmm / aq_qmv calls (M >= 64) rewrite x into MFMA operand order first and keep that
 * copy (about M*K*2 bytes) in a workspace the context owns.  The workspace grows on demand, which
 * drains the stream and allocates: not allowed while a capture is open and unwelcome in a serving
 * loop.  This call sizes it ahead of time for activations of up to M x K.  The reference sizes its
 * own scratch the same way at model load (hipMLXQ4DeviceWeightConfig and the batch scratch of
 * go/engine/hip/hip_projection_launch.go:2671-2720). */
int aq_reserve_workspace(aq_ctx *ctx, int M, int K);
/* The same by size.  Besides the prefill copy of x the workspace holds: the fp32 partial tiles of calls with
 * 5..64 rows whose K is shared out over workgroups (up to 64*M*N bytes), the intermediates of the unfused
 * fallbacks of the fused MLP / lm_head entry points, and the scratch of aq_packed_topk.  A call that needs
 * more than is there grows it (not possible while a capture is open): run such a call once before capturing,
 * or reserve its bytes here. */
int aq_reserve_workspace_bytes(aq_ctx *ctx, size_t bytes);
/* Device bytes the context holds as scratch right now (the workspace above plus the partial maxima of
 * aq_qmv_greedy): lets a caller, or a test, see whether a call made either of them grow.  No reference counterpart. */
size_t aq_workspace_bytes(aq_ctx *ctx);

/* gather_qmv: for each route z, y[z,:N] = x[lhs[z] or 0, :K] . dequant(W_e)^T with
 * e = rhs[z] read ON DEVICE; W_e = rows [row_base, row_base+N) of expert e's slab.
 *   packed [num_experts, expert_rows, K*bits/32], scales/biases [num_experts, expert_rows, K/group]
 *   lhs, rhs: device int32[routes]; lhs may be NULL (every route reads x row 0)
 * Semantics: go/engine/metal/kernels/moe/lthn_gather_qmv.metal:54-66,
 * go/engine/metal/qmv_gather.go:295-313; replaces the host-grouped
 * rocm_moe_mlx_affine_routes path (go/engine/hip/hip_gemma4_moe.go:294-446).
 * A route whose expert id or x row is out of range yields zeros (the host
 * cannot see device ids; the by-index helper of qmv_gather.go:405-409 checks
 * on the host instead). */
int aq_gather_qmv(aq_ctx *ctx, const void *x, const void *packed, const void *scales, const void *biases,
                  const int32_t *lhs, const int32_t *rhs, void *y, int routes, int x_rows, int K, int N,
                  int num_experts, int expert_rows, int row_base, int group_size, int bits, unsigned flags);

/* Activation kinds of the fused MLP entry points below.  GELU is the tanh approximation
 * 0.5*v*(1 + tanh(0.7978845608028654*(v + 0.044715*v^3))) of rocm_gelu_tanh_value
 * (go/engine/hip/kernels/common/math.hipinc:3-9); SiLU is v / (1 + exp(-v))
 * (go/model/attn/gated_delta.go:228). */
#define AQ_ACT_GELU_TANH 1
#define AQ_ACT_SILU 2

/* Fused gate|up projection with the activation as epilogue:
 *   y[m,n] = act(x[m,:] . dequant(gate)[n,:]) * (x[m,:] . dequant(up)[n,:])
 * both sums in fp32, the activation and the product in fp32, one rounding at the store.  Replaces
 * rocm_mlx_q4_gelu_tanh_multiply and its batch form (go/engine/hip/kernels/quant/affine_gelu_tanh.hipinc:3-182,
 * launch go/engine/hip/hip_projection_launch.go:3086-3160, packet contract/launch_abi.hipinc:634-657).
 * gate and up are [N, K*bits/32] with their own scales/biases; for a row-concatenated gate|up slab
 * (model.ConcatQuantRows, go/model/quant_weight.go:32-62) pass the slab for gate and slab + N rows for up.
 * M == 1 with 4/8-bit codes (up to 4 rows of 4-bit group-64 codes when K is a multiple of 256 between 1280 and 8192) runs as ONE launch
 * that reads every weight once; other shapes run the two
 * projections and the element-wise step as separate launches through the context's workspace (which grows
 * on demand like aq_qmm's; not while a capture is open). */
int aq_qmv_gate_up(aq_ctx *ctx, const void *x, const void *gate_packed, const void *gate_scales,
                   const void *gate_biases, const void *up_packed, const void *up_scales, const void *up_biases,
                   void *y, int M, int K, int N, int group_size, int bits, int act, unsigned flags);

/* The same fusion with expert ids read on the device: for each route z, with e = rhs[z],
 *   y[z,:N] = act(x_z . gate_e^T) * (x_z . up_e^T)
 * where gate_e / up_e are rows [gate_row_base, +N) / [up_row_base, +N) of expert e's slab (a fused
 * gate|up slab has expert_rows = 2N, gate_row_base = 0, up_row_base = N).  Stands in for the gate|up
 * half of rocm_moe_mlx_affine_routes (go/engine/hip/kernels/moe/routing.hipinc:160-399, store :312) and for
 * the two emitGatherQMVAllRoutes + gelu dispatches of go/engine/metal/moe_block.go:2344-2358.
 * Index rules as aq_gather_qmv. */
int aq_gather_qmv_gate_up(aq_ctx *ctx, const void *x, const void *packed, const void *scales, const void *biases,
                          const int32_t *lhs, const int32_t *rhs, void *y, int routes, int x_rows, int K, int N,
                          int num_experts, int expert_rows, int gate_row_base, int up_row_base, int group_size,
                          int bits, int act, unsigned flags);

/* Projection whose input is formed on the fly: y[m,:N] = bf16(act(g[m,:]) * u[m,:]) . dequant(w)^T, where g and
 * u are the bf16 gate and up activations [M, K].  The gated value is rounded to bf16 once, exactly as the
 * stand-alone aq_act_mul stores it, so the result is byte-identical to aq_act_mul followed by aq_qmv.
 * Replaces lthn_gelu_qmv (emitGeluQMV, go/engine/metal/dispatch_sink.go:533-552; x-load
 * go/engine/metal/kernels/moe/lthn_gelu_qmv_impl.h:24-33). */
int aq_qmv_act(aq_ctx *ctx, const void *gate_x, const void *up_x, const void *packed, const void *scales,
               const void *biases, void *y, int M, int K, int N, int group_size, int bits, int act, unsigned flags);

/* The gathered form, lthn_gather_qmv_gelu (go/engine/metal/kernels/moe/lthn_gather_qmv.metal:98-132,
 * emitLthnGatherQMVGeluRoutes go/engine/metal/qmv_gather.go:319-345): gate_x and up_x are [x_rows, K] and
 * ride the same lhs indexing. */
int aq_gather_qmv_act(aq_ctx *ctx, const void *gate_x, const void *up_x, const void *packed, const void *scales,
                      const void *biases, const int32_t *lhs, const int32_t *rhs, void *y, int routes, int x_rows,
                      int K, int N, int num_experts, int expert_rows, int row_base, int group_size, int bits,
                      int act, unsigned flags);

/* y[i] = bf16(act(gate[i]) * up[i]) over n bf16 values: rocm_gelu_tanh_multiply
 * (go/engine/hip/hip_transformer_launch.go:3765) / lthn_gelu_gate_mul_bf16, host mirror
 * hostGeluMul (go/engine/metal/ffn_megakernel_test.go:17-31). */
int aq_act_mul(aq_ctx *ctx, const void *gate, const void *up, void *y, int64_t n, int act);

/* Device MoE router: for each of `rows` tokens, the top_k experts by (score descending, expert id
 * ascending on ties) and their weights, written where aq_gather_qmv* read them, so no score ever visits the
 * host.  logits [rows, num_experts] float32 (bf16 with AQ_LOGITS_BF16), device-resident.
 *   ids            int32 [rows, top_k]   -> the `rhs` of the gathers
 *   weights        float [rows, top_k]   -> aq_moe_combine
 *   token_of_route int32 [rows, top_k]   (may be NULL) = the row, i.e. the `lhs` of the gate|up gather
 * normalise_top_k != 0: weights = softmax over the selected scores (rocm_moe_router,
 * go/engine/hip/kernels/moe/routing.hipinc:3-77; CPU form rocmReferenceRouteExperts,
 * go/engine/hip/moe_quant_reference.go:27-78); == 0: softmax over all experts, gathered, not renormalised
 * (hipQwen3MoERouterSelect, go/engine/hip/hip_qwen3_moe_router.go:25-88).  expert_scales (device float
 * [num_experts], may be NULL) multiplies each weight by its expert's scale, as
 * hipGemma4MoEBatchRouteGroups does on the host (go/engine/hip/hip_gemma4_moe.go:294-366) - the D2H copy,
 * host grouping and chunk upload of that path are what this call removes.  num_experts <= 1024,
 * top_k <= 64.  A NaN score ranks last; the reference rejects non-finite scores on the host, which a
 * device-resident router cannot do. */
int aq_moe_route(aq_ctx *ctx, const void *logits, int rows, int num_experts, int top_k, const float *expert_scales,
                 int normalise_top_k, int32_t *ids, float *weights, int32_t *token_of_route, unsigned flags);

/* MoE combine: out[row, :n] = sum over rank of route_rows[row*top_k + rank, :n] * weights[row*top_k + rank],
 * ranks ascending, fp32 (rocm_moe_batch_scatter_routes + rocm_moe_batch_reduce_routes,
 * go/engine/hip/kernels/moe/routing.hipinc:100-158).  route_rows is the down gather's output: bf16, or
 * float32 with AQ_IN_F32; out is bf16, or float32 with AQ_OUT_F32.  AQ_BF16_STEPS rounds the weight, every
 * product and every partial sum to bf16, which reproduces lthn_moe_weighted_sum_bf16 byte for byte
 * (go/engine/metal/kernels/moe/lthn_moe_weighted_sum.metal:17-38). */
int aq_moe_combine(aq_ctx *ctx, const void *route_rows, const float *weights, void *out, int rows, int top_k, int n,
                   unsigned flags);

/* lm_head with the argmax fused in: best[m] = max over vocabulary rows n of pack(score[m,n], n), where
 * score = x[m,:] . dequant(w)[n,:] in fp32 and pack() is aq_pack_best's layout (score key in the high word,
 * ~n in the low word, so the highest score wins and equal scores go to the lowest token id, the order of
 * hipReferenceGreedySample, go/engine/hip/hip_transformer_reference.go:401-437).  Non-finite scores and the
 * token ids listed in `suppress` (device int32[suppress_count], may be NULL) never win; best[m] == 0 means no
 * row qualified.  best is device uint64[M]; the call clears it itself.  Replaces
 * rocm_mlx_q4_projection_greedy / _greedy_batch (go/engine/hip/kernels/quant/affine_projection_fused.hipinc:190-410):
 * for M == 1 and 4/8-bit codes 8 bytes leave the kernel instead of N logits; other shapes run the projection
 * into the context's workspace and reduce it there.  Greedy calls on one context share one set of partial
 * maxima and fold tickets: they must be ordered with each other on the stream (no greedy call, direct or
 * inside a replayed graph, may overlap another one of the same context). */
int aq_qmv_greedy(aq_ctx *ctx, const void *x, const void *packed, const void *scales, const void *biases,
                  const int32_t *suppress, int suppress_count, uint64_t *best, int M, int K, int N, int group_size,
                  int bits);

/* Greedy over a list of candidate rows (speculative or constrained decoding): best[0] = max over the candidates r of
 * pack(x . dequant(w)[r,:], r), rows being a device int32[count] read on the device.  Ids outside [0, N) are skipped,
 * duplicates are harmless, non-finite scores never win, best[0] == 0 means no candidate qualified; ties go to the lowest
 * row id (the packing's order).  Replaces rocm_mlx_q4_projection_selected_greedy
 * (go/engine/hip/kernels/quant/affine_projection_fused.hipinc:485-546; like it, this form has no suppress list: the
 * list IS the selection).  One activation row.  A candidate is scored by the gathered matvec as one row of a window of
 * 16 weight rows, so it costs 16 rows of weights; scratch comes from the context's workspace (count * 68 bytes; grows
 * on demand, not during capture).  count <= 65535. */
int aq_qmv_greedy_selected(aq_ctx *ctx, const void *x, const void *packed, const void *scales, const void *biases,
                           const int32_t *rows, int count, uint64_t *best, int K, int N, int group_size, int bits);

/* aq_qmv_greedy for one activation row with NO allocation of any kind (no hipMalloc / hipFree, no workspace
 * growth): it has no counterpart in the reference and exists for callers that cannot allocate - code under
 * HIP graph capture, tight serving loops, harnesses that forbid it.  The partial maxima and the fold tickets
 * live in a static device array of 2 MiB + 1 KiB that every GPU the library has a context on holds until the
 * process ends.  Limits: M == 1; 4- or 8-bit codes whose rows are 16-byte aligned (the shapes the fused
 * kernels take, anything else returns AQ_ERR_UNSUPPORTED); at most 262144 partial maxima (one per 16 rows for
 * 4-bit group-32/64 codes with K > 1024, else one per 1..4 rows), i.e. vocabularies of up to 4 M rows on the
 * fast path and at least 262144 rows otherwise: beyond that AQ_ERR_SIZE.  A variant forced with aq_force_variant
 * is not consulted (the fused kernels are the only route that needs no scratch).  best[0] is bit-identical to
 * aq_qmv_greedy's.  All calls on one GPU share that GPU's array (also across contexts): calls that overlap on
 * one GPU race; order them on one stream. */
int aq_qmv_greedy_static(aq_ctx *ctx, const void *x, const void *packed, const void *scales, const void *biases,
                         const int32_t *suppress, int suppress_count, uint64_t *best, int K, int N, int group_size,
                         int bits);

/* The same projection storing every row's packed (score, row): scores is device uint64[M, N]; suppressed or
 * non-finite rows hold 0.  rocm_mlx_q4_projection_scores (affine_projection_fused.hipinc:411-446), the input
 * of top-k sampling. */
int aq_qmv_scores(aq_ctx *ctx, const void *x, const void *packed, const void *scales, const void *biases,
                  const int32_t *suppress, int suppress_count, uint64_t *scores, int M, int K, int N, int group_size,
                  int bits);

/* The top_k (1..64) largest of `count` packed values, sorted descending, into device out[top_k]; fewer than
 * top_k non-zero inputs leave zeros at the end.  rocm_packed_topk (go/engine/hip/kernels/sampling/topk.hipinc:45-84)
 * applied chunk by chunk until one chunk is left; scratch comes from the context's workspace. */
int aq_packed_topk(aq_ctx *ctx, const uint64_t *scores, int64_t count, int top_k, uint64_t *out);

/* Temperature / top-p sampling over the list aq_packed_topk wrote (descending packed values, zeros = no candidate),
 * the device sampler rocm_packed_topk_sample (go/engine/hip/kernels/sampling/topk.hipinc:86-191, launched by
 * hipRunPackedTopKSampleKernel, go/engine/hip/hip_projection_launch.go:4538): weights exp(score / temperature -
 * max) in double over the soft-capped scores (softcap 0 = none), the nucleus cut at cumulative / total >= top_p,
 * then the candidate whose cumulative weight first reaches draw * (sum of the kept weights); `draw` in [0, 1) comes
 * from the caller's generator, so a run is reproducible.  temperature <= 0 and top_p <= 0 together select the first
 * candidate (greedy); a zero of either alone stands for 1.  out[0] (device) receives the chosen packed value, to
 * be read with aq_unpack_best; 0 when nothing can be sampled.  Argument rules of topk_validate.hipinc:53-77:
 * top_k 1..128 (AQ_ERR_SHAPE / AQ_ERR_UNSUPPORTED), temperature >= 0 finite, top_p in [0, 1], softcap >= 0
 * finite, draw finite (AQ_ERR_ARG).  Sums run in list order as in the reference; exp and tanh are the device
 * library's double-precision ones.  Stream-ordered, may be captured. */
int aq_packed_topk_sample(aq_ctx *ctx, const uint64_t *top, int top_k, float temperature, float top_p, float softcap,
                          double draw, uint64_t *out);

/* Host-side codec of the packed values: hipPackGreedyBest / hipUnpackGreedyBest
 * (go/engine/hip/hip_projection_launch.go:2393-2416).  Unpacking rejects packed == 0 ("did not produce a
 * result"), a token outside [0, vocab_size) and a negative or non-finite softcap; softcap > 0 returns
 * tanh(score / softcap) * softcap. */
uint64_t aq_pack_best(float score, int token);
int aq_unpack_best(uint64_t packed, float softcap, int vocab_size, int *token, float *score);

/* A quantised weight resident on the device, the three arrays every kernel entry point takes.
 * experts == 0: [rows, ...]; experts > 0: an expert slab [experts, rows, ...] for the gathers. */
typedef struct aq_device_linear {
    void *weight, *scales, *biases;
    int rows, in_dim, group_size, bits, experts;
} aq_device_linear;
struct aqh_linear; /* include/aq_mi355_host.h */

/* Uploads one loaded weight (aqh_load_linear) straight from its file mapping: the device-binding half of the
 * loader (the reference hands model.Linear's mmap views to hipUploadByteBuffer,
 * go/engine/hip/hip_projection_launch.go:3086-3124 deviceBuffers).  Synchronous.  Dense (unquantised) weights are
 * rejected with AQ_ERR_UNSUPPORTED. */
int aq_upload_linear(aq_ctx *ctx, const struct aqh_linear *lin, aq_device_linear *out);

/* Uploads gate and up as ONE slab whose experts hold [gate rows | up rows] (rank-2 weights: one "expert"), the
 * layout aq_qmv_gate_up / aq_gather_qmv_gate_up read with up_row_base = rows.  This is the fused expert
 * gate+up tensor the reference synthesises on the heap at load when a checkpoint ships them apart
 * (Arch.FuseExpertGateUp, go/model/arch.go:167; row concatenation model.ConcatQuantRows,
 * go/model/quant_weight.go:45-63); here the interleave happens in the copy itself (strided H2D), with no
 * host copy of the weights.  out->rows is 2 * the rows of each part. */
int aq_upload_fused_gate_up(aq_ctx *ctx, const struct aqh_linear *gate, const struct aqh_linear *up, aq_device_linear *out);

int aq_free_device_linear(aq_ctx *ctx, aq_device_linear *lin);

/* GGUF block tensors -> affine tensors on the device, for checkpoints that ship Q4_0 / Q4_1 / Q8_0 / Q4_K / Q5_K /
 * Q6_K blocks (or F32, quantised to eight bits in groups of 32) instead of MLX-affine triples.  Replaces the
 * host round trip of synthesizeGemma4GGUFAffineTensor (go/engine/hip/hip_gguf_affine_adapter.go:199-218: device
 * -> host copy, hipRepackGGUFKQuantToAffine :321-341 on the CPU, three uploads) with one kernel over the tensor
 * where it lies; the three outputs are bit-identical to that function's payload (Weights / Scales / Biases,
 * :61-71): Q4_0 -> 4 bits, group 32, bias -8*d; Q4_1 -> 4 bits, group 32; Q8_0 -> 8 bits, group 32, codes
 * q + 128, bias -128*d; Q4_K -> 4 bits, group 32, scale d*sc, bias -dmin*m; Q5_K -> 6-bit fields holding
 * five-bit codes, group 32; Q6_K -> 6 bits, group 16, bias -32*scale; F32 -> min/max quantiser.
 * gguf_type is GGUF's tensor type id (F32 0, Q4_0 2, Q4_1 3, Q8_0 8, Q4_K 12, Q5_K 13, Q6_K 14).  rows and
 * cols are the tensor's (GGUF lists the dimensions as [cols, rows]); stacked expert tensors pass experts * rows.
 * aq_gguf_affine_layout_of needs no device: it tells the caller what to allocate.
 * Errors as the reference raises them: another type AQ_ERR_UNSUPPORTED; cols not a whole number of blocks (32,
 * or 256 for the K formats) or non-positive dims AQ_ERR_SHAPE; src_bytes != rows * blocks * block bytes
 * AQ_ERR_SHAPE.  packed must be 16-byte aligned, F32 input 4-byte aligned.  Stream-ordered, may be captured. */
typedef struct aq_gguf_affine_layout {
    int bits, group_size;
    int64_t packed_cols, groups;                   /* uint32 words per row, groups per row */
    uint64_t src_bytes, packed_bytes, scales_bytes; /* scales_bytes is also the size of biases */
} aq_gguf_affine_layout;
int aq_gguf_affine_layout_of(int gguf_type, int64_t rows, int64_t cols, aq_gguf_affine_layout *out);
int aq_gguf_to_affine(aq_ctx *ctx, int gguf_type, const void *src, uint64_t src_bytes, int64_t rows, int64_t cols,
                      void *packed, void *scales, void *biases);

/* A device layout made once at load time, as the reference synthesises the device layouts of GGUF tensors at load
 * (go/engine/hip/hip_gguf_affine_adapter.go:199-218).  The tile-major form of a 4-bit group-64 tensor (K a multiple
 * of 128) stores, for every set of 16 rows and every step of K that one wavefront of the matvec kernels works on, the
 * codes AND that step's scales and biases as one contiguous tile whose every KiB is in lane order, so a load
 * instruction of a wavefront takes 1 KiB of consecutive bytes instead of 64 bytes of each of 16 rows (the MLX
 * row-major arrays cost the single-row projection 4096 -> 14336 about 1.5 us of 8).  aq_tiled_bytes gives the
 * size of the tile-major tensor (as many bytes as the three MLX arrays when N is a multiple of 16; -1 when the
 * geometry has no such form); aq_tile_weights writes it from the MLX arrays (device to device, stream-ordered, may
 * be captured); aq_untile_weights is its exact inverse.  Calls that take AQ_W_TILED compute the same bytes as the
 * same call on the MLX arrays (same kernels, same order of additions); shapes no tile-major kernel takes (more
 * than eight rows of x, K beyond 16384, forced variants of other families) rebuild the MLX arrays in the context's
 * workspace first (one extra pass over the tensor; the workspace grows on demand, not during capture). */
int64_t aq_tiled_bytes(int64_t N, int K, int group_size, int bits);
int aq_tile_weights(aq_ctx *ctx, const void *packed, const void *scales, const void *biases, int64_t N, int K,
                    int group_size, int bits, void *tiled);
int aq_untile_weights(aq_ctx *ctx, const void *tiled, int64_t N, int K, int group_size, int bits, void *packed,
                      void *scales, void *biases);
/* The load-time step for a weight uploaded with aq_upload_linear / aq_upload_fused_gate_up (rank-2 weights only): its
 * three arrays are replaced by one tile-major tensor in lin->weight, lin->scales and lin->biases become NULL, and the
 * calls on it take AQ_W_TILED (a fused gate|up slab whose halves have a multiple of 16 rows is one tile-major tensor:
 * the up half starts aq_tiled_bytes(rows / 2, ...) bytes in).  Synchronous; the device holds both forms for the
 * duration of the call.  AQ_ERR_UNSUPPORTED for expert slabs (the gathers read MLX arrays) and for geometries with no
 * tile-major form. */
int aq_tile_device_linear(aq_ctx *ctx, aq_device_linear *lin);

/* mlxaffine.DequantizeTensor on device (go/model/quant/mlxaffine/mlxaffine.go:178-208):
 * out_f32[N,K] = scale*code + bias, bit-exact with the CPU path. */
int aq_dequant_f32(aq_ctx *ctx, const void *packed, const void *scales, const void *biases, float *out_f32, int64_t N,
                   int K, int group_size, int bits);

/* model.QuantMatVec.MatVec with HOST byte slices (go/model/quant.go:35-38): uploads,
 * runs aq_qmv with M = 1, downloads out_dim*2 bf16 bytes into out, synchronous.
 * Lengths are checked like enginetest.ReferenceAffineMatVec checks them
 * (go/engine/enginetest/quant_reference.go:78-106); out_dim == 0 or in_dim == 0
 * returns AQ_OK and writes nothing. */
int aq_matvec_host(aq_ctx *ctx, const uint8_t *x, size_t x_len, const uint8_t *packed, size_t packed_len,
                   const uint8_t *scales, size_t scales_len, const uint8_t *biases, size_t biases_len, int out_dim,
                   int in_dim, int group_size, int bits, uint8_t *out, size_t out_len);

/* attn.ProjQuantMatMulInto with HOST slices (go/model/attn/gated_delta.go:46-58), behaviour of
 * native.MatMulQuantF32NTInto (go/engine/metal/quant_seam_backend.go:37-75): x f32 [M,K] is
 * rounded to bf16 (RNE), M == 1 runs qmv and M > 1 qmm, the bf16 result is widened
 * into out f32 [M,N].  Synchronous. */
int aq_proj_quant_matmul_host(aq_ctx *ctx, float *out, const float *x, size_t x_len, const uint8_t *packed,
                              size_t packed_len, const uint8_t *scales, size_t scales_len, const uint8_t *biases,
                              size_t biases_len, int M, int K, int N, int group_size, int bits);

/* Kernel-variant introspection and override, for tuning sweeps and profiles.
 * op: 0 = qmv/gather (matvec kernel families), 1 = qmm (matmul kernel families).  variant -1 restores automatic
 * selection (the counterpart of the reference's shape->kernel selector tables,
 * go/engine/hip/hip_projection_launch.go:4925-5064).
 * Route switches (the reference's GO_ROCM_DISABLE_* variables, hip_projection_launch.go:95-137): the environment
 * variable AQ_MI355_DISABLE=name[,name...] over dot2, blk, diag, tok, tiles is read by aq_create and takes those
 * kernel families out of that context's selection; a call then runs on the next family that takes its shape (the
 * any-width kernel at the end cannot be switched off).  aq_qmm with five rows and more is not affected, and the
 * fused head, gate|up and multi-matrix calls honour `diag` only (their dot2 kernels have no switch).  There is
 * no code-object override (GO_ROCM_KERNEL_HSACO, hip_kernel_module.go:14-35): the kernels are part of the library. */
int aq_variant_count(int op);
const char *aq_variant_name(int op, int variant);
int aq_force_variant(aq_ctx *ctx, int op, int variant);
/* Name of the kernel variant the last launch of `op` on this context used; an aq_qmv call with more than
 * four rows that ran on the matmul tiles reports the tile kernel under both ops. */
const char *aq_last_variant(aq_ctx *ctx, int op);

#ifdef __cplusplus
}
#endif
#endif
