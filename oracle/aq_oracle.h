/*
 * aq_oracle.h -- CPU restatement of go-inference's MLX group-affine quantized
 * dequant / matvec / matmul / gather path.
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the GPU kernels are compared
 * against and the CPU baseline the benchmark times.  Nothing the product ships
 * may call, link or import it: only tests/, the smoke check and the benchmark's
 * cpu_baseline leg load liborc.so.
 *
 * Every function names the reference file:line whose arithmetic it restates
 * (paths relative to the go-inference checkout).  Build: `make -C oracle`
 * (gcc, -ffp-contract=off so no multiply-add is fused behind the algorithm's
 * back).
 *
 * Layout used everywhere (go/model/quant/mlxaffine/mlxaffine.go:14-20):
 *   packed  uint32 little-endian [N, K*bits/32]; code p of a word sits at bits
 *           [p*bits, p*bits+bits), LSB first, along K
 *   scales  bf16 [N, K/group]      biases  bf16 [N, K/group]
 *   w[n,k] = scale[n,k/group] * code[n,k] + bias[n,k/group]
 *
 * Return value of every int function: 0 = ok, negative = rejected argument
 * (the reference returns a Go error in the same situations).
 */
#ifndef AQ_ORACLE_H
#define AQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_OK 0
#define ORC_ERR_BITS (-1)  /* unsupported code width            */
#define ORC_ERR_DIMS (-2)  /* non-positive / non-dividing dims  */
#define ORC_ERR_SIZE (-3)  /* a buffer length disagrees         */
#define ORC_ERR_INDEX (-4) /* expert / row index out of range   */

/* bf16 codecs: mlxaffine.go:229-241, quant_reference.go:22-34,
 * hip_bf16_portable.go:12-23.  Round-to-nearest-even, NaN -> quiet NaN. */
uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t h);

/* LSB-first code extraction over a bit-contiguous byte row, any width 1..8,
 * codes may straddle bytes: quant_reference.go:36-52 (affineExtractCode). */
uint32_t orc_extract_code(const uint8_t *row, int64_t bit_off, int bits);
/* inverse, used to build fixtures: quant_reference.go:54-68 (affineSetCode). */
void orc_set_code(uint8_t *row, int64_t bit_off, int bits, uint32_t code);

/* uint32-word code extraction incl. codes that cross a word boundary (6-bit):
 * hip_projection_reference.go:200-222 (hipMLXAffineUnpackValue). */
int orc_unpack_word_value(const uint32_t *row_words, int64_t n_words, int col, int bits, uint32_t *code);

/* mlxaffine.DequantizeTensor, mlxaffine.go:178-208.  bits in {1,2,4,8}.
 * packed_len / sb_len are byte lengths and are checked exactly as the
 * reference checks its slices.  out holds out_dim*in_dim float32. */
int orc_dequantize(const uint8_t *packed, size_t packed_len, const uint8_t *scales, size_t scales_len,
                   const uint8_t *biases, size_t biases_len, int out_dim, int in_dim, int bits, int group_size,
                   float *out);

/* mlxaffine.QuantizeTensor, mlxaffine.go:80-176 (affineGroup edge anchoring,
 * round-half-away codes).  Only used to build realistic fixtures. */
int orc_quantize(const float *values, size_t n_values, int out_dim, int in_dim, int bits, int group_size,
                 uint8_t *packed, uint8_t *scales, uint8_t *biases);

/* mlxaffine.RepackB1ToB2, repack.go:27-62: widen 1-bit codes to 2-bit fields. */
int orc_repack_b1_to_b2(const uint8_t *packed, size_t packed_len, int out_dim, int in_dim, uint8_t *packed2);

/* attn.matNTQuantHost, gated_delta.go:63-89: the reference's CPU qmv/qmm.
 * Per output row n: fp32 dequant of the row, then for each activation row m an
 * ascending-k float64 dot, stored as float32 at out[m*N+n].
 * threads <= 1: the single-threaded loop the Go original runs.
 * threads  > 1: the same loop with output rows shared out over OpenMP threads
 * (each row's arithmetic is unchanged, so results are bit-identical). */
int orc_matnt_quant_host(float *out, const float *x, const uint8_t *packed, const uint8_t *scales,
                         const uint8_t *biases, int M, int K, int N, int group_size, int bits, int threads);

/* enginetest.ReferenceAffineMatVec, quant_reference.go:78-127: bf16 x, weight
 * formed in float64 (no fp32 rounding of w), float64 accumulate, bf16 result.
 * Any width 1..8 over bit-contiguous rows.  Zero out_dim/in_dim: ok, nothing
 * written.  x_len etc. are byte lengths. */
int orc_reference_affine_matvec(const uint8_t *x, size_t x_len, const uint8_t *packed, size_t packed_len,
                                const uint8_t *scales, size_t scales_len, const uint8_t *biases, size_t biases_len,
                                int out_dim, int in_dim, int group_size, int bits, uint8_t *out);

/* hip.hipReferenceMLXAffineProjection, hip_projection_reference.go:92-116 with
 * the shape validation of :122-144 -- fp32 weight, fp32 ascending-col
 * accumulate ("the fp32-accumulated reference").  bits in {4,6,8}.  Lengths
 * are element counts, as in the Go signature. */
int orc_hip_reference_projection(const float *input, size_t input_len, const uint32_t *weights, size_t weight_len,
                                 const uint16_t *scales, size_t scale_len, const uint16_t *biases, size_t bias_len,
                                 int rows, int cols, int group_size, int bits, float *output);

/* Batched form of the same projection as the reference batch kernels are
 * tested with (hip_kernels_test.go:612-654): out[m*rows + r]. */
int orc_hip_reference_projection_batch(const float *input, int tokens, const uint32_t *weights,
                                       const uint16_t *scales, const uint16_t *biases, int rows, int cols,
                                       int group_size, int bits, float *output);

/* Expert-gathered matvec.  Addressing: lthn_gather_qmv.metal:54-66 (expert
 * slab offsets from rhs[z], x row from lhs[z] when batched, y row z) and the
 * range check of qmv_gather.go:401-409.  Arithmetic per route is the fp64
 * form of orc_reference_affine_matvec; out_f64 (optional) receives the
 * unrounded sums, out_bf16 (optional) the bf16 stores.
 *   packed [E, expert_rows, K*bits/32] u32, scales/biases [E, expert_rows, K/group]
 *   row_base selects rows [row_base, row_base+N) of each expert's slab
 *   lhs == NULL -> every route reads x row 0 */
int orc_gather_qmv(const uint16_t *x, int x_rows, const uint32_t *packed, const uint16_t *scales,
                   const uint16_t *biases, const int32_t *lhs, const int32_t *rhs, int routes, int num_experts,
                   int expert_rows, int row_base, int N, int K, int group_size, int bits, double *out_f64,
                   uint16_t *out_bf16);

/* Activations of the fused MLP kernels. */
#define ORC_ACT_GELU_TANH 1
#define ORC_ACT_SILU 2

/* act(gate) * up over fp32 vectors, the expectation the reference's fused gate|up kernels are tested
 * against.  GELU: expectedGELUTanhMultiply, hip_kernels_test.go:8127-8137 -- the tanh-approximated GELU
 * evaluated in float64 from the fp32 gate, rounded to float32, then one float32 multiply by up.
 * SiLU: the same composition with gdSilu, gated_delta.go:228 (v / (1 + exp(-v)) in float64). */
int orc_act_multiply(int act, const float *gate, const float *up, int64_t n, float *out);

/* bf16(act(gate) * up) over bf16 vectors with fp32 internals and one rounding at the store: hostGeluMul,
 * go/engine/metal/ffn_megakernel_test.go:17-31 (mirror of lthn_gelu_gate_mul_bf16 and of the x-load of
 * lthn_gelu_qmv_impl.h:24-33); tanh is taken in float64 and rounded to float32 as there.  SiLU keeps the
 * structure with expf's role played by float64 exp rounded to float32. */
int orc_act_gate_mul_bf16(int act, const uint16_t *gate, const uint16_t *up, int64_t n, uint16_t *out);

/* MoE router, one call over `rows` token rows.  Selection: the top_k experts by (score descending, expert
 * id ascending) -- rocmReferenceRouteExperts' stable sort, go/engine/hip/moe_quant_reference.go:27-55, the
 * same order hipGemma4MoEBatchRouteGroups' insertion keeps (hip_gemma4_moe.go:318-342).
 * normalise != 0: softmaxFloat32 over the selected scores (moe_quant_reference.go:268-286: float64 exp of
 * the float32 difference, stored as float32, divided by the float64 sum); == 0: hipQwen3MoERouterSelect
 * with normalise=false (hip_qwen3_moe_router.go:33-45,78-85): float64 softmax over all experts, gathered.
 * expert_scales (may be NULL): weight = prob * scale in float32, hip_gemma4_moe.go:356-360.
 * Rejects non-finite scores (ORC_ERR_INDEX) as both Go routers do. */
int orc_moe_route(const float *logits, int rows, int num_experts, int top_k, const float *expert_scales, int normalise,
                  int32_t *ids, float *weights);

/* MoE combine.  bf16_steps == 0: out[row,c] = sum over rank (ascending) of float32(in * weight), float32
 * adds: rocm_moe_batch_scatter_routes + rocm_moe_batch_reduce_routes, kernels/moe/routing.hipinc:100-158.
 * bf16_steps != 0: lthn_moe_weighted_sum_bf16, go/engine/metal/kernels/moe/lthn_moe_weighted_sum.metal:17-38
 * (weight, each product and each partial sum rounded to bf16).  in/out are float32 here; the caller
 * widens / narrows bf16 storage. */
int orc_moe_combine(const float *route_rows, const float *weights, int rows, int top_k, int n, int bf16_steps,
                    float *out);

/* Packed (score, token) values of the fused lm_head kernels: hipOrderedFloat32Key / hipPackGreedyBest /
 * hipUnpackGreedyBest, go/engine/hip/hip_projection_launch.go:2375-2416 (device side
 * kernels/common/numeric.hipinc:84-104).  Unsigned comparison of packed values orders by score, then by
 * lower token id.  Unpack returns ORC_ERR_DIMS for a non-positive vocab, ORC_ERR_INDEX for packed == 0 or
 * a token outside the vocab, ORC_ERR_SIZE for a bad softcap. */
uint64_t orc_pack_greedy_best(float score, int token);
int orc_unpack_greedy_best(uint64_t packed, float softcap, int vocab_size, int *token, float *score);

/* hipReferenceGreedySample / hipReferenceGreedySampleSuppress, go/engine/hip/hip_transformer_reference.go:401-437:
 * first maximum wins; suppressed tokens are skipped; ORC_ERR_DIMS without logits, ORC_ERR_INDEX when every
 * token is suppressed. */
int orc_greedy_sample_suppress(const float *logits, int n, const int32_t *suppress, int suppress_count, int *index,
                               float *value);

/* GGUF block formats -> the affine layout, the synthesis the HIP engine's loader runs on the host
 * (hipRepackGGUFKQuantToAffine, go/engine/hip/hip_gguf_affine_adapter.go:321-341): Q4_0 (:342-397), Q4_1
 * (:399-455), Q4_K (:457-502, block :722-751), Q5_K (:504-549, block :753-772, codes :801-820, six-bit fields),
 * Q6_K (:551-596, block :774-791, codes :822-841, groups of 16), Q8_0 (:598-648), F32 quantised to eight bits
 * (:650-720); the 6-bit scale/min unpack :793-799; code placement hipPutAffinePackedValue :843-857; half to
 * float hipFloat16ToFloat32, go/engine/hip/hip_projection_reference.go:240-261; float to bf16 WITHOUT a NaN case,
 * hipFloat32ToBFloat16, go/engine/hip/hip_bf16_portable.go:19-23.  `type` is the GGUF tensor type id (F32 0,
 * Q4_0 2, Q4_1 3, Q8_0 8, Q4_K 12, Q5_K 13, Q6_K 14; :19-25, :56).  ORC_ERR_BITS for another type, ORC_ERR_DIMS
 * when cols is not a whole number of blocks, ORC_ERR_SIZE when data_len is not rows * blocks * block bytes.
 * The layout query fills bits, group size, words per row and groups per row. */
int orc_gguf_affine_layout(int type, int64_t rows, int64_t cols, int *bits, int *group_size, int64_t *packed_cols,
                           int64_t *groups, uint64_t *src_bytes);
int orc_gguf_to_affine(int type, int64_t rows, int64_t cols, const uint8_t *data, uint64_t data_len, uint8_t *weights,
                       uint8_t *scales, uint8_t *biases);
uint16_t orc_gguf_f32_to_bf16(float v);
float orc_gguf_f16_to_f32(uint16_t h);

/* rocm_packed_topk_sample, go/engine/hip/kernels/sampling/topk.hipinc:86-191 (argument rules
 * topk_validate.hipinc:53-77, score decode + softcap kernels/common/numeric.hipinc:95-110): temperature / top-p
 * sampling over a descending list of packed (score, token) values (zeros = no candidate), every sum in double and
 * in list order, `draw` in [0,1) chosen by the caller.  *out = 0 when nothing can be sampled (no candidate, a
 * non-finite weight).  temperature <= 0 and top_p <= 0 together mean greedy (the first candidate); a zero of
 * either alone means 1.  ORC_ERR_DIMS for top_k outside 1..128, ORC_ERR_SIZE for temperature / top_p / softcap /
 * draw outside their ranges. */
int orc_packed_topk_sample(const uint64_t *input, int top_k, float temperature, float top_p, float softcap, double draw,
                           uint64_t *out);

/* The host sampler the reference checks that kernel against (hipGemma4Q4HostSampleResult,
 * go/engine/hip/hip_tiny_model.go:2763-2879, without suppression, repeat penalty and min-p; candidate order
 * hip_transformer_reference.go:502-506: score descending, token ascending) over full logits, which the caller
 * softcaps first as hipGemma4Q4SoftcapLogits does (hip_gemma4_q4_layer.go:3166-3178: orc_softcap_logits).
 * ORC_ERR_DIMS without logits or top_k outside 0..n, ORC_ERR_SIZE for a bad temperature / top-p, ORC_ERR_INDEX
 * when no logit is finite. */
int orc_host_sample(const float *logits, int n, float temperature, int top_k, float top_p, double draw, int *token,
                    float *score);
int orc_softcap_logits(float *logits, int n, float softcap);

/* Number of hardware threads OpenMP would use (for reporting). */
int orc_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
