/*
 * aq_oracle.c -- CPU restatement of the reference's MLX group-affine path.
 * TEST INFRASTRUCTURE ONLY (see aq_oracle.h).  Plain C, scalar loops, one
 * function per reference function; the file:line each follows is in the header
 * and repeated above each body.
 */
#include "aq_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- bf16 codecs ------------------------------------------------------- */

/* mlxaffine.go:229-237 / quant_reference.go:27-34 */
uint16_t orc_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) { /* NaN stays NaN: force a quiet bit */
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    u += 0x7fffu + ((u >> 16) & 1u); /* ties to even on the kept LSB */
    return (uint16_t)(u >> 16);
}

/* mlxaffine.go:239-241 / quant_reference.go:22-24 */
float orc_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t ld_u16(const uint8_t *p) { return (uint16_t)(p[0] | ((uint16_t)p[1] << 8)); }
static inline uint32_t ld_u32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
static inline void st_u16(uint8_t *p, uint16_t v) {
    p[0] = (uint8_t)v;
    p[1] = (uint8_t)(v >> 8);
}
static inline void st_u32(uint8_t *p, uint32_t v) {
    p[0] = (uint8_t)v;
    p[1] = (uint8_t)(v >> 8);
    p[2] = (uint8_t)(v >> 16);
    p[3] = (uint8_t)(v >> 24);
}

/* ---- code extraction ---------------------------------------------------- */

/* quant_reference.go:36-52: gather `bits` bits starting at bit_off, LSB first,
 * walking bytes. */
uint32_t orc_extract_code(const uint8_t *row, int64_t bit_off, int bits) {
    uint32_t v = 0;
    int got = 0;
    while (got < bits) {
        int64_t pos = bit_off + got;
        int in_byte = (int)(pos & 7);
        int take = 8 - in_byte;
        if (take > bits - got) take = bits - got;
        uint32_t piece = ((uint32_t)row[pos >> 3] >> in_byte) & ((1u << take) - 1u);
        v |= piece << got;
        got += take;
    }
    return v;
}

/* quant_reference.go:54-68 */
void orc_set_code(uint8_t *row, int64_t bit_off, int bits, uint32_t code) {
    int got = 0;
    while (got < bits) {
        int64_t pos = bit_off + got;
        int in_byte = (int)(pos & 7);
        int take = 8 - in_byte;
        if (take > bits - got) take = bits - got;
        uint8_t mask = (uint8_t)(((1u << take) - 1u) << in_byte);
        uint8_t val = (uint8_t)(((code >> got) << in_byte) & mask);
        row[pos >> 3] = (uint8_t)((row[pos >> 3] & (uint8_t)~mask) | val);
        got += take;
    }
}

/* hip_projection_reference.go:200-222: word-granular extraction, a code whose
 * field runs past bit 31 takes its high part from the next word. */
int orc_unpack_word_value(const uint32_t *row_words, int64_t n_words, int col, int bits, uint32_t *code) {
    if (bits == 0) bits = 4;
    if (bits != 4 && bits != 6 && bits != 8) return ORC_ERR_BITS;
    if (col < 0) return ORC_ERR_DIMS;
    uint64_t bit = (uint64_t)col * (uint64_t)bits;
    int64_t wi = (int64_t)(bit / 32);
    unsigned sh = (unsigned)(bit % 32);
    if (wi >= n_words) return ORC_ERR_SIZE;
    uint32_t v = row_words[wi] >> sh;
    if (sh + (unsigned)bits > 32) {
        if (wi + 1 >= n_words) return ORC_ERR_SIZE;
        v |= row_words[wi + 1] << (32 - sh);
    }
    *code = v & ((1u << bits) - 1u);
    return ORC_OK;
}

/* ---- dequantize --------------------------------------------------------- */

static int width_is_word_clean(int bits) { return bits == 1 || bits == 2 || bits == 4 || bits == 8; }

/* mlxaffine.go:178-208.  fp32: out = scale * float(code) + bias, one element
 * at a time.  Built with -ffp-contract=off: mul then add (scale*code is exact
 * in fp32 for bf16 scales and <=8-bit codes, so a fused form agrees anyway). */
int orc_dequantize(const uint8_t *packed, size_t packed_len, const uint8_t *scales, size_t scales_len,
                   const uint8_t *biases, size_t biases_len, int out_dim, int in_dim, int bits, int group_size,
                   float *out) {
    if (!width_is_word_clean(bits)) return ORC_ERR_BITS;
    if (out_dim <= 0 || in_dim <= 0 || group_size <= 0 || in_dim % group_size != 0) return ORC_ERR_DIMS;
    int per_word = 32 / bits;
    size_t words_per_row = (size_t)in_dim * (size_t)bits / 32;
    size_t groups_per_row = (size_t)(in_dim / group_size);
    if (packed_len != (size_t)out_dim * words_per_row * 4) return ORC_ERR_SIZE;
    if (scales_len != (size_t)out_dim * groups_per_row * 2 || biases_len != scales_len) return ORC_ERR_SIZE;
    uint32_t mask = (1u << bits) - 1u;
    for (int r = 0; r < out_dim; r++) {
        for (int j = 0; j < in_dim; j++) {
            size_t wi = (size_t)r * words_per_row + (size_t)(j / per_word);
            unsigned sh = (unsigned)(j % per_word) * (unsigned)bits;
            uint32_t code = (ld_u32(packed + wi * 4) >> sh) & mask;
            size_t gi = ((size_t)r * groups_per_row + (size_t)(j / group_size)) * 2;
            float scale = orc_bf16_to_f32(ld_u16(scales + gi));
            float bias = orc_bf16_to_f32(ld_u16(biases + gi));
            float prod = scale * (float)code;
            out[(size_t)r * (size_t)in_dim + (size_t)j] = prod + bias;
        }
    }
    return ORC_OK;
}

/* ---- quantize (fixture builder) ---------------------------------------- */

static float round_half_away(float v) { return (float)round((double)v); } /* mlxaffine.go:210-213 */

/* mlxaffine.go:131-162 (affineGroup): anchor the larger-magnitude edge to an
 * exact code, sign the scale by which edge dominates, re-derive scale = edge/q0. */
static void affine_group(const float *g, int n, float n_bins, float *scale_out, float *bias_out) {
    float lo = g[0], hi = g[0];
    for (int i = 1; i < n; i++) {
        if (g[i] < lo) lo = g[i];
        if (g[i] > hi) hi = g[i];
    }
    float scale = (hi - lo) / n_bins;
    if (scale < 1e-7f) scale = 1e-7f;
    float edge = hi;
    if (fabsf(lo) > fabsf(hi)) {
        edge = lo;
    } else {
        scale = -scale;
    }
    float q0 = round_half_away(edge / scale);
    if (q0 == 0.0f) {
        *scale_out = scale;
        *bias_out = 0.0f;
        return;
    }
    *scale_out = edge / q0;
    *bias_out = edge;
}

/* mlxaffine.go:80-129 with quantiseCode :164-174.  Codes are derived from the
 * UNROUNDED fp32 scale/bias; the bf16 rounding only affects what is stored. */
int orc_quantize(const float *values, size_t n_values, int out_dim, int in_dim, int bits, int group_size,
                 uint8_t *packed, uint8_t *scales, uint8_t *biases) {
    if (!width_is_word_clean(bits)) return ORC_ERR_BITS;
    if (out_dim <= 0 || in_dim <= 0) return ORC_ERR_DIMS;
    if (group_size <= 0 || in_dim % group_size != 0) return ORC_ERR_DIMS;
    int per_word = 32 / bits;
    if (group_size % per_word != 0) return ORC_ERR_DIMS;
    if (n_values != (size_t)out_dim * (size_t)in_dim) return ORC_ERR_SIZE;
    size_t words_per_row = (size_t)in_dim * (size_t)bits / 32;
    int words_per_group = group_size / per_word;
    int groups_per_row = in_dim / group_size;
    float n_bins = (float)((1 << bits) - 1);
    for (int r = 0; r < out_dim; r++) {
        for (int g = 0; g < groups_per_row; g++) {
            const float *grp = values + (size_t)r * (size_t)in_dim + (size_t)g * (size_t)group_size;
            float scale, bias;
            affine_group(grp, group_size, n_bins, &scale, &bias);
            size_t sbi = ((size_t)r * (size_t)groups_per_row + (size_t)g) * 2;
            st_u16(scales + sbi, orc_f32_to_bf16(scale));
            st_u16(biases + sbi, orc_f32_to_bf16(bias));
            for (int wg = 0; wg < words_per_group; wg++) {
                uint32_t word = 0;
                for (int p = 0; p < per_word; p++) {
                    float q = round_half_away((grp[wg * per_word + p] - bias) / scale);
                    if (q < 0.0f) {
                        q = 0.0f;
                    } else if (q > n_bins) {
                        q = n_bins;
                    }
                    word |= (uint32_t)q << ((unsigned)p * (unsigned)bits);
                }
                size_t wi = (size_t)r * words_per_row + (size_t)g * (size_t)words_per_group + (size_t)wg;
                st_u32(packed + wi * 4, word);
            }
        }
    }
    return ORC_OK;
}

/* repack.go:27-62 (codes only; scales/biases are carried through unchanged by
 * the caller). */
int orc_repack_b1_to_b2(const uint8_t *packed, size_t packed_len, int out_dim, int in_dim, uint8_t *packed2) {
    if (out_dim <= 0 || in_dim <= 0) return ORC_ERR_DIMS;
    if (in_dim % 32 != 0) return ORC_ERR_DIMS;
    size_t w1 = (size_t)in_dim / 32, w2 = (size_t)in_dim / 16;
    if (packed_len != (size_t)out_dim * w1 * 4) return ORC_ERR_SIZE;
    memset(packed2, 0, (size_t)out_dim * w2 * 4);
    for (int r = 0; r < out_dim; r++) {
        for (int j = 0; j < in_dim; j++) {
            uint32_t src = ld_u32(packed + ((size_t)r * w1 + (size_t)(j / 32)) * 4);
            uint32_t code = (src >> (unsigned)(j % 32)) & 1u;
            if (!code) continue;
            uint8_t *dst = packed2 + ((size_t)r * w2 + (size_t)(j / 16)) * 4;
            st_u32(dst, ld_u32(dst) | (code << ((unsigned)(j % 16) * 2)));
        }
    }
    return ORC_OK;
}

/* ---- the reference's CPU qmv / qmm -------------------------------------- */

/* gated_delta.go:63-89.  A row of K fp32 weights is materialised by the
 * dequantizer above, then dotted against each activation row in float64,
 * ascending k; the float64 sum is narrowed to float32 on store. */
int orc_matnt_quant_host(float *out, const float *x, const uint8_t *packed, const uint8_t *scales,
                         const uint8_t *biases, int M, int K, int N, int group_size, int bits, int threads) {
    if (!width_is_word_clean(bits)) return ORC_ERR_BITS;
    if (M <= 0 || K <= 0 || N <= 0 || group_size <= 0 || K % group_size != 0) return ORC_ERR_DIMS;
    size_t row_bytes = (size_t)K * (size_t)bits / 32 * 4;
    size_t sb_bytes = (size_t)(K / group_size) * 2;
    int bad = 0;
#ifdef _OPENMP
    if (threads < 1) threads = 1;
#pragma omp parallel num_threads(threads)
#endif
    {
        float *wrow = (float *)malloc((size_t)K * sizeof(float));
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
        for (int n = 0; n < N; n++) {
            if (!wrow || orc_dequantize(packed + (size_t)n * row_bytes, row_bytes, scales + (size_t)n * sb_bytes,
                                        sb_bytes, biases + (size_t)n * sb_bytes, sb_bytes, 1, K, bits, group_size,
                                        wrow) != ORC_OK) {
#ifdef _OPENMP
#pragma omp atomic write
#endif
                bad = 1;
                continue;
            }
            for (int m = 0; m < M; m++) {
                const float *xr = x + (size_t)m * (size_t)K;
                double acc = 0.0;
                for (int k = 0; k < K; k++) {
                    acc += (double)xr[k] * (double)wrow[k];
                }
                out[(size_t)m * (size_t)N + (size_t)n] = (float)acc;
            }
        }
        free(wrow);
    }
    (void)threads;
    return bad ? ORC_ERR_SIZE : ORC_OK;
}

/* quant_reference.go:78-127 */
int orc_reference_affine_matvec(const uint8_t *x, size_t x_len, const uint8_t *packed, size_t packed_len,
                                const uint8_t *scales, size_t scales_len, const uint8_t *biases, size_t biases_len,
                                int out_dim, int in_dim, int group_size, int bits, uint8_t *out) {
    if (out_dim < 0 || in_dim < 0) return ORC_ERR_DIMS;
    if (out_dim == 0 || in_dim == 0) {
        if (out && out_dim > 0) memset(out, 0, (size_t)out_dim * 2);
        return ORC_OK;
    }
    if (bits <= 0 || bits > 8) return ORC_ERR_BITS;
    if (group_size <= 0 || in_dim % group_size != 0) return ORC_ERR_DIMS;
    if (((int64_t)in_dim * bits) % 8 != 0) return ORC_ERR_DIMS;
    if (x_len != (size_t)in_dim * 2) return ORC_ERR_SIZE;
    size_t row_packed = (size_t)in_dim * (size_t)bits / 8;
    size_t row_sb = (size_t)(in_dim / group_size) * 2;
    if (packed_len != (size_t)out_dim * row_packed || scales_len != (size_t)out_dim * row_sb ||
        biases_len != (size_t)out_dim * row_sb) {
        return ORC_ERR_SIZE;
    }
    double *xf = (double *)malloc((size_t)in_dim * sizeof(double));
    if (!xf) return ORC_ERR_SIZE;
    for (int i = 0; i < in_dim; i++) xf[i] = (double)orc_bf16_to_f32(ld_u16(x + (size_t)i * 2));
    for (int r = 0; r < out_dim; r++) {
        const uint8_t *prow = packed + (size_t)r * row_packed;
        const uint8_t *srow = scales + (size_t)r * row_sb;
        const uint8_t *brow = biases + (size_t)r * row_sb;
        double acc = 0.0;
        for (int c = 0; c < in_dim; c++) {
            int g = c / group_size;
            double scale = (double)orc_bf16_to_f32(ld_u16(srow + (size_t)g * 2));
            double bias = (double)orc_bf16_to_f32(ld_u16(brow + (size_t)g * 2));
            double code = (double)orc_extract_code(prow, (int64_t)c * bits, bits);
            double w = scale * code + bias;
            acc += w * xf[c];
        }
        st_u16(out + (size_t)r * 2, orc_f32_to_bf16((float)acc));
    }
    free(xf);
    return ORC_OK;
}

/* hip_projection_reference.go:122-144 + :161-178 */
static int projection_shape_ok(size_t input_len, size_t weight_len, size_t scale_len, size_t bias_len, int rows,
                               int cols, int group_size, int bits, size_t *words_per_row) {
    if (rows <= 0 || cols <= 0 || group_size <= 0) return ORC_ERR_DIMS;
    if (bits != 4 && bits != 6 && bits != 8) return ORC_ERR_BITS;
    uint64_t total_bits = (uint64_t)cols * (uint64_t)bits;
    if (total_bits % 32 != 0) return ORC_ERR_DIMS;
    *words_per_row = (size_t)(total_bits / 32);
    if (cols % group_size != 0) return ORC_ERR_DIMS;
    if (input_len != (size_t)cols) return ORC_ERR_SIZE;
    if (weight_len != (size_t)rows * *words_per_row) return ORC_ERR_SIZE;
    size_t groups = (size_t)rows * (size_t)(cols / group_size);
    if (scale_len != groups || bias_len != groups) return ORC_ERR_SIZE;
    return ORC_OK;
}

/* hip_projection_reference.go:92-116: everything in float32, weight formed as
 * float(q)*scale + bias, then sum += input*weight in ascending column order. */
int orc_hip_reference_projection(const float *input, size_t input_len, const uint32_t *weights, size_t weight_len,
                                 const uint16_t *scales, size_t scale_len, const uint16_t *biases, size_t bias_len,
                                 int rows, int cols, int group_size, int bits, float *output) {
    if (bits == 0) bits = 4;
    size_t wpr = 0;
    int rc = projection_shape_ok(input_len, weight_len, scale_len, bias_len, rows, cols, group_size, bits, &wpr);
    if (rc != ORC_OK) return rc;
    int groups_per_row = cols / group_size;
    for (int row = 0; row < rows; row++) {
        float sum = 0.0f;
        for (int col = 0; col < cols; col++) {
            uint32_t q = 0;
            rc = orc_unpack_word_value(weights + (size_t)row * wpr, (int64_t)wpr, col, bits, &q);
            if (rc != ORC_OK) return rc;
            size_t g = (size_t)row * (size_t)groups_per_row + (size_t)(col / group_size);
            float qs = (float)q * orc_bf16_to_f32(scales[g]);
            float weight = qs + orc_bf16_to_f32(biases[g]);
            float term = input[col] * weight;
            sum = sum + term;
        }
        output[row] = sum;
    }
    return ORC_OK;
}

int orc_hip_reference_projection_batch(const float *input, int tokens, const uint32_t *weights,
                                       const uint16_t *scales, const uint16_t *biases, int rows, int cols,
                                       int group_size, int bits, float *output) {
    if (tokens <= 0) return ORC_ERR_DIMS;
    if (bits == 0) bits = 4;
    if (rows <= 0 || cols <= 0 || group_size <= 0 || cols % group_size != 0) return ORC_ERR_DIMS;
    if (((uint64_t)cols * (uint64_t)bits) % 32 != 0) return ORC_ERR_DIMS;
    size_t wpr = (size_t)cols * (size_t)bits / 32;
    size_t groups = (size_t)rows * (size_t)(cols / group_size);
    for (int m = 0; m < tokens; m++) {
        int rc = orc_hip_reference_projection(input + (size_t)m * (size_t)cols, (size_t)cols, weights,
                                              (size_t)rows * wpr, scales, groups, biases, groups, rows, cols,
                                              group_size, bits, output + (size_t)m * (size_t)rows);
        if (rc != ORC_OK) return rc;
    }
    return ORC_OK;
}

/* ---- expert-gathered matvec -------------------------------------------- */

/* lthn_gather_qmv.metal:54-66: w += rhs[z]*expert_rows*K*bits/32 words,
 * scales/biases += rhs[z]*expert_rows*(K/group), x += lhs[z]*K (batched x),
 * y += z*N; the row_base byte offsets of qmv_gather.go:295-313 select a
 * sub-slab of rows.  Range check: qmv_gather.go:405-409. */
int orc_gather_qmv(const uint16_t *x, int x_rows, const uint32_t *packed, const uint16_t *scales,
                   const uint16_t *biases, const int32_t *lhs, const int32_t *rhs, int routes, int num_experts,
                   int expert_rows, int row_base, int N, int K, int group_size, int bits, double *out_f64,
                   uint16_t *out_bf16) {
    if (routes < 0 || num_experts <= 0 || expert_rows <= 0 || N < 0 || K < 0 || x_rows <= 0) return ORC_ERR_DIMS;
    if (routes == 0 || N == 0 || K == 0) return ORC_OK;
    if (bits <= 0 || bits > 8) return ORC_ERR_BITS;
    if (group_size <= 0 || K % group_size != 0) return ORC_ERR_DIMS;
    if (((int64_t)K * bits) % 32 != 0) return ORC_ERR_DIMS;
    if (row_base < 0 || row_base + N > expert_rows) return ORC_ERR_DIMS;
    size_t wpr = (size_t)K * (size_t)bits / 32;
    size_t gpr = (size_t)(K / group_size);
    for (int z = 0; z < routes; z++) {
        if (rhs[z] < 0 || rhs[z] >= num_experts) return ORC_ERR_INDEX;
        if (lhs && (lhs[z] < 0 || lhs[z] >= x_rows)) return ORC_ERR_INDEX;
    }
    for (int z = 0; z < routes; z++) {
        size_t e = (size_t)rhs[z];
        const uint16_t *xr = x + (lhs ? (size_t)lhs[z] * (size_t)K : 0);
        for (int n = 0; n < N; n++) {
            size_t row = e * (size_t)expert_rows + (size_t)row_base + (size_t)n;
            const uint8_t *prow = (const uint8_t *)(packed + row * wpr);
            const uint16_t *srow = scales + row * gpr;
            const uint16_t *brow = biases + row * gpr;
            double acc = 0.0;
            for (int c = 0; c < K; c++) {
                int g = c / group_size;
                double w = (double)orc_bf16_to_f32(srow[g]) * (double)orc_extract_code(prow, (int64_t)c * bits, bits) +
                           (double)orc_bf16_to_f32(brow[g]);
                acc += w * (double)orc_bf16_to_f32(xr[c]);
            }
            size_t o = (size_t)z * (size_t)N + (size_t)n;
            if (out_f64) out_f64[o] = acc;
            if (out_bf16) out_bf16[o] = orc_f32_to_bf16((float)acc);
        }
    }
    return ORC_OK;
}

/* hip_kernels_test.go:8127-8137 (expectedGELUTanhMultiply); SiLU per gated_delta.go:228. */
int orc_act_multiply(int act, const float *gate, const float *up, int64_t n, float *out) {
    if (act != ORC_ACT_GELU_TANH && act != ORC_ACT_SILU) return ORC_ERR_BITS;
    if (n < 0) return ORC_ERR_DIMS;
    const double sqrt2_over_pi = 0.7978845608028654;
    const double coeff = 0.044715;
    for (int64_t i = 0; i < n; i++) {
        const double value = (double)gate[i];
        double a;
        if (act == ORC_ACT_GELU_TANH) {
            a = 0.5 * value * (1 + tanh(sqrt2_over_pi * (value + coeff * value * value * value)));
        } else {
            a = value / (1 + exp(-value));
        }
        out[i] = (float)a * up[i];
    }
    return ORC_OK;
}

/* ffn_megakernel_test.go:17-31 (hostGeluMul). */
int orc_act_gate_mul_bf16(int act, const uint16_t *gate, const uint16_t *up, int64_t n, uint16_t *out) {
    if (act != ORC_ACT_GELU_TANH && act != ORC_ACT_SILU) return ORC_ERR_BITS;
    if (n < 0) return ORC_ERR_DIMS;
    for (int64_t i = 0; i < n; i++) {
        const float g = orc_bf16_to_f32(gate[i]);
        const float u = orc_bf16_to_f32(up[i]);
        float a;
        if (act == ORC_ACT_GELU_TANH) {
            const float inner = g + 0.044715f * (g * g * g);
            const float t = (float)tanh((double)(0.7978845608028654f * inner));
            a = 0.5f * g * (1.0f + t);
        } else {
            const float e = (float)exp((double)(-g));
            a = g / (1.0f + e);
        }
        out[i] = orc_f32_to_bf16(a * u);
    }
    return ORC_OK;
}

/* moe_quant_reference.go:27-55,268-286; hip_gemma4_moe.go:318-360; hip_qwen3_moe_router.go:33-45,78-85. */
int orc_moe_route(const float *logits, int rows, int num_experts, int top_k, const float *expert_scales, int normalise,
                  int32_t *ids, float *weights) {
    if (rows < 0 || num_experts <= 0 || top_k <= 0 || top_k > num_experts) return ORC_ERR_DIMS;
    int *sel = (int *)malloc((size_t)top_k * sizeof(int));
    if (!sel) return ORC_ERR_SIZE;
    for (int row = 0; row < rows; row++) {
        const float *sc = logits + (size_t)row * num_experts;
        for (int e = 0; e < num_experts; e++)
            if (isnan(sc[e]) || isinf(sc[e])) {
                free(sel);
                return ORC_ERR_INDEX;
            }
        /* insertion into a list kept in (score desc, id asc) order */
        int count = 0;
        for (int e = 0; e < num_experts; e++) {
            int insert = top_k;
            for (int r = 0; r < top_k; r++) {
                if (r >= count || sc[e] > sc[sel[r]] || (sc[e] == sc[sel[r]] && e < sel[r])) {
                    insert = r;
                    break;
                }
            }
            if (insert == top_k) continue;
            for (int r = top_k - 1; r > insert; r--) sel[r] = sel[r - 1];
            sel[insert] = e;
            if (count < top_k) count++;
        }
        if (normalise) {
            float max_value = sc[sel[0]];
            for (int r = 1; r < top_k; r++)
                if (sc[sel[r]] > max_value) max_value = sc[sel[r]];
            double sum = 0;
            for (int r = 0; r < top_k; r++) {
                const double ex = exp((double)(sc[sel[r]] - max_value));
                weights[(size_t)row * top_k + r] = (float)ex;
                sum += ex;
            }
            for (int r = 0; r < top_k; r++)
                weights[(size_t)row * top_k + r] = (float)((double)weights[(size_t)row * top_k + r] / sum);
        } else {
            float max_logit = -INFINITY;
            for (int e = 0; e < num_experts; e++)
                if (sc[e] > max_logit) max_logit = sc[e];
            double total = 0;
            for (int e = 0; e < num_experts; e++) total += exp((double)(sc[e] - max_logit));
            if (total == 0) total = 1;
            for (int r = 0; r < top_k; r++)
                weights[(size_t)row * top_k + r] = (float)(exp((double)(sc[sel[r]] - max_logit)) / total);
        }
        for (int r = 0; r < top_k; r++) {
            ids[(size_t)row * top_k + r] = sel[r];
            if (expert_scales) weights[(size_t)row * top_k + r] *= expert_scales[sel[r]];
        }
    }
    free(sel);
    return ORC_OK;
}

/* routing.hipinc:100-158; lthn_moe_weighted_sum.metal:17-38. */
int orc_moe_combine(const float *route_rows, const float *weights, int rows, int top_k, int n, int bf16_steps,
                    float *out) {
    if (rows < 0 || top_k <= 0 || n < 0) return ORC_ERR_DIMS;
    for (int row = 0; row < rows; row++) {
        for (int c = 0; c < n; c++) {
            float acc = 0.0f;
            for (int r = 0; r < top_k; r++) {
                const size_t pair = (size_t)row * top_k + r;
                const float y = route_rows[pair * n + c];
                if (bf16_steps) {
                    const float w = orc_bf16_to_f32(orc_f32_to_bf16(weights[pair]));
                    const float scaled = orc_bf16_to_f32(orc_f32_to_bf16(y * w));
                    acc = r == 0 ? scaled : orc_bf16_to_f32(orc_f32_to_bf16(acc + scaled));
                } else {
                    const float scaled = y * weights[pair];
                    acc = acc + scaled;
                }
            }
            out[(size_t)row * n + c] = acc;
        }
    }
    return ORC_OK;
}

/* hip_projection_launch.go:2375-2395 */
static uint32_t ordered_float32_key(float value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    if (bits & 0x80000000u) return ~bits;
    return bits ^ 0x80000000u;
}

uint64_t orc_pack_greedy_best(float score, int token) {
    return ((uint64_t)ordered_float32_key(score) << 32) | (uint64_t)(~(uint32_t)token);
}

/* hip_projection_launch.go:2386-2416 */
int orc_unpack_greedy_best(uint64_t packed, float softcap, int vocab_size, int *token, float *score) {
    if (vocab_size <= 0) return ORC_ERR_DIMS;
    if (packed == 0) return ORC_ERR_INDEX;
    if (softcap < 0 || isnan(softcap) || isinf(softcap)) return ORC_ERR_SIZE;
    const int64_t id = (int64_t)(int32_t)(~(uint32_t)packed);
    if (id < 0 || id >= vocab_size) return ORC_ERR_INDEX;
    const uint32_t key = (uint32_t)(packed >> 32);
    const uint32_t bits = (key & 0x80000000u) ? (key ^ 0x80000000u) : ~key;
    float s;
    memcpy(&s, &bits, 4);
    if (softcap > 0) s = (float)tanh((double)(s / softcap)) * softcap;
    *token = (int)id;
    *score = s;
    return ORC_OK;
}

/* hip_transformer_reference.go:401-437 */
int orc_greedy_sample_suppress(const float *logits, int n, const int32_t *suppress, int suppress_count, int *index,
                               float *value) {
    if (n <= 0) return ORC_ERR_DIMS;
    int best = -1;
    float best_value = 0;
    for (int i = 0; i < n; i++) {
        int skip = 0;
        for (int s = 0; s < suppress_count; s++)
            if (suppress[s] == i) skip = 1;
        if (skip) continue;
        if (best < 0 || logits[i] > best_value) {
            best = i;
            best_value = logits[i];
        }
    }
    if (best < 0) return ORC_ERR_INDEX;
    *index = best;
    *value = best_value;
    return ORC_OK;
}

/* ---- GGUF blocks -> affine layout (go/engine/hip/hip_gguf_affine_adapter.go) ---- */

/* hip_projection_reference.go:240-261 */
float orc_gguf_f16_to_f32(uint16_t value) {
    uint32_t sign = (uint32_t)(value & 0x8000) << 16;
    int exponent = (value >> 10) & 0x1f;
    uint32_t fraction = value & 0x03ff;
    uint32_t bits;
    if (exponent == 0) {
        if (fraction == 0) {
            bits = sign;
        } else {
            exponent = -14;
            while ((fraction & 0x0400) == 0) {
                fraction <<= 1;
                exponent--;
            }
            fraction &= 0x03ff;
            bits = sign | (uint32_t)(exponent + 127) << 23 | fraction << 13;
        }
    } else if (exponent == 0x1f) {
        bits = sign | 0x7f800000u | fraction << 13;
    } else {
        bits = sign | (uint32_t)(exponent - 15 + 127) << 23 | fraction << 13;
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* hip_bf16_portable.go:19-23: round to nearest even on the bit pattern, NaN payloads included */
uint16_t orc_gguf_f32_to_bf16(float v) {
    uint32_t bits;
    memcpy(&bits, &v, 4);
    bits += 0x7fff + ((bits >> 16) & 1);
    return (uint16_t)(bits >> 16);
}

static uint16_t gguf_le16(const uint8_t *p) { return (uint16_t)(p[0] | p[1] << 8); }
static void gguf_put16(uint8_t *p, uint16_t v) {
    p[0] = (uint8_t)v;
    p[1] = (uint8_t)(v >> 8);
}

/* hip_gguf_affine_adapter.go:843-857 (weights start zeroed; a code may straddle two words) */
static void gguf_put_code(uint8_t *weights, int64_t row_word_base, int64_t col, int bits, uint32_t value) {
    int64_t bit_off = col * bits;
    int64_t word = row_word_base + bit_off / 32;
    unsigned shift = (unsigned)(bit_off % 32);
    uint32_t mask = (1u << bits) - 1;
    uint32_t w;
    memcpy(&w, weights + word * 4, 4);
    w |= (value & mask) << shift;
    memcpy(weights + word * 4, &w, 4);
    if (shift + (unsigned)bits > 32) {
        memcpy(&w, weights + word * 4 + 4, 4);
        w |= (value & mask) >> (32 - shift);
        memcpy(weights + word * 4 + 4, &w, 4);
    }
}

/* :793-799 */
static void gguf_k_scale_min(const uint8_t *s, int group, uint8_t *scale, uint8_t *min) {
    if (group < 4) {
        *scale = s[group] & 63;
        *min = s[group + 4] & 63;
    } else {
        *scale = (uint8_t)((s[group + 4] & 0x0f) | ((s[group - 4] >> 6) << 4));
        *min = (uint8_t)((s[group + 4] >> 4) | ((s[group] >> 6) << 4));
    }
}

/* :801-820 */
static uint8_t gguf_q5k_code(const uint8_t *block, int group, int lane) {
    int il = group / 2, high = group % 2 == 1, ir = lane / 2, sub = lane % 2;
    uint8_t value = block[48 + 32 * il + 2 * ir + sub];
    if (high) value >>= 4;
    value &= 0x0f;
    uint8_t mask = (uint8_t)(1u << (2 * il));
    if (high) mask <<= 1;
    if (block[16 + 2 * ir + sub] & mask) value += 16;
    return value & 0x1f;
}

/* :822-841 */
static uint8_t gguf_q6k_code(const uint8_t *block, int group, int lane) {
    int ip = group / 8, local = group % 8;
    int lane_off = local % 2 == 1 ? 16 : 0;
    int quartile = local / 2;
    int ql_index = ip * 64 + lane_off + lane;
    if (quartile == 1 || quartile == 3) ql_index += 32;
    uint8_t ql = block[ql_index];
    if (quartile >= 2) ql >>= 4;
    int qh_index = 128 + ip * 32 + lane_off + lane;
    return (uint8_t)((ql & 0x0f) | (((block[qh_index] >> (quartile * 2)) & 0x03) << 4));
}

static int gguf_format(int type, int *block_cols, int *block_bytes, int *bits, int *group) {
    switch (type) {
        case 0: *block_cols = 32, *block_bytes = 128, *bits = 8, *group = 32; return 1;  /* F32, :650-720 */
        case 2: *block_cols = 32, *block_bytes = 18, *bits = 4, *group = 32; return 1;   /* Q4_0, :27-30 */
        case 3: *block_cols = 32, *block_bytes = 20, *bits = 4, *group = 32; return 1;   /* Q4_1, :31-34 */
        case 8: *block_cols = 32, *block_bytes = 34, *bits = 8, *group = 32; return 1;   /* Q8_0, :52-54 */
        case 12: *block_cols = 256, *block_bytes = 144, *bits = 4, *group = 32; return 1; /* Q4_K, :37-41 */
        case 13: *block_cols = 256, *block_bytes = 176, *bits = 6, *group = 32; return 1; /* Q5_K, :42-46 */
        case 14: *block_cols = 256, *block_bytes = 210, *bits = 6, *group = 16; return 1; /* Q6_K, :47-51 */
        default: return 0;
    }
}

int orc_gguf_affine_layout(int type, int64_t rows, int64_t cols, int *bits, int *group_size, int64_t *packed_cols,
                           int64_t *groups, uint64_t *src_bytes) {
    int bc, bb, b, g;
    if (!gguf_format(type, &bc, &bb, &b, &g)) return ORC_ERR_BITS;
    if (rows <= 0 || cols <= 0 || cols % bc != 0) return ORC_ERR_DIMS;
    *bits = b;
    *group_size = g;
    *packed_cols = cols * b / 32;
    *groups = cols / g;
    *src_bytes = (uint64_t)rows * (uint64_t)(cols / bc) * (uint64_t)bb;
    return ORC_OK;
}

int orc_gguf_to_affine(int type, int64_t rows, int64_t cols, const uint8_t *data, uint64_t data_len, uint8_t *weights,
                       uint8_t *scales, uint8_t *biases) {
    int bits, gs;
    int64_t packed_cols, groups;
    uint64_t want;
    int rc = orc_gguf_affine_layout(type, rows, cols, &bits, &gs, &packed_cols, &groups, &want);
    if (rc != ORC_OK) return rc;
    if (data_len != want) return ORC_ERR_SIZE;
    memset(weights, 0, (size_t)(rows * packed_cols * 4));
    for (int64_t row = 0; row < rows; row++) {
        if (type == 0) { /* :677-718 */
            for (int64_t group = 0; group < groups; group++) {
                float values[32], lo = 0, hi = 0;
                for (int lane = 0; lane < 32; lane++) {
                    float v;
                    memcpy(&v, data + ((size_t)row * cols + group * 32 + lane) * 4, 4);
                    if (isnan(v) || isinf(v)) v = 0;
                    values[lane] = v;
                    if (lane == 0 || v < lo) lo = v;
                    if (lane == 0 || v > hi) hi = v;
                }
                float scale = (hi - lo) / 255;
                if (scale == 0) scale = 1;
                gguf_put16(scales + (row * groups + group) * 2, orc_gguf_f32_to_bf16(scale));
                gguf_put16(biases + (row * groups + group) * 2, orc_gguf_f32_to_bf16(lo));
                for (int lane = 0; lane < 32; lane++) {
                    uint32_t q = 0;
                    if (hi != lo) {
                        float quotient = (values[lane] - lo) / scale;
                        q = (uint32_t)round((double)quotient);
                        if (q > 255) q = 255;
                    }
                    gguf_put_code(weights, row * packed_cols, group * 32 + lane, 8, q);
                }
            }
            continue;
        }
        if (type == 2 || type == 3 || type == 8) {
            int bb = type == 2 ? 18 : type == 3 ? 20 : 34;
            int64_t blocks = cols / 32;
            for (int64_t bi = 0; bi < blocks; bi++) {
                const uint8_t *block = data + (size_t)(row * blocks + bi) * bb;
                float scale = orc_gguf_f16_to_f32(gguf_le16(block));
                float bias = type == 2 ? -8 * scale : type == 3 ? orc_gguf_f16_to_f32(gguf_le16(block + 2)) : -128 * scale;
                gguf_put16(scales + (row * groups + bi) * 2, orc_gguf_f32_to_bf16(scale));
                gguf_put16(biases + (row * groups + bi) * 2, orc_gguf_f32_to_bf16(bias));
                for (int lane = 0; lane < 32; lane++) {
                    uint32_t value;
                    if (type == 8) {
                        value = (uint32_t)((int)(int8_t)block[2 + lane] + 128); /* :631 */
                    } else {
                        uint8_t packed = block[(type == 2 ? 2 : 4) + lane % 16]; /* :374-378, :432-436 */
                        value = lane >= 16 ? packed >> 4 : packed & 0x0f;
                    }
                    gguf_put_code(weights, row * packed_cols, bi * 32 + lane, bits, value);
                }
            }
            continue;
        }
        int bb = type == 12 ? 144 : type == 13 ? 176 : 210;
        int64_t blocks = cols / 256;
        for (int64_t bi = 0; bi < blocks; bi++) {
            const uint8_t *block = data + (size_t)(row * blocks + bi) * bb;
            if (type == 14) { /* :774-791 */
                float d = orc_gguf_f16_to_f32(gguf_le16(block + 208));
                for (int group = 0; group < 16; group++) {
                    float scale = d * (float)(int8_t)block[192 + group];
                    int64_t gi = row * groups + bi * 16 + group;
                    gguf_put16(scales + gi * 2, orc_gguf_f32_to_bf16(scale));
                    gguf_put16(biases + gi * 2, orc_gguf_f32_to_bf16(-32 * scale));
                    for (int lane = 0; lane < 16; lane++)
                        gguf_put_code(weights, row * packed_cols, bi * 256 + group * 16 + lane, 6,
                                      gguf_q6k_code(block, group, lane));
                }
                continue;
            }
            float d = orc_gguf_f16_to_f32(gguf_le16(block));
            float dmin = orc_gguf_f16_to_f32(gguf_le16(block + 2));
            for (int group = 0; group < 8; group++) { /* :722-751, :753-772 */
                uint8_t sc, mn;
                gguf_k_scale_min(block + 4, group, &sc, &mn);
                int64_t gi = row * groups + bi * 8 + group;
                gguf_put16(scales + gi * 2, orc_gguf_f32_to_bf16(d * (float)sc));
                gguf_put16(biases + gi * 2, orc_gguf_f32_to_bf16(-dmin * (float)mn));
                for (int lane = 0; lane < 32; lane++) {
                    uint32_t value;
                    if (type == 12) {
                        uint8_t q = block[16 + (group / 2) * 32 + lane]; /* word w, lane l: qs[pair*32 + w*8 + l] */
                        value = group % 2 == 1 ? q >> 4 : q & 0x0f;
                    } else {
                        value = gguf_q5k_code(block, group, lane);
                    }
                    gguf_put_code(weights, row * packed_cols, bi * 256 + group * 32 + lane, bits, value);
                }
            }
        }
    }
    return ORC_OK;
}

/* ---- temperature / top-p sampling over the packed top-k ---- */

/* kernels/common/numeric.hipinc:95-110 */
static double sample_score(uint64_t packed, double softcap) {
    uint32_t key = (uint32_t)(packed >> 32);
    uint32_t bits = (key & 0x80000000u) ? key ^ 0x80000000u : ~key;
    float f;
    memcpy(&f, &bits, 4);
    double score = (double)f;
    return softcap > 0.0 ? tanh(score / softcap) * softcap : score;
}

/* kernels/sampling/topk.hipinc:86-191 */
int orc_packed_topk_sample(const uint64_t *input, int top_k, float raw_temperature, float raw_top_p, float softcap_f,
                           double draw, uint64_t *out) {
    if (top_k <= 0 || top_k > 128) return ORC_ERR_DIMS;
    if (!(raw_temperature >= 0.0f) || !isfinite(raw_temperature) || !(raw_top_p >= 0.0f) || !(raw_top_p <= 1.0f) ||
        !(softcap_f >= 0.0f) || !isfinite(softcap_f) || !isfinite(draw))
        return ORC_ERR_SIZE;
    *out = 0;
    int first_valid = top_k;
    for (int i = 0; i < top_k; i++)
        if (input[i] != 0) {
            first_valid = i;
            break;
        }
    if (first_valid >= top_k) return ORC_OK;
    if (raw_temperature <= 0.0f && raw_top_p <= 0.0f) {
        *out = input[first_valid];
        return ORC_OK;
    }
    const double temperature = raw_temperature == 0.0f ? 1.0 : (double)raw_temperature;
    const double top_p = raw_top_p == 0.0f ? 1.0 : (double)raw_top_p;
    if (!(temperature > 0.0) || !(top_p > 0.0 && top_p <= 1.0)) return ORC_OK;
    const double softcap = (double)softcap_f;
    const double max_value = sample_score(input[first_valid], softcap) / temperature;
    double total = 0.0;
    for (int i = first_valid; i < top_k; i++) {
        if (input[i] == 0) continue;
        double weight = exp(sample_score(input[i], softcap) / temperature - max_value);
        if (!isfinite(weight)) return ORC_OK;
        total += weight;
    }
    if (!(total > 0.0) || !isfinite(total)) return ORC_OK;
    int limit = top_k;
    if (top_p < 1.0) {
        double cumulative = 0.0;
        for (int i = first_valid; i < top_k; i++) {
            if (input[i] == 0) continue;
            cumulative += exp(sample_score(input[i], softcap) / temperature - max_value);
            if (cumulative / total >= top_p) {
                limit = i + 1;
                break;
            }
        }
    }
    double selected_total = 0.0;
    uint64_t fallback = input[first_valid];
    for (int i = first_valid; i < limit; i++) {
        if (input[i] == 0) continue;
        fallback = input[i];
        selected_total += exp(sample_score(input[i], softcap) / temperature - max_value);
    }
    if (!(selected_total > 0.0) || !isfinite(selected_total)) return ORC_OK;
    if (draw < 0.0) draw = 0.0;
    if (draw >= 1.0) draw = nextafter(1.0, 0.0);
    const double target = draw * selected_total;
    double cumulative = 0.0;
    for (int i = first_valid; i < limit; i++) {
        if (input[i] == 0) continue;
        cumulative += exp(sample_score(input[i], softcap) / temperature - max_value);
        if (target <= cumulative) {
            *out = input[i];
            return ORC_OK;
        }
    }
    *out = fallback;
    return ORC_OK;
}

/* hip_gemma4_q4_layer.go:3166-3178 */
int orc_softcap_logits(float *logits, int n, float softcap) {
    if (softcap < 0 || isnan(softcap) || isinf(softcap)) return ORC_ERR_SIZE;
    if (softcap == 0) return ORC_OK;
    for (int i = 0; i < n; i++) logits[i] = (float)tanh((double)(logits[i] / softcap)) * softcap;
    return ORC_OK;
}

typedef struct {
    int index;
    float value;
} host_candidate;

/* hip_transformer_reference.go:502-506: score descending, token id ascending */
static int host_candidate_cmp(const void *a, const void *b) {
    const host_candidate *x = a, *y = b;
    if (x->value > y->value) return -1;
    if (x->value < y->value) return 1;
    return x->index < y->index ? -1 : x->index > y->index;
}

/* hip_tiny_model.go:2763-2879 (no suppression list, history or min-p) */
int orc_host_sample(const float *logits, int n, float temperature, int top_k, float top_p, double draw, int *token,
                    float *score) {
    if (n <= 0) return ORC_ERR_DIMS;
    if (temperature <= 0 && top_k <= 0 && top_p <= 0) return orc_greedy_sample_suppress(logits, n, NULL, 0, token, score);
    if (temperature == 0) temperature = 1;
    if (temperature <= 0 || isnan(temperature) || isinf(temperature)) return ORC_ERR_SIZE;
    if (top_p == 0) top_p = 1;
    if (top_p <= 0 || top_p > 1 || isnan(top_p)) return ORC_ERR_SIZE;
    host_candidate *cand = malloc((size_t)n * sizeof *cand);
    int count = 0;
    for (int i = 0; i < n; i++)
        if (!isnan(logits[i]) && !isinf(logits[i])) cand[count++] = (host_candidate){i, logits[i]};
    if (count == 0) {
        free(cand);
        return ORC_ERR_INDEX;
    }
    qsort(cand, (size_t)count, sizeof *cand, host_candidate_cmp);
    if (top_k < 0 || top_k > n) {
        free(cand);
        return ORC_ERR_DIMS;
    }
    if (top_k == 0 || top_k > count) top_k = count;
    double *weights = malloc((size_t)top_k * sizeof *weights);
    double max_value = (double)cand[0].value / (double)temperature, total = 0.0;
    for (int i = 0; i < top_k; i++) {
        weights[i] = exp((double)cand[i].value / (double)temperature - max_value);
        total += weights[i];
    }
    int rc = ORC_OK;
    if (total <= 0 || isnan(total) || isinf(total)) {
        rc = ORC_ERR_SIZE;
    } else {
        int limit = top_k;
        if (top_p < 1) {
            double cumulative = 0.0;
            for (int i = 0; i < top_k; i++) {
                cumulative += weights[i];
                if (cumulative / total >= (double)top_p) {
                    limit = i + 1;
                    break;
                }
            }
        }
        double selected_total = 0.0;
        for (int i = 0; i < limit; i++) selected_total += weights[i];
        if (draw < 0) draw = 0;
        if (draw >= 1) draw = nextafter(1.0, 0.0);
        double target = draw * selected_total, cumulative = 0.0;
        int pick = limit - 1;
        for (int i = 0; i < limit; i++) {
            cumulative += weights[i];
            if (target <= cumulative) {
                pick = i;
                break;
            }
        }
        *token = cand[pick].index;
        *score = cand[pick].value;
    }
    free(weights);
    free(cand);
    return rc;
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
