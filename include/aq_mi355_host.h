/*
 * aq_mi355_host.h -- C doors onto the host-side mirror of go-inference's quant plug-in
 * surface (built into libaq_mi355.so).  The mirror exists because the Go toolchain is
 * not part of this build: it reproduces, in C++, the interfaces a Go backend registers
 * against, with the same names, argument meaning and error behaviour, and these doors
 * let an FFI caller drive them.
 *
 *   model.RegisterBackendQuant / BackendQuant / QuantMatVec.MatVec   go/model/quant.go:35-63
 *   attn.ProjQuantMatMulInto                                          go/model/attn/gated_delta.go:46-58
 *   model.ConcatQuantRows                                             go/model/quant_weight.go:45-63
 *   model affineGeometry                                              go/model/linear.go:91-102
 *   safetensors.ReadSafetensors / tensor views                        go/model/safetensors/safetensors.go:53-95
 *   model.LoadLinear                                                  go/model/linear.go:42-84
 *   mlxaffine.RepackB1ToB2                                            go/model/quant/mlxaffine/repack.go:27-62
 *
 * Return value: 0 ok, otherwise the AQ_ERR_* / hipError_t code; aqh_last_error() gives
 * the message (the Go `error` string).
 */
#ifndef AQ_MI355_HOST_H
#define AQ_MI355_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *aqh_last_error(void);

/* The backend package's init(): model.RegisterBackendQuant("rocm", affine) and
 * attn.ProjQuantMatMulInto = MatMulQuantF32NTInto (go/engine/metal/model_quant.go:25,
 * go/engine/metal/quant_seam_backend.go:27-29 are the Metal twins). */
void aqh_register_rocm_backend(void);

/* model.BackendQuant(backend, kind): 1 if registered (go/model/quant.go:58-63). */
int aqh_backend_quant_registered(const char *backend, const char *kind);
/* QuantScheme.Bits() of the registered impl, -1 if none (go/engine/metal/model_quant.go:19). */
int aqh_backend_quant_bits(const char *backend, const char *kind);

/* model.BackendQuant(backend, kind).MatVec(x, packed, scales, biases, outDim, inDim, groupSize, bits)
 * (go/model/quant.go:35-38).  *out_len receives len(result). */
int aqh_backend_quant_matvec(const char *backend, const char *kind, const uint8_t *x, size_t x_len,
                             const uint8_t *packed, size_t packed_len, const uint8_t *scales, size_t scales_len,
                             const uint8_t *biases, size_t biases_len, int out_dim, int in_dim, int group_size,
                             int bits, uint8_t *out, size_t out_cap, size_t *out_len);

/* attn.ProjQuantMatMulInto(out, x, packed, scales, biases, M, K, N, groupSize, bits)
 * (go/model/attn/gated_delta.go:46-51); fails with AQ_ERR_UNSUPPORTED while the hook is nil. */
int aqh_proj_quant_matmul_into(float *out, size_t out_cap, const float *x, size_t x_len, const uint8_t *packed,
                               size_t packed_len, const uint8_t *scales, size_t scales_len, const uint8_t *biases,
                               size_t biases_len, int M, int K, int N, int group_size, int bits);

/* model.ConcatQuantRows(a, b) (go/model/quant_weight.go:45-63); AQ_ERR_SHAPE where Go returns nil. */
int aqh_concat_quant_rows(const uint8_t *a_packed, size_t a_packed_len, const uint8_t *a_scales, size_t a_sb_len,
                          const uint8_t *a_biases, int a_out_dim, const uint8_t *b_packed, size_t b_packed_len,
                          const uint8_t *b_scales, size_t b_sb_len, const uint8_t *b_biases, int b_out_dim,
                          int a_in_dim, int b_in_dim, int a_bits, int b_bits, int a_group, int b_group,
                          uint8_t *packed_out, uint8_t *scales_out, uint8_t *biases_out, int *out_dim);

/* affineGeometry(inDim, scalesShape, weightShape) with the shapes' last dims (negative = empty shape)
 * (go/model/linear.go:91-110). */
void aqh_affine_geometry(int in_dim, int scales_last_dim, int weight_last_dim, int *group_size, int *bits);

/* A safetensors file, memory-mapped; tensors are views into the mapping and stay valid until
 * aqh_safetensors_close (go/model/safetensors/safetensors.go:53-95; entry rules
 * go/model/safetensors/header_parse.go:343-437: dtype, shape and data_offsets are required, unknown keys are
 * skipped, offsets must be ordered and inside the file). */
typedef struct aqh_safetensors aqh_safetensors;
int aqh_safetensors_open(const char *path, aqh_safetensors **out);
void aqh_safetensors_close(aqh_safetensors *f);
int aqh_safetensors_count(const aqh_safetensors *f);
/* Name of tensor `index` in sorted order; AQ_ERR_INDEX past the end, AQ_ERR_SIZE if buf is too short. */
int aqh_safetensors_name(const aqh_safetensors *f, int index, char *buf, size_t buf_len);
/* dtype (at most 15 characters), shape (at most 8 dims), bytes.  AQ_ERR_INDEX when the tensor is absent. */
int aqh_safetensors_tensor(const aqh_safetensors *f, const char *name, char dtype[16], int64_t shape[8], int *rank,
                           const uint8_t **data, size_t *len);

/* model.Linear (go/model/linear.go:21-33) as plain data: views into the file (or, after the 1-bit -> 2-bit
 * widening, into a buffer the file object owns).  scales == NULL means dense bf16.  experts / expert_rows
 * describe a rank-3 [experts, expert_rows, words] weight (an MoE expert stack); experts == 0 for rank 2. */
typedef struct aqh_linear {
    const uint8_t *weight, *scales, *biases, *bias;
    size_t weight_len, scales_len, biases_len, bias_len;
    int out_dim, in_dim, group_size, bits;
    int quantised;
    int experts, expert_rows;
} aqh_linear;

/* model.LoadLinear(tensors, prefix, inDim, "affine") (go/model/linear.go:42-84): ".scales" present means
 * quantised, geometry from the shapes, a 1-bit pack is widened to 2 bits and written back into the file
 * object's tensor map.  AQ_ERR_INDEX when prefix + ".weight" is absent (Go returns nil). */
int aqh_load_linear(aqh_safetensors *f, const char *prefix, int in_dim, aqh_linear *out);

/* mlxaffine.RepackB1ToB2 on caller buffers: packed2 holds out_dim * in_dim / 4 bytes. */
int aqh_repack_b1_to_b2(const uint8_t *packed, size_t packed_len, size_t scales_len, size_t biases_len, int out_dim,
                        int in_dim, int group_size, uint8_t *packed2, size_t packed2_len);

#ifdef __cplusplus
}
#endif
#endif
