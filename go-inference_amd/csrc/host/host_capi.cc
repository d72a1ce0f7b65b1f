// extern "C" doors onto the C++ mirror of the Go plug-in surface, so tests (and any
// FFI caller) can drive model.BackendQuant(...).MatVec and attn.ProjQuantMatMulInto
// exactly as Go code would.  Declared in include/aq_mi355_host.h.
#include <cstring>

#include "../../../include/aq_mi355.h"
#include "../../../include/aq_mi355_host.h"
#include "model_quant.h"
#include "rocm_affine.h"

namespace {
thread_local std::string g_err;
int report(const model::Error& e) {
    g_err = e.msg;
    return e.code;
}
}  // namespace

extern "C" {

const char* aqh_last_error(void) { return g_err.c_str(); }

void aqh_register_rocm_backend(void) { rocm::Register(); }

int aqh_backend_quant_registered(const char* backend, const char* kind) {
    return model::BackendQuant(backend ? backend : "", kind ? kind : "") ? 1 : 0;
}

int aqh_backend_quant_bits(const char* backend, const char* kind) {
    auto q = model::BackendQuant(backend ? backend : "", kind ? kind : "");
    return q ? q->Bits() : -1;
}

int aqh_backend_quant_matvec(const char* backend, const char* kind, const uint8_t* x, size_t x_len,
                             const uint8_t* packed, size_t packed_len, const uint8_t* scales, size_t scales_len,
                             const uint8_t* biases, size_t biases_len, int out_dim, int in_dim, int group_size,
                             int bits, uint8_t* out, size_t out_cap, size_t* out_len) {
    auto q = model::BackendQuant(backend ? backend : "", kind ? kind : "");
    if (!q) return report(model::Error::make(AQ_ERR_UNSUPPORTED, "no backend quant registered"));
    model::Bytes res;
    model::Error e = q->MatVec(x, x_len, packed, packed_len, scales, scales_len, biases, biases_len, out_dim, in_dim,
                               group_size, bits, &res);
    if (!e.ok()) return report(e);
    if (out_len) *out_len = res.size();
    if (res.size() > out_cap) return report(model::Error::make(AQ_ERR_SIZE, "output buffer too small"));
    if (!res.empty()) memcpy(out, res.data(), res.size());
    return AQ_OK;
}

int aqh_proj_quant_matmul_into(float* out, size_t out_cap, const float* x, size_t x_len, const uint8_t* packed,
                               size_t packed_len, const uint8_t* scales, size_t scales_len, const uint8_t* biases,
                               size_t biases_len, int M, int K, int N, int group_size, int bits) {
    if (!attn::ProjQuantMatMulInto) return report(model::Error::make(AQ_ERR_UNSUPPORTED, "ProjQuantMatMulInto is nil"));
    std::vector<float> res;
    model::Error e = attn::ProjQuantMatMulInto(&res, x, x_len, packed, packed_len, scales, scales_len, biases,
                                               biases_len, M, K, N, group_size, bits);
    if (!e.ok()) return report(e);
    if (res.size() > out_cap) return report(model::Error::make(AQ_ERR_SIZE, "output buffer too small"));
    if (!res.empty()) memcpy(out, res.data(), res.size() * sizeof(float));
    return AQ_OK;
}

int aqh_concat_quant_rows(const uint8_t* a_packed, size_t a_packed_len, const uint8_t* a_scales, size_t a_sb_len,
                          const uint8_t* a_biases, int a_out_dim, const uint8_t* b_packed, size_t b_packed_len,
                          const uint8_t* b_scales, size_t b_sb_len, const uint8_t* b_biases, int b_out_dim,
                          int a_in_dim, int b_in_dim, int a_bits, int b_bits, int a_group, int b_group,
                          uint8_t* packed_out, uint8_t* scales_out, uint8_t* biases_out, int* out_dim) {
    model::QuantWeight a, b;
    a.Packed.assign(a_packed, a_packed + a_packed_len);
    a.Scales.assign(a_scales, a_scales + a_sb_len);
    a.Biases.assign(a_biases, a_biases + a_sb_len);
    a.Bits = a_bits, a.GroupSize = a_group, a.OutDim = a_out_dim, a.InDim = a_in_dim;
    b.Packed.assign(b_packed, b_packed + b_packed_len);
    b.Scales.assign(b_scales, b_scales + b_sb_len);
    b.Biases.assign(b_biases, b_biases + b_sb_len);
    b.Bits = b_bits, b.GroupSize = b_group, b.OutDim = b_out_dim, b.InDim = b_in_dim;
    auto c = model::ConcatQuantRows(&a, &b);
    if (!c) return report(model::Error::make(AQ_ERR_SHAPE, "ConcatQuantRows: geometry mismatch"));
    memcpy(packed_out, c->Packed.data(), c->Packed.size());
    memcpy(scales_out, c->Scales.data(), c->Scales.size());
    memcpy(biases_out, c->Biases.data(), c->Biases.size());
    if (out_dim) *out_dim = c->OutDim;
    return AQ_OK;
}

void aqh_affine_geometry(int in_dim, int scales_last_dim, int weight_last_dim, int* group_size, int* bits) {
    std::vector<int> s, w;
    if (scales_last_dim >= 0) s = {1, scales_last_dim};
    if (weight_last_dim >= 0) w = {1, weight_last_dim};
    model::affineGeometry(in_dim, s, w, group_size, bits);
}

}  // extern "C"
