// extern "C" doors onto the C++ mirror of the Go plug-in surface, so tests (and any
// FFI caller) can drive model.BackendQuant(...).MatVec and attn.ProjQuantMatMulInto
// exactly as Go code would.  Declared in include/aq_mi355_host.h.
#include <cstring>
#include <iterator>

#include "../../../include/aq_mi355.h"
#include "../../../include/aq_mi355_host.h"
#include "model_quant.h"
#include "rocm_affine.h"
#include "safetensors.h"

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

int aqh_safetensors_open(const char* path, aqh_safetensors** out) {
    if (!path || !out) return report(model::Error::make(AQ_ERR_ARG, "aqh_safetensors_open: bad argument"));
    *out = nullptr;
    std::unique_ptr<safetensors::File> f;
    model::Error e = safetensors::File::Open(path, &f);
    if (!e.ok()) return report(e);
    *out = reinterpret_cast<aqh_safetensors*>(f.release());
    return AQ_OK;
}

void aqh_safetensors_close(aqh_safetensors* f) { delete reinterpret_cast<safetensors::File*>(f); }

int aqh_safetensors_count(const aqh_safetensors* f) {
    return f ? (int)reinterpret_cast<const safetensors::File*>(f)->Tensors.size() : 0;
}

int aqh_safetensors_name(const aqh_safetensors* f, int index, char* buf, size_t buf_len) {
    if (!f || !buf) return report(model::Error::make(AQ_ERR_ARG, "aqh_safetensors_name: bad argument"));
    const auto& m = reinterpret_cast<const safetensors::File*>(f)->Tensors;
    if (index < 0 || (size_t)index >= m.size()) return report(model::Error::make(AQ_ERR_INDEX, "tensor index out of range"));
    auto it = m.begin();
    std::advance(it, index);
    if (it->first.size() + 1 > buf_len) return report(model::Error::make(AQ_ERR_SIZE, "name buffer too small"));
    memcpy(buf, it->first.c_str(), it->first.size() + 1);
    return AQ_OK;
}

int aqh_safetensors_tensor(const aqh_safetensors* f, const char* name, char dtype[16], int64_t shape[8], int* rank,
                           const uint8_t** data, size_t* len) {
    if (!f || !name) return report(model::Error::make(AQ_ERR_ARG, "aqh_safetensors_tensor: bad argument"));
    const auto& m = reinterpret_cast<const safetensors::File*>(f)->Tensors;
    auto it = m.find(name);
    if (it == m.end()) return report(model::Error::make(AQ_ERR_INDEX, std::string("no tensor named ") + name));
    const safetensors::Tensor& t = it->second;
    if (t.Shape.size() > 8 || t.Dtype.size() > 15) return report(model::Error::make(AQ_ERR_UNSUPPORTED, "tensor rank or dtype name too long"));
    if (dtype) {
        memset(dtype, 0, 16);
        memcpy(dtype, t.Dtype.c_str(), t.Dtype.size());
    }
    if (shape)
        for (size_t i = 0; i < t.Shape.size(); i++) shape[i] = t.Shape[i];
    if (rank) *rank = (int)t.Shape.size();
    if (data) *data = t.Data;
    if (len) *len = t.Len;
    return AQ_OK;
}

int aqh_load_linear(aqh_safetensors* f, const char* prefix, int in_dim, aqh_linear* out) {
    if (!f || !prefix || !out) return report(model::Error::make(AQ_ERR_ARG, "aqh_load_linear: bad argument"));
    memset(out, 0, sizeof *out);
    auto lin = model::LoadLinear(reinterpret_cast<safetensors::File*>(f), prefix, in_dim, "affine");
    if (!lin) return report(model::Error::make(AQ_ERR_INDEX, std::string("no weight at ") + prefix));
    out->weight = lin->Weight, out->weight_len = lin->WeightLen;
    out->scales = lin->Scales, out->scales_len = lin->ScalesLen;
    out->biases = lin->Biases, out->biases_len = lin->BiasesLen;
    out->bias = lin->Bias, out->bias_len = lin->BiasLen;
    out->out_dim = lin->OutDim, out->in_dim = lin->InDim, out->group_size = lin->GroupSize, out->bits = lin->Bits;
    out->quantised = lin->Quantised() ? 1 : 0;
    if (lin->WeightShape.size() == 3) {
        out->experts = lin->WeightShape[0];
        out->expert_rows = lin->WeightShape[1];
    } else {
        out->experts = 0;
        out->expert_rows = lin->OutDim;
    }
    return AQ_OK;
}

int aqh_repack_b1_to_b2(const uint8_t* packed, size_t packed_len, size_t scales_len, size_t biases_len, int out_dim,
                        int in_dim, int group_size, uint8_t* packed2, size_t packed2_len) {
    if (!packed || !packed2) return report(model::Error::make(AQ_ERR_ARG, "aqh_repack_b1_to_b2: bad argument"));
    model::Bytes p2;
    model::Error e = model::RepackB1ToB2(packed, packed_len, scales_len, biases_len, out_dim, in_dim, group_size, &p2);
    if (!e.ok()) return report(e);
    if (p2.size() != packed2_len) return report(model::Error::make(AQ_ERR_SIZE, "aqh_repack_b1_to_b2: packed2 must hold out_dim*in_dim/4 bytes"));
    memcpy(packed2, p2.data(), p2.size());
    return AQ_OK;
}

}  // extern "C"
