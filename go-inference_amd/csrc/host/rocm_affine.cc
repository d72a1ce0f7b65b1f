#include "rocm_affine.h"

#include <mutex>

#include "../../../include/aq_mi355.h"

namespace rocm {

namespace {
std::mutex g_mu;
aq_ctx* g_ctx = nullptr;

model::Error from_rc(int rc) {
    if (rc == AQ_OK) return model::Error::none();
    return model::Error::make(rc, aq_last_error());
}
}  // namespace

model::Error EnsureInit(int device) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_ctx) return model::Error::none();
    return from_rc(aq_create(device, &g_ctx));
}

aq_ctx* Context() { return g_ctx; }

model::Error AffineQuant::MatVec(const uint8_t* x, size_t x_len, const uint8_t* packed, size_t packed_len,
                                 const uint8_t* scales, size_t scales_len, const uint8_t* biases, size_t biases_len,
                                 int outDim, int inDim, int groupSize, int bits, model::Bytes* out) {
    if (!out) return model::Error::make(AQ_ERR_ARG, "rocm.AffineQuant.MatVec: out is null");
    out->clear();
    if (outDim < 0 || inDim < 0)
        return model::Error::make(AQ_ERR_SHAPE, "rocm.AffineQuant.MatVec: outDim/inDim must be non-negative");
    // zero-sized fast path returns an empty/zeroed slice and never touches the device (qmv.go:365-371)
    if (outDim == 0 || inDim == 0) {
        out->assign((size_t)outDim * 2, 0);
        return model::Error::none();
    }
    if (model::Error e = EnsureInit(); !e.ok()) return e;
    out->assign((size_t)outDim * 2, 0);
    int rc = aq_matvec_host(g_ctx, x, x_len, packed, packed_len, scales, scales_len, biases, biases_len, outDim, inDim,
                            groupSize, bits, out->data(), out->size());
    if (rc != AQ_OK) out->clear();
    return from_rc(rc);
}

model::Error MatMulQuantF32NTInto(std::vector<float>* out, const float* x, size_t x_len, const uint8_t* packed,
                                  size_t packed_len, const uint8_t* scales, size_t scales_len, const uint8_t* biases,
                                  size_t biases_len, int M, int K, int N, int groupSize, int bits) {
    if (!out) return model::Error::make(AQ_ERR_ARG, "rocm.MatMulQuantF32NTInto: out is null");
    if (model::Error e = EnsureInit(); !e.ok()) return e;
    if (M <= 0 || N <= 0 || K <= 0)
        return model::Error::make(AQ_ERR_SHAPE, "rocm.MatMulQuantF32NTInto: M, N, K must be positive");
    const size_t want = (size_t)M * (size_t)N;
    std::vector<float> res(want);
    int rc = aq_proj_quant_matmul_host(g_ctx, res.data(), x, x_len, packed, packed_len, scales, scales_len, biases,
                                       biases_len, M, K, N, groupSize, bits);
    if (rc != AQ_OK) return from_rc(rc);
    // reuse the caller's buffer when it is large enough (cap(out) >= M*N), else hand back a new one
    if (out->capacity() >= want) {
        out->assign(res.begin(), res.end());
    } else {
        out->swap(res);
    }
    return model::Error::none();
}

void Register() {
    model::RegisterBackendQuant(kBackendName, std::make_shared<AffineQuant>());
    attn::ProjQuantMatMulInto = MatMulQuantF32NTInto;
}

}  // namespace rocm
