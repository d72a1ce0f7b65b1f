// The "rocm" backend's affine quant compute: what a go-inference engine/hip
// build registers so that model.BackendQuant("rocm", "affine") and
// attn.ProjQuantMatMulInto reach the gfx950 kernels.  Mirrors the Metal
// backend's bindings (go/engine/metal/model_quant.go:15-27,
// go/engine/metal/quant_seam_backend.go:27-75) on top of libaq_mi355's C ABI.
#pragma once
#include "model_quant.h"

struct aq_ctx;

namespace rocm {

constexpr const char* kBackendName = "rocm";

// Process-wide context (the Go side's ensureInit()).  Error if no gfx950 device.
model::Error EnsureInit(int device = 0);
aq_ctx* Context();

class AffineQuant final : public model::QuantMatVec {
   public:
    std::string Kind() const override { return "affine"; }
    int Bits() const override { return 0; }
    model::Error MatVec(const uint8_t* x, size_t x_len, const uint8_t* packed, size_t packed_len,
                        const uint8_t* scales, size_t scales_len, const uint8_t* biases, size_t biases_len, int outDim,
                        int inDim, int groupSize, int bits, model::Bytes* out) override;
};

// native.MatMulQuantF32NTInto (go/engine/metal/quant_seam_backend.go:37-75).
model::Error MatMulQuantF32NTInto(std::vector<float>* out, const float* x, size_t x_len, const uint8_t* packed,
                                  size_t packed_len, const uint8_t* scales, size_t scales_len, const uint8_t* biases,
                                  size_t biases_len, int M, int K, int N, int groupSize, int bits);

// The backend package's init(): registers ("rocm","affine") and binds the seam.
void Register();

}  // namespace rocm
