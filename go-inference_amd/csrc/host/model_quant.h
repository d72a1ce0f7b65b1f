// C++ mirror of go-inference's backend-agnostic quant contract, so the library
// can be exercised through the same plug-in surface a Go backend registers
// against.  Names follow the Go declarations they mirror:
//   model.QuantMatVec / RegisterBackendQuant / BackendQuant   go/model/quant.go:35-63
//   model.QuantWeight / ConcatQuantRows                        go/model/quant_weight.go:22-63
//   model.Linear geometry (affineGeometry, lastDim)            go/model/linear.go:91-110
//   attn.ProjQuantMatMulInto                                   go/model/attn/gated_delta.go:46-51
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <vector>

namespace model {

// Go `error`: ok() == (err == nil).
struct Error {
    int code = 0;
    std::string msg;
    bool ok() const { return code == 0; }
    static Error none() { return Error{}; }
    static Error make(int code, std::string msg) { return Error{code, std::move(msg)}; }
};

using Bytes = std::vector<uint8_t>;

// go/model/quant.go:35-38.  Raw bytes in and out: bf16 activations, MLX packed
// weight + bf16 scales/biases; the result is a freshly allocated outDim*2-byte
// slice.  Bits() == 0 means "the model config declares the width".
class QuantMatVec {
   public:
    virtual ~QuantMatVec() = default;
    virtual std::string Kind() const = 0;
    virtual int Bits() const = 0;
    virtual Error MatVec(const uint8_t* x, size_t x_len, const uint8_t* packed, size_t packed_len,
                         const uint8_t* scales, size_t scales_len, const uint8_t* biases, size_t biases_len,
                         int outDim, int inDim, int groupSize, int bits, Bytes* out) = 0;
};

// go/model/quant.go:48-63: keyed "backend/kind", a second registration replaces the first.
void RegisterBackendQuant(const std::string& backend, std::shared_ptr<QuantMatVec> q);
std::shared_ptr<QuantMatVec> BackendQuant(const std::string& backend, const std::string& kind);

// go/model/quant_weight.go:22-30
struct QuantWeight {
    Bytes Packed;  // [OutDim, InDim*Bits/32] u32 little-endian
    Bytes Scales;  // [OutDim, InDim/GroupSize] bf16
    Bytes Biases;
    int Bits = 0;
    int GroupSize = 0;
    int OutDim = 0;
    int InDim = 0;
};

// go/model/quant_weight.go:45-63: row concatenation is a byte append; nullptr on a nil
// input or a geometry mismatch.
std::unique_ptr<QuantWeight> ConcatQuantRows(const QuantWeight* a, const QuantWeight* b);

// go/model/linear.go:91-102: groupSize = inDim / lastDim(scales), bits = lastDim(packed)*32 / inDim.
void affineGeometry(int inDim, const std::vector<int>& scalesShape, const std::vector<int>& weightShape,
                    int* groupSize, int* bits);

}  // namespace model

namespace attn {

// go/model/attn/gated_delta.go:46-51: out[M,N] = x[M,K] . dequant(w)^T, f32 at the seam.
// `out` is reused when its capacity is at least M*N, as the Go hook reuses cap(out).
using ProjQuantMatMulIntoFn =
    std::function<model::Error(std::vector<float>* out, const float* x, size_t x_len, const uint8_t* packed,
                               size_t packed_len, const uint8_t* scales, size_t scales_len, const uint8_t* biases,
                               size_t biases_len, int M, int K, int N, int groupSize, int bits)>;
extern ProjQuantMatMulIntoFn ProjQuantMatMulInto;  // empty == Go nil

}  // namespace attn
