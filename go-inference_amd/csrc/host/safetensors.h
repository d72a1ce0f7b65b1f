// Read-only view of a safetensors file: 8-byte little-endian header length, a JSON header
// {name: {"dtype": str, "shape": [ints], "data_offsets": [begin, end]}, "__metadata__": {...}},
// then the tensor bytes.  The file is memory-mapped and tensors are views into the mapping, the
// zero-copy contract of go/model/safetensors (ReadSafetensors, safetensors.go:53-95; entry
// validation header_parse.go:343-437).
#pragma once
#include <cstddef>
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "model_quant.h"

namespace safetensors {

struct Tensor {
    std::string Dtype;
    std::vector<int> Shape;
    const uint8_t* Data = nullptr;  // view into the mapping (or into an owned buffer after a repack)
    size_t Len = 0;
};

class File {
   public:
    ~File();
    static model::Error Open(const std::string& path, std::unique_ptr<File>* out);
    // Parses an in-memory image (tests; the mapping path ends here too).
    model::Error Parse(const uint8_t* data, size_t len);

    std::map<std::string, Tensor> Tensors;  // "__metadata__" is dropped, as ReadSafetensors does
    std::map<std::string, std::string> Metadata;
    // Buffers that replaced a mapped tensor (the 1-bit -> 2-bit repack writes its result back into
    // the tensor map, go/model/linear.go:74-79); they live as long as the file.
    std::vector<std::unique_ptr<model::Bytes>> Owned;

   private:
    void* map_ = nullptr;
    size_t map_len_ = 0;
};

}  // namespace safetensors

namespace model {

// go/model/linear.go:21-33
struct Linear {
    const uint8_t* Weight = nullptr;
    size_t WeightLen = 0;
    const uint8_t* Scales = nullptr;
    size_t ScalesLen = 0;
    const uint8_t* Biases = nullptr;
    size_t BiasesLen = 0;
    const uint8_t* Bias = nullptr;
    size_t BiasLen = 0;
    int OutDim = 0, InDim = 0, GroupSize = 0, Bits = 0;
    std::string Kind;
    std::vector<int> WeightShape;  // beyond the Go struct: rank-3 expert stacks keep [E, rows, words]
    bool Quantised() const { return Scales != nullptr && !Kind.empty(); }
};

// go/model/linear.go:42-84.  nullptr when prefix+".weight" is absent.
std::unique_ptr<Linear> LoadLinear(safetensors::File* f, const std::string& prefix, int inDim, const std::string& kind);

// mlxaffine.RepackB1ToB2, go/model/quant/mlxaffine/repack.go:27-62 (packed codes only; scales and biases
// are invariant and stay where they are).
Error RepackB1ToB2(const uint8_t* packed, size_t packed_len, size_t scales_len, size_t biases_len, int outDim, int inDim,
                   int groupSize, Bytes* packed2);

}  // namespace model
