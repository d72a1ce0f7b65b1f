// model.ConcatQuantRows (go/model/quant_weight.go:45-63) and affineGeometry
// (go/model/linear.go:91-110).
#include "model_quant.h"

namespace model {

std::unique_ptr<QuantWeight> ConcatQuantRows(const QuantWeight* a, const QuantWeight* b) {
    if (!a || !b || a->InDim != b->InDim || a->Bits != b->Bits || a->GroupSize != b->GroupSize) return nullptr;
    auto cat = [](const Bytes& x, const Bytes& y) {
        Bytes out;
        out.reserve(x.size() + y.size());
        out.insert(out.end(), x.begin(), x.end());
        out.insert(out.end(), y.begin(), y.end());
        return out;
    };
    auto w = std::make_unique<QuantWeight>();
    w->Packed = cat(a->Packed, b->Packed);
    w->Scales = cat(a->Scales, b->Scales);
    w->Biases = cat(a->Biases, b->Biases);
    w->Bits = a->Bits;
    w->GroupSize = a->GroupSize;
    w->OutDim = a->OutDim + b->OutDim;
    w->InDim = a->InDim;
    return w;
}

static int lastDim(const std::vector<int>& shape) { return shape.empty() ? 0 : shape.back(); }

void affineGeometry(int inDim, const std::vector<int>& scalesShape, const std::vector<int>& weightShape,
                    int* groupSize, int* bits) {
    *groupSize = 0;
    *bits = 0;
    if (inDim <= 0) return;
    if (int n = lastDim(scalesShape); n > 0) *groupSize = inDim / n;
    if (int packedCols = lastDim(weightShape); packedCols > 0) *bits = packedCols * 32 / inDim;
}

}  // namespace model
