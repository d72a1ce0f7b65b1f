// model.RegisterBackendQuant / BackendQuant (go/model/quant.go:40-63).
#include <map>
#include <mutex>

#include "model_quant.h"

namespace model {

namespace {
std::mutex& mu() {
    static std::mutex m;
    return m;
}
std::map<std::string, std::shared_ptr<QuantMatVec>>& table() {
    static std::map<std::string, std::shared_ptr<QuantMatVec>> t;
    return t;
}
std::string key(const std::string& backend, const std::string& kind) { return backend + "/" + kind; }
}  // namespace

void RegisterBackendQuant(const std::string& backend, std::shared_ptr<QuantMatVec> q) {
    if (!q) return;
    std::lock_guard<std::mutex> lk(mu());
    table()[key(backend, q->Kind())] = std::move(q);
}

std::shared_ptr<QuantMatVec> BackendQuant(const std::string& backend, const std::string& kind) {
    std::lock_guard<std::mutex> lk(mu());
    auto it = table().find(key(backend, kind));
    return it == table().end() ? nullptr : it->second;
}

}  // namespace model

namespace attn {
ProjQuantMatMulIntoFn ProjQuantMatMulInto;
}
