// safetensors reader and the per-weight loader that sits on it.
//   go/model/safetensors/safetensors.go:53-95     file framing
//   go/model/safetensors/header_parse.go:343-437  tensor entry: dtype, shape, data_offsets required;
//                                                 unknown keys skipped; begin >= 0, end >= begin
//   go/model/linear.go:42-84                      LoadLinear
//   go/model/quant/mlxaffine/repack.go:27-62      RepackB1ToB2
#include "safetensors.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>

#include "../../../include/aq_mi355.h"

namespace safetensors {

namespace {

// Just enough JSON for a safetensors header.
struct Parser {
    const uint8_t* p;
    const uint8_t* end;
    bool fail = false;

    void ws() {
        while (p < end && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) p++;
    }
    bool eat(char c) {
        ws();
        if (p < end && *p == (uint8_t)c) {
            p++;
            return true;
        }
        return false;
    }
    char peek() {
        ws();
        return p < end ? (char)*p : '\0';
    }
    static void utf8(std::string* out, uint32_t cp) {
        if (cp < 0x80) {
            out->push_back((char)cp);
        } else if (cp < 0x800) {
            out->push_back((char)(0xC0 | (cp >> 6)));
            out->push_back((char)(0x80 | (cp & 0x3F)));
        } else if (cp < 0x10000) {
            out->push_back((char)(0xE0 | (cp >> 12)));
            out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
            out->push_back((char)(0x80 | (cp & 0x3F)));
        } else {
            out->push_back((char)(0xF0 | (cp >> 18)));
            out->push_back((char)(0x80 | ((cp >> 12) & 0x3F)));
            out->push_back((char)(0x80 | ((cp >> 6) & 0x3F)));
            out->push_back((char)(0x80 | (cp & 0x3F)));
        }
    }
    bool hex4(uint32_t* v) {
        if (end - p < 4) return false;
        uint32_t r = 0;
        for (int i = 0; i < 4; i++) {
            const uint8_t c = p[i];
            r <<= 4;
            if (c >= '0' && c <= '9') r |= c - '0';
            else if (c >= 'a' && c <= 'f') r |= c - 'a' + 10;
            else if (c >= 'A' && c <= 'F') r |= c - 'A' + 10;
            else return false;
        }
        p += 4;
        *v = r;
        return true;
    }
    bool string(std::string* out) {
        if (!eat('"')) return false;
        out->clear();
        while (p < end) {
            const uint8_t c = *p++;
            if (c == '"') return true;
            if (c != '\\') {
                out->push_back((char)c);
                continue;
            }
            if (p >= end) return false;
            const uint8_t e = *p++;
            switch (e) {
                case '"': out->push_back('"'); break;
                case '\\': out->push_back('\\'); break;
                case '/': out->push_back('/'); break;
                case 'b': out->push_back('\b'); break;
                case 'f': out->push_back('\f'); break;
                case 'n': out->push_back('\n'); break;
                case 'r': out->push_back('\r'); break;
                case 't': out->push_back('\t'); break;
                case 'u': {
                    uint32_t cp;
                    if (!hex4(&cp)) return false;
                    // every \uXXXX escape becomes the UTF-8 form of its own 16-bit value, surrogate halves included
                    // (header_parse.go:262-292 does not pair them): tensor names keep the reference's bytes
                    utf8(out, cp);
                    break;
                }
                default: return false;
            }
        }
        return false;
    }
    bool int64(int64_t* v) {
        ws();
        bool neg = false;
        if (p < end && *p == '-') {
            neg = true;
            p++;
        }
        if (p >= end || *p < '0' || *p > '9') return false;
        int64_t r = 0;
        while (p < end && *p >= '0' && *p <= '9') {
            if (r > (INT64_MAX - 9) / 10) return false;
            r = r * 10 + (*p - '0');
            p++;
        }
        if (p < end && (*p == '.' || *p == 'e' || *p == 'E')) return false;  // integers only
        *v = neg ? -r : r;
        return true;
    }
    bool skip_value(int depth = 0) {
        if (depth > 64) return false;
        const char c = peek();
        if (c == '"') {
            std::string s;
            return string(&s);
        }
        if (c == '{') {
            p++;
            if (eat('}')) return true;
            do {
                std::string k;
                if (!string(&k) || !eat(':') || !skip_value(depth + 1)) return false;
            } while (eat(','));
            return eat('}');
        }
        if (c == '[') {
            p++;
            if (eat(']')) return true;
            do {
                if (!skip_value(depth + 1)) return false;
            } while (eat(','));
            return eat(']');
        }
        // number / true / false / null
        const uint8_t* start = p;
        while (p < end && *p != ',' && *p != '}' && *p != ']' && *p != ' ' && *p != '\n' && *p != '\t' && *p != '\r') p++;
        return p > start;
    }
};

size_t dtype_bytes(const std::string& d) {
    if (d == "F64" || d == "I64" || d == "U64") return 8;
    if (d == "F32" || d == "I32" || d == "U32") return 4;
    if (d == "F16" || d == "BF16" || d == "I16" || d == "U16") return 2;
    if (d == "I8" || d == "U8" || d == "BOOL" || d == "F8_E4M3" || d == "F8_E5M2") return 1;
    return 0;
}

model::Error bad(const std::string& msg) { return model::Error::make(AQ_ERR_SHAPE, "safetensors: " + msg); }

}  // namespace

File::~File() {
    if (map_) munmap(map_, map_len_);
}

model::Error File::Open(const std::string& path, std::unique_ptr<File>* out) {
    out->reset();
    const int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) return model::Error::make(AQ_ERR_ARG, "safetensors.ReadSafetensors: read file: " + path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 8) {
        close(fd);
        return bad("file too small");
    }
    void* m = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (m == MAP_FAILED) return model::Error::make(AQ_ERR_NOMEM, "safetensors: mmap failed: " + path);
    std::unique_ptr<File> f(new File());
    f->map_ = m;
    f->map_len_ = (size_t)st.st_size;
    model::Error e = f->Parse(static_cast<const uint8_t*>(m), f->map_len_);
    if (!e.ok()) return e;
    *out = std::move(f);
    return model::Error::none();
}

model::Error File::Parse(const uint8_t* data, size_t len) {
    Tensors.clear();
    Metadata.clear();
    if (len < 8) return bad("file too small");
    uint64_t header_size = 0;
    for (int i = 7; i >= 0; i--) header_size = (header_size << 8) | data[i];
    if (header_size > len - 8) return bad("invalid header size " + std::to_string(header_size));
    const uint8_t* payload = data + 8 + header_size;
    const size_t payload_len = len - 8 - (size_t)header_size;
    Parser ps{data + 8, data + 8 + header_size};
    if (!ps.eat('{')) return bad("parse header: not an object");
    if (!ps.eat('}')) {
        do {
            std::string name;
            if (!ps.string(&name) || !ps.eat(':')) return bad("parse header: bad key");
            if (name == "__metadata__") {
                if (!ps.eat('{')) return bad("parse header: __metadata__ is not an object");
                if (!ps.eat('}')) {
                    do {
                        std::string k, v;
                        if (!ps.string(&k) || !ps.eat(':')) return bad("parse header: bad metadata key");
                        if (ps.peek() == '"') {
                            if (!ps.string(&v)) return bad("parse header: bad metadata value");
                            Metadata[k] = v;
                        } else if (!ps.skip_value()) {
                            return bad("parse header: bad metadata value");
                        }
                    } while (ps.eat(','));
                    if (!ps.eat('}')) return bad("parse header: unterminated __metadata__");
                }
                continue;
            }
            if (!ps.eat('{')) return bad("tensor entry is not an object: " + name);
            Tensor t;
            int64_t begin = 0, endo = 0;
            bool have_dtype = false, have_shape = false, have_offsets = false;
            if (!ps.eat('}')) {
                do {
                    std::string key;
                    if (!ps.string(&key)) return bad("tensor key parse failed: " + name);
                    if (!ps.eat(':')) return bad("tensor entry missing ':': " + name);
                    if (key == "dtype") {
                        if (!ps.string(&t.Dtype)) return bad("dtype is not a string: " + name);
                        have_dtype = true;
                    } else if (key == "shape") {
                        if (!ps.eat('[')) return bad("shape is not an array: " + name);
                        t.Shape.clear();
                        if (!ps.eat(']')) {
                            do {
                                int64_t d;
                                if (!ps.int64(&d) || d < 0 || d > INT32_MAX) return bad("shape dimension is invalid: " + name);
                                t.Shape.push_back((int)d);
                            } while (ps.eat(','));
                            if (!ps.eat(']')) return bad("shape is unterminated: " + name);
                        }
                        have_shape = true;
                    } else if (key == "data_offsets") {
                        if (!ps.eat('[') || !ps.int64(&begin) || !ps.eat(',') || !ps.int64(&endo) || !ps.eat(']'))
                            return bad("data_offsets must be two integers: " + name);
                        have_offsets = true;
                    } else if (!ps.skip_value()) {
                        return bad("tensor entry has a malformed value: " + name);
                    }
                } while (ps.eat(','));
                if (!ps.eat('}')) return bad("tensor entry is unterminated: " + name);
            }
            if (!have_dtype || !have_shape || !have_offsets) return bad("tensor is missing required field: " + name);
            if (begin < 0 || endo < begin) return bad("tensor offsets are invalid: " + name);
            if ((uint64_t)endo > payload_len) return bad("tensor data lies outside the file: " + name);
            t.Data = payload + begin;
            t.Len = (size_t)(endo - begin);
            if (const size_t eb = dtype_bytes(t.Dtype)) {
                uint64_t elements = 1;
                bool fits = true;  // the product of the dimensions, as long as it can still describe t.Len bytes
                for (int d : t.Shape) {
                    if (d != 0 && elements > (uint64_t)payload_len / (uint64_t)d) fits = false;
                    elements *= (uint64_t)d;
                }
                if (!fits || elements * eb != t.Len) return bad("tensor byte length does not match dtype and shape: " + name);
            }
            Tensors[name] = std::move(t);
        } while (ps.eat(','));
        if (!ps.eat('}')) return bad("parse header: unterminated object");
    }
    return model::Error::none();
}

}  // namespace safetensors

namespace model {

Error RepackB1ToB2(const uint8_t* packed, size_t packed_len, size_t scales_len, size_t biases_len, int outDim, int inDim,
                   int groupSize, Bytes* packed2) {
    if (outDim <= 0 || inDim <= 0 || groupSize <= 0 || inDim % groupSize != 0)
        return Error::make(AQ_ERR_SHAPE, "mlxaffine.RepackB1ToB2: invalid dimensions");
    if (inDim % 32 != 0)
        return Error::make(AQ_ERR_SHAPE, "mlxaffine.RepackB1ToB2: inDim " + std::to_string(inDim) +
                                             " must be a multiple of 32 (b1 packs 32 codes per word)");
    const size_t words1 = (size_t)inDim / 32, words2 = (size_t)inDim / 16;
    if (packed_len != (size_t)outDim * words1 * 4)
        return Error::make(AQ_ERR_SIZE, "mlxaffine.RepackB1ToB2: packed length " + std::to_string(packed_len) + " != " +
                                            std::to_string((size_t)outDim * words1 * 4));
    const size_t want_sb = (size_t)outDim * (size_t)(inDim / groupSize) * 2;
    if (scales_len != want_sb || biases_len != want_sb)
        return Error::make(AQ_ERR_SIZE, "mlxaffine.RepackB1ToB2: scales/biases length does not match [outDim, inDim/groupSize]");
    packed2->assign((size_t)outDim * words2 * 4, 0);
    // every 1-bit word spreads into two 2-bit words: bit j of the source lands at bit 2*(j%16) of word j/16
    for (size_t w = 0; w < (size_t)outDim * words1; w++) {
        uint32_t src;
        memcpy(&src, packed + w * 4, 4);
        uint32_t lo = 0, hi = 0;
        for (int j = 0; j < 16; j++) {
            lo |= ((src >> j) & 1u) << (2 * j);
            hi |= ((src >> (16 + j)) & 1u) << (2 * j);
        }
        memcpy(packed2->data() + (w * 2) * 4, &lo, 4);
        memcpy(packed2->data() + (w * 2 + 1) * 4, &hi, 4);
    }
    return Error::none();
}

std::unique_ptr<Linear> LoadLinear(safetensors::File* f, const std::string& prefix, int inDim, const std::string& kind) {
    if (!f) return nullptr;
    auto w = f->Tensors.find(prefix + ".weight");
    if (w == f->Tensors.end()) return nullptr;
    auto lin = std::make_unique<Linear>();
    lin->Weight = w->second.Data;
    lin->WeightLen = w->second.Len;
    lin->WeightShape = w->second.Shape;
    lin->OutDim = w->second.Shape.empty() ? 0 : w->second.Shape.front();  // firstDim: rows are never packed
    lin->InDim = inDim;
    if (auto b = f->Tensors.find(prefix + ".bias"); b != f->Tensors.end()) {
        lin->Bias = b->second.Data;
        lin->BiasLen = b->second.Len;
    }
    auto s = f->Tensors.find(prefix + ".scales");
    if (s != f->Tensors.end() && s->second.Len > 0) {
        lin->Scales = s->second.Data;
        lin->ScalesLen = s->second.Len;
        if (auto b = f->Tensors.find(prefix + ".biases"); b != f->Tensors.end()) {
            lin->Biases = b->second.Data;
            lin->BiasesLen = b->second.Len;
        }
        lin->Kind = kind;
        affineGeometry(inDim, s->second.Shape, w->second.Shape, &lin->GroupSize, &lin->Bits);
        if (lin->Bits == 1) {
            // no 1-bit kernel ships: widen to the exact 2-bit form and write it back into the tensor map, so
            // that a tied second read finds the widened weight (go/model/linear.go:62-80); on a malformed
            // pack the weight passes through unchanged
            auto p2 = std::make_unique<Bytes>();
            if (RepackB1ToB2(lin->Weight, lin->WeightLen, lin->ScalesLen, lin->BiasesLen, lin->OutDim, inDim,
                             lin->GroupSize, p2.get())
                    .ok()) {
                lin->Weight = p2->data();
                lin->WeightLen = p2->size();
                lin->Bits = 2;
                w->second.Data = p2->data();
                w->second.Len = p2->size();
                w->second.Shape = {lin->OutDim, inDim / 16};
                lin->WeightShape = w->second.Shape;
                f->Owned.push_back(std::move(p2));
            }
        }
    }
    return lin;
}

}  // namespace model
