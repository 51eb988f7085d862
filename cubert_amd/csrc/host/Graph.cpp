#include "Graph.h"

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <fstream>
#include <iostream>
#include <stdexcept>

namespace cuBERT {

namespace {

// A view on a length-delimited protobuf message.
struct Reader {
    const uint8_t *p;
    const uint8_t *end;

    bool done() const { return p >= end; }

    uint64_t varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 64; shift += 7) {
            if (p >= end) throw std::invalid_argument("model file invalid");
            const uint8_t b = *p++;
            v |= (uint64_t) (b & 0x7f) << shift;
            if (!(b & 0x80)) return v;
        }
        throw std::invalid_argument("model file invalid");
    }

    Reader bytes() {
        const uint64_t n = varint();
        if (n > (uint64_t) (end - p)) throw std::invalid_argument("model file invalid");
        Reader r{p, p + n};
        p += n;
        return r;
    }

    // Reads the next tag; returns false at the end of the message.
    bool next(uint32_t *field, uint32_t *wire) {
        if (done()) return false;
        const uint64_t tag = varint();
        *field = (uint32_t) (tag >> 3);
        *wire = (uint32_t) (tag & 7);
        return true;
    }

    void skip(uint32_t wire) {
        switch (wire) {
            case 0: varint(); break;
            case 1: advance(8); break;
            case 2: bytes(); break;
            case 5: advance(4); break;
            default: throw std::invalid_argument("model file invalid");
        }
    }

    void advance(size_t n) {
        if (n > (size_t) (end - p)) throw std::invalid_argument("model file invalid");
        p += n;
    }

    std::string str() const { return std::string((const char *) p, (size_t) (end - p)); }
};

struct Tensor {
    int dtype = 0;
    std::vector<long long> dims;
    Reader content{nullptr, nullptr};
    std::vector<float> float_val;      // TensorProto.float_val(5), packed or one fixed32 per tag
    std::vector<uint16_t> half_val;    // TensorProto.half_val(13): binary16 bit patterns carried as int32
};

float fixed32_as_float(const uint8_t *p) {
    // protobuf fixed32 is little-endian, like every host this library is built for
    float v;
    std::memcpy(&v, p, sizeof(v));
    return v;
}

Tensor read_tensor(Reader r) {
    Tensor t;
    uint32_t f, w;
    while (r.next(&f, &w)) {
        if (f == 1 && w == 0) {
            t.dtype = (int) r.varint();
        } else if (f == 2 && w == 2) {  // TensorShapeProto
            Reader s = r.bytes();
            t.dims.clear();  // a repeated singular message field merges; shapes are written once in practice
            uint32_t sf, sw;
            while (s.next(&sf, &sw)) {
                if (sf == 2 && sw == 2) {  // Dim
                    Reader d = s.bytes();
                    long long size = 0;
                    uint32_t df, dw;
                    while (d.next(&df, &dw)) {
                        if (df == 1 && dw == 0) size = (long long) d.varint();
                        else d.skip(dw);
                    }
                    t.dims.push_back(size);
                } else {
                    s.skip(sw);
                }
            }
        } else if (f == 4 && w == 2) {
            t.content = r.bytes();
        } else if (f == 5 && w == 2) {  // packed float_val
            Reader v = r.bytes();
            while ((size_t) (v.end - v.p) >= 4) {
                t.float_val.push_back(fixed32_as_float(v.p));
                v.p += 4;
            }
        } else if (f == 5 && w == 5) {  // unpacked float_val
            if ((size_t) (r.end - r.p) < 4) throw std::invalid_argument("model file invalid");
            t.float_val.push_back(fixed32_as_float(r.p));
            r.advance(4);
        } else if (f == 13 && w == 2) {  // packed half_val
            Reader v = r.bytes();
            while (!v.done()) t.half_val.push_back((uint16_t) v.varint());
        } else if (f == 13 && w == 0) {  // unpacked half_val
            t.half_val.push_back((uint16_t) r.varint());
        } else {
            r.skip(w);
        }
    }
    return t;
}

// Elements a shape describes; 0 for a shape with a negative (unknown) or absurd dimension.
size_t declared_elements(const std::vector<long long> &dims) {
    unsigned long long n = 1;
    for (long long d : dims) {
        if (d < 0) return 0;
        if (d > 0 && n > (1ull << 40) / (unsigned long long) d) return 0;
        n *= (unsigned long long) d;
    }
    return (size_t) n;
}

// TensorFlow writes a constant of one element, or of many equal elements, as a short float_val / half_val
// list instead of tensor_content; a reader repeats the last listed value up to the declared size.  Such
// constants are scalars and splats of a few elements in a frozen BERT (epsilon, 1/sqrt(d), -10000, ...).
constexpr size_t kMaxExpandedElements = (size_t) 1 << 24;

constexpr int kDtFloat = 1, kDtHalf = 19;

}  // namespace

template <typename T>
Graph<T>::Graph(const char *filename) {
    std::ifstream input(filename, std::ios::binary | std::ios::ate);
    if (!input) {
        throw std::invalid_argument("model file not found");
    }
    const std::streamsize size = input.tellg();
    input.seekg(0);
    std::vector<uint8_t> buffer((size_t) size);
    if (size > 0 && !input.read((char *) buffer.data(), size)) {
        throw std::invalid_argument("model file invalid");
    }
    input.close();
    std::cerr << "model loaded from: " << filename << std::endl;

    Reader graph{buffer.data(), buffer.data() + buffer.size()};
    uint32_t f, w;
    while (graph.next(&f, &w)) {
        if (!(f == 1 && w == 2)) {  // only GraphDef.node
            graph.skip(w);
            continue;
        }
        Reader node = graph.bytes();
        std::string name;
        bool has_value = false;
        Tensor value;
        uint32_t nf, nw;
        while (node.next(&nf, &nw)) {
            if (nf == 1 && nw == 2) {
                name = node.bytes().str();
            } else if (nf == 5 && nw == 2) {  // map entry: key(1), value(2)
                Reader entry = node.bytes();
                std::string key;
                Reader attr{nullptr, nullptr};
                uint32_t ef, ew;
                while (entry.next(&ef, &ew)) {
                    if (ef == 1 && ew == 2) key = entry.bytes().str();
                    else if (ef == 2 && ew == 2) attr = entry.bytes();
                    else entry.skip(ew);
                }
                if (key != "value") continue;
                uint32_t af, aw;
                while (attr.next(&af, &aw)) {
                    if (af == 8 && aw == 2) {  // AttrValue.tensor
                        value = read_tensor(attr.bytes());
                        has_value = true;
                    } else {
                        // AttrValue is a oneof over fields 1..10: the member written last is the one set
                        if (af >= 1 && af <= 10) has_value = false;
                        attr.skip(aw);
                    }
                }
            } else {
                node.skip(nw);
            }
        }
        if (!has_value) continue;
        if (value.dtype != kDtFloat && value.dtype != kDtHalf) continue;

        // The element count is what the file holds, whatever the declared shape says
        // (reference tensorflow/Graph.cpp:50-56: len = tensor_content.len / sizeof).  The sizes of the tensors a
        // model reads are checked where the model is built, against the shapes it needs.
        const size_t elem = value.dtype == kDtFloat ? sizeof(float) : sizeof(half);
        const size_t content_len = (size_t) (value.content.end - value.content.p) / elem;
        const size_t listed = value.dtype == kDtFloat ? value.float_val.size() : value.half_val.size();
        size_t len = content_len;
        if (content_len == 0 && listed > 0) {
            const size_t declared = declared_elements(value.dims);
            len = declared >= listed && declared <= kMaxExpandedElements ? declared : listed;
        } else if (content_len == 0 && !value.dims.empty()) {
            // neither bytes nor a value list, but a declared shape: how TensorFlow's tensor compression writes a
            // tensor whose elements are all zero (proto3 drops the default value of the one listed element)
            const size_t declared = declared_elements(value.dims);
            if (declared <= kMaxExpandedElements) len = declared;
        }

        storage.emplace_back(new T[len]);
        T *data = storage.back().get();
        if (content_len > 0) {
            // tensor_content sits at an arbitrary byte offset of the file: copy out before converting
            if (value.dtype == kDtFloat) {
                std::vector<float> tmp(len);
                std::memcpy(tmp.data(), value.content.p, len * sizeof(float));
                T2T(tmp.data(), data, len);
            } else {
                std::vector<half> tmp(len);
                std::memcpy(tmp.data(), value.content.p, len * sizeof(half));
                T2T(tmp.data(), data, len);
            }
        } else if (len > 0) {
            if (value.dtype == kDtFloat) {
                std::vector<float> tmp(len, listed > 0 ? value.float_val.back() : 0.f);
                std::copy(value.float_val.begin(), value.float_val.end(), tmp.begin());
                T2T(tmp.data(), data, len);
            } else {
                std::vector<half> tmp(len);
                for (size_t i = 0; i < len; ++i) {
                    const uint16_t bits = listed > 0 ? value.half_val[i < listed ? i : listed - 1] : (uint16_t) 0;
                    std::memcpy(&tmp[i], &bits, sizeof(bits));
                }
                T2T(tmp.data(), data, len);
            }
        }
        var[name] = data;  // a repeated name keeps its last tensor
        shape[name] = value.dims;
        this->size[name] = len;

        const std::vector<long long> &d = value.dims;
        if (name == "bert/embeddings/word_embeddings" && d.size() >= 2) {
            vocab_size = (size_t) d[0];
            hidden_size = (size_t) d[1];
        } else if (name == "bert/embeddings/token_type_embeddings" && d.size() >= 2) {
            type_vocab_size = (size_t) d[0];
            hidden_size = (size_t) d[1];
        } else if (name == "bert/encoder/layer_0/intermediate/dense/bias" && d.size() >= 1) {
            intermediate_size = (size_t) d[0];
        } else if (name == "output_weights" && d.size() >= 1) {
            num_labels = (size_t) d[0];
        }
    }

    if (var.empty()) {
        throw std::invalid_argument("model file invalid");
    }
    std::cerr << "model param: {vocab_size=" << vocab_size << ";type_vocab_size=" << type_vocab_size
              << ";hidden_size=" << hidden_size << ";intermediate_size=" << intermediate_size
              << ";num_labels=" << num_labels << "}" << std::endl;
}

template <typename T>
Graph<T>::~Graph() = default;

template class Graph<float>;
template class Graph<half>;

}  // namespace cuBERT
