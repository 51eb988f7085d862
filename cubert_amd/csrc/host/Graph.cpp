#include "Graph.h"

#include <cstdint>
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
};

Tensor read_tensor(Reader r) {
    Tensor t;
    uint32_t f, w;
    while (r.next(&f, &w)) {
        if (f == 1 && w == 0) {
            t.dtype = (int) r.varint();
        } else if (f == 2 && w == 2) {  // TensorShapeProto
            Reader s = r.bytes();
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
        } else {
            r.skip(w);
        }
    }
    return t;
}

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
                        attr.skip(aw);
                    }
                }
            } else {
                node.skip(nw);
            }
        }
        if (!has_value) continue;

        size_t len;
        if (value.dtype == kDtFloat) len = (size_t) (value.content.end - value.content.p) / sizeof(float);
        else if (value.dtype == kDtHalf) len = (size_t) (value.content.end - value.content.p) / sizeof(half);
        else continue;

        // a declared shape must describe the bytes that are there (a scalar has no dims)
        unsigned long long declared = 1;
        for (long long d : value.dims) {
            if (d < 0 || (d > 0 && declared > (1ull << 40) / (unsigned long long) d)) {
                throw std::invalid_argument("model file invalid: bad shape of " + name);
            }
            declared *= (unsigned long long) d;
        }
        if (declared != len) {
            throw std::invalid_argument("model file invalid: " + name + " holds " + std::to_string(len) +
                                        " elements, its shape says " + std::to_string(declared));
        }

        storage.emplace_back(new T[len]);
        T *data = storage.back().get();
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
