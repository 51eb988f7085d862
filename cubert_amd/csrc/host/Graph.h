// Weights of a frozen TensorFlow GraphDef (.pb), by node name.  Public surface
// of the reference's Graph<T> (src/cuBERT/tensorflow/Graph.h:10-23).
//
// The file is read with a small protobuf wire-format reader that knows only
// the fields the loader needs:
//   GraphDef.node(1) -> NodeDef{ name(1), attr(5) = map<string, AttrValue> }
//   AttrValue.tensor(8) -> TensorProto{ dtype(1), tensor_shape(2){ dim(2){ size(1) } }, tensor_content(4) }
// Every node whose attr "value" holds a DT_FLOAT(1) or DT_HALF(19) tensor with
// tensor_content becomes var[name], converted to T.
#ifndef CUBERT_HOST_GRAPH_H
#define CUBERT_HOST_GRAPH_H

#include <cstddef>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"

namespace cuBERT {

template <typename T>
class Graph {
public:
    explicit Graph(const char *filename);
    ~Graph();

    Graph(const Graph &) = delete;
    Graph &operator=(const Graph &) = delete;

    std::unordered_map<std::string, T *> var;
    std::unordered_map<std::string, std::vector<long long>> shape;
    std::unordered_map<std::string, size_t> size;  // elements held by var[name]

    size_t vocab_size = 0;
    size_t type_vocab_size = 0;
    size_t hidden_size = 0;
    size_t intermediate_size = 0;
    size_t num_labels = 1;

private:
    // Owns what var points at.  A member (not the destructor) so that a constructor that throws half way
    // through a damaged file releases what it had already converted.
    std::vector<std::unique_ptr<T[]>> storage;
};

}  // namespace cuBERT

#endif  // CUBERT_HOST_GRAPH_H
