"""Writes tests/golden/tf_style_graphdef.pb and tf_style_graphdef_expected.npz.

The loader under test (cubert_amd/csrc/host/Graph.cpp) has its own wire-format reader, and the package's own
writer (cubert_amd/graphdef.py) emits one shape of node only.  This script is an independent encoder: it declares
the TensorFlow framework messages to google.protobuf at run time, field by field, with the numbers of the .proto
files the reference vendors (reference tensorflow/core/framework/graph.proto, node_def.proto, attr_value.proto,
tensor.proto, tensor_shape.proto, versions.proto, function.proto, types.proto) and lets the protobuf library
serialise a GraphDef the way TensorFlow's freeze_graph writes one:

  * a tiny BERT's weights as `Const` nodes with tensor_content (what make_tensor_proto does for > 1 element),
    one of them stored as DT_HALF;
  * scalar constants in float_val and half_val, packed (proto3 default) and unpacked (second message set whose
    repeated scalars are declared [packed = false]; the wire format allows both and parsers must accept both);
  * a splat (shape [5], one float_val), a one-element vector in float_val, an empty Const, all-zero tensors
    written as a bare shape (what TensorFlow's tensor compression leaves of them);
  * nodes that are not weights: Placeholder, MatMul with bool/type attrs, an op with a float attr (fixed32),
    int32 Consts in tensor_content and int_val, a node whose attr "value" is a string, a list attr;
  * GraphDef.versions, GraphDef.version and a GraphDef.library whose FunctionDef holds a Const named like a
    weight (must not be picked up: it is not a GraphDef.node);
  * one repeated node name (the later node wins, reference tensorflow/Graph.cpp:66).

Needs only numpy and google.protobuf; run in the build container:  python tests/golden/make_tf_graphdef_fixture.py
"""
import os
import sys

import numpy as np
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

FD = descriptor_pb2.FieldDescriptorProto
DT_FLOAT, DT_INT32, DT_BOOL, DT_HALF = 1, 3, 10, 19  # types.proto

TINY = dict(vocab=37, hidden=16, layers=2, heads=2, intermediate=32, max_position=12, type_vocab=2)
TINY_LABELS = 3
TINY_SEQ = 8


def _messages(package, packed):
    """The message classes of one package.  packed=False declares every repeated scalar [packed = false]."""
    f = descriptor_pb2.FileDescriptorProto(name=package + ".proto", package=package, syntax="proto3")

    def msg(parent, name):
        m = parent.message_type.add() if parent is f else parent.nested_type.add()
        m.name = name
        return m

    def field(m, name, number, ftype, label=FD.LABEL_OPTIONAL, type_name=None, oneof=None):
        x = m.field.add(name=name, number=number, type=ftype, label=label)
        if type_name:
            x.type_name = "." + package + "." + type_name
        if oneof is not None:
            x.oneof_index = oneof
        if label == FD.LABEL_REPEATED and not packed and ftype in (
                FD.TYPE_INT32, FD.TYPE_INT64, FD.TYPE_FLOAT, FD.TYPE_DOUBLE, FD.TYPE_BOOL, FD.TYPE_ENUM):
            x.options.packed = False
        return x

    def map_field(m, name, number, value_type, value_type_name=None):
        entry = msg(m, "".join(p.capitalize() for p in name.split("_")) + "Entry")
        entry.options.map_entry = True
        field(entry, "key", 1, FD.TYPE_STRING)
        field(entry, "value", 2, value_type, type_name=value_type_name)
        field(m, name, number, FD.TYPE_MESSAGE, FD.LABEL_REPEATED, m.name + "." + entry.name)

    R = FD.LABEL_REPEATED
    shape = msg(f, "TensorShapeProto")                       # tensor_shape.proto
    dim = msg(shape, "Dim")
    field(dim, "size", 1, FD.TYPE_INT64)
    field(dim, "name", 2, FD.TYPE_STRING)
    field(shape, "dim", 2, FD.TYPE_MESSAGE, R, "TensorShapeProto.Dim")
    field(shape, "unknown_rank", 3, FD.TYPE_BOOL)

    tensor = msg(f, "TensorProto")                           # tensor.proto
    field(tensor, "dtype", 1, FD.TYPE_INT32)                 # DataType enum, carried as its number
    field(tensor, "tensor_shape", 2, FD.TYPE_MESSAGE, type_name="TensorShapeProto")
    field(tensor, "version_number", 3, FD.TYPE_INT32)
    field(tensor, "tensor_content", 4, FD.TYPE_BYTES)
    field(tensor, "float_val", 5, FD.TYPE_FLOAT, R)
    field(tensor, "double_val", 6, FD.TYPE_DOUBLE, R)
    field(tensor, "int_val", 7, FD.TYPE_INT32, R)
    field(tensor, "string_val", 8, FD.TYPE_BYTES, R)
    field(tensor, "int64_val", 10, FD.TYPE_INT64, R)
    field(tensor, "bool_val", 11, FD.TYPE_BOOL, R)
    field(tensor, "half_val", 13, FD.TYPE_INT32, R)

    attr = msg(f, "AttrValue")                               # attr_value.proto
    lst = msg(attr, "ListValue")
    field(lst, "s", 2, FD.TYPE_BYTES, R)
    field(lst, "i", 3, FD.TYPE_INT64, R)
    field(lst, "f", 4, FD.TYPE_FLOAT, R)
    field(lst, "b", 5, FD.TYPE_BOOL, R)
    field(lst, "type", 6, FD.TYPE_INT32, R)
    field(lst, "shape", 7, FD.TYPE_MESSAGE, R, "TensorShapeProto")
    field(lst, "tensor", 8, FD.TYPE_MESSAGE, R, "TensorProto")
    attr.oneof_decl.add(name="value")
    field(attr, "list", 1, FD.TYPE_MESSAGE, type_name="AttrValue.ListValue", oneof=0)
    field(attr, "s", 2, FD.TYPE_BYTES, oneof=0)
    field(attr, "i", 3, FD.TYPE_INT64, oneof=0)
    field(attr, "f", 4, FD.TYPE_FLOAT, oneof=0)
    field(attr, "b", 5, FD.TYPE_BOOL, oneof=0)
    field(attr, "type", 6, FD.TYPE_INT32, oneof=0)
    field(attr, "shape", 7, FD.TYPE_MESSAGE, type_name="TensorShapeProto", oneof=0)
    field(attr, "tensor", 8, FD.TYPE_MESSAGE, type_name="TensorProto", oneof=0)
    field(attr, "placeholder", 9, FD.TYPE_STRING, oneof=0)

    node = msg(f, "NodeDef")                                 # node_def.proto
    field(node, "name", 1, FD.TYPE_STRING)
    field(node, "op", 2, FD.TYPE_STRING)
    field(node, "input", 3, FD.TYPE_STRING, R)
    field(node, "device", 4, FD.TYPE_STRING)
    map_field(node, "attr", 5, FD.TYPE_MESSAGE, "AttrValue")

    versions = msg(f, "VersionDef")                          # versions.proto
    field(versions, "producer", 1, FD.TYPE_INT32)
    field(versions, "min_consumer", 2, FD.TYPE_INT32)
    field(versions, "bad_consumers", 3, FD.TYPE_INT32, R)

    opdef = msg(f, "OpDef")                                  # op_def.proto (name only)
    field(opdef, "name", 1, FD.TYPE_STRING)
    fdef = msg(f, "FunctionDef")                             # function.proto
    field(fdef, "signature", 1, FD.TYPE_MESSAGE, type_name="OpDef")
    field(fdef, "node_def", 3, FD.TYPE_MESSAGE, R, "NodeDef")
    map_field(fdef, "ret", 4, FD.TYPE_STRING)
    map_field(fdef, "attr", 5, FD.TYPE_MESSAGE, "AttrValue")
    grad = msg(f, "GradientDef")
    field(grad, "function_name", 1, FD.TYPE_STRING)
    field(grad, "gradient_func", 2, FD.TYPE_STRING)
    flib = msg(f, "FunctionDefLibrary")
    field(flib, "function", 1, FD.TYPE_MESSAGE, R, "FunctionDef")
    field(flib, "gradient", 2, FD.TYPE_MESSAGE, R, "GradientDef")

    graph = msg(f, "GraphDef")                               # graph.proto
    field(graph, "node", 1, FD.TYPE_MESSAGE, R, "NodeDef")
    field(graph, "library", 2, FD.TYPE_MESSAGE, type_name="FunctionDefLibrary")
    field(graph, "version", 3, FD.TYPE_INT32)
    field(graph, "versions", 4, FD.TYPE_MESSAGE, type_name="VersionDef")

    pool = descriptor_pool.DescriptorPool()
    pool.Add(f)
    return {name: message_factory.GetMessageClass(pool.FindMessageTypeByName(package + "." + name))
            for name in ("GraphDef", "NodeDef", "AttrValue", "TensorProto", "TensorShapeProto")}


def _set_shape(tensor, shape):
    tensor.tensor_shape.SetInParent()  # a scalar still carries an (empty) tensor_shape, as TensorFlow writes it
    for d in shape:
        tensor.tensor_shape.dim.add(size=int(d))


def _const(graph, name, dtype, shape, content=None, float_val=None, half_val=None, int_val=None):
    """A Const node as freeze_graph writes it: attr dtype + attr value (in that or the other order)."""
    n = graph.node.add(name=name, op="Const")
    n.attr["dtype"].type = dtype
    t = n.attr["value"].tensor
    t.dtype = dtype
    _set_shape(t, shape)
    if content is not None:
        t.tensor_content = content
    if float_val is not None:
        t.float_val.extend(float(v) for v in float_val)
    if half_val is not None:
        t.half_val.extend(int(np.float16(v).view(np.uint16)) for v in half_val)
    if int_val is not None:
        t.int_val.extend(int(v) for v in int_val)
    return n


def build():
    from cubert_amd.testing import random_bert_weights
    weights = random_bert_weights(seed=21, labels=TINY_LABELS, ln_random=True, **TINY)
    expected = {}

    P = _messages("tensorflow", packed=True)
    g = P["GraphDef"]()
    g.versions.producer = 27
    g.versions.min_consumer = 12
    g.versions.bad_consumers.extend([3, 5])
    g.version = 27

    # inputs and ops around the weights
    for name, dt in (("input_ids", DT_INT32), ("input_mask", DT_INT32), ("segment_ids", DT_INT32)):
        n = g.node.add(name=name, op="Placeholder")
        n.attr["dtype"].type = dt
        n.attr["shape"].shape.dim.add(size=-1)
        n.attr["shape"].shape.dim.add(size=TINY_SEQ)
    n = g.node.add(name="bert/encoder/layer_0/attention/self/query/MatMul", op="MatMul",
                   input=["bert/encoder/Reshape_1", "bert/encoder/layer_0/attention/self/query/kernel/read"])
    n.attr["T"].type = DT_FLOAT
    n.attr["transpose_a"].b = False
    n.attr["transpose_b"].b = True
    n = g.node.add(name="bert/encoder/layer_0/intermediate/dense/LeakyRelu", op="LeakyRelu", device="/device:CPU:0")
    n.attr["alpha"].f = 0.2              # AttrValue.f: a fixed32 on the wire
    n.attr["T"].type = DT_FLOAT
    n = g.node.add(name="bert/embeddings/Slice/hints", op="NoOp")
    n.attr["_output_shapes"].list.shape.add().dim.add(size=TINY_SEQ)
    n.attr["_class"].list.s.append(b"loc:@bert/embeddings/position_embeddings")
    n.attr["value"].s = b"a string under the key the loader looks for"
    n = g.node.add(name="bert/embeddings/word_embeddings/read", op="Identity",
                   input=["bert/embeddings/word_embeddings"])
    n.attr["T"].type = DT_FLOAT
    n.attr["_class"].list.s.append(b"loc:@bert/embeddings/word_embeddings")

    # int32 constants: skipped by the loader
    _const(g, "bert/encoder/Reshape/shape", DT_INT32, [2], content=np.array([-1, 16], np.int32).tobytes())
    _const(g, "bert/encoder/strided_slice/stack", DT_INT32, [1], int_val=[0])
    _const(g, "bert/embeddings/ExpandDims/dim", DT_INT32, [], int_val=[-1])

    # the weights, tensor_content; one of them in half precision
    for name, array in weights.items():
        if name == "bert/pooler/dense/bias":
            half = array.astype(np.float16)
            _const(g, name, DT_HALF, half.shape, content=half.tobytes())
            expected[name] = half.astype(np.float32)
        else:
            _const(g, name, DT_FLOAT, array.shape, content=array.tobytes())
            expected[name] = array

    # scalars and splats the way make_tensor_proto writes them (packed)
    _const(g, "bert/embeddings/LayerNorm/batchnorm/add/y", DT_FLOAT, [], float_val=[1e-12])
    expected["bert/embeddings/LayerNorm/batchnorm/add/y"] = np.array([1e-12], np.float32)
    _const(g, "bert/encoder/layer_0/attention/self/Mul/y", DT_FLOAT, [], float_val=[0.35355338])
    expected["bert/encoder/layer_0/attention/self/Mul/y"] = np.array([0.35355338], np.float32)
    _const(g, "bert/encoder/mul_1/y_half", DT_HALF, [], half_val=[-10000.0])
    expected["bert/encoder/mul_1/y_half"] = np.array([-10000.0], np.float32)
    _const(g, "bert/encoder/ones_splat", DT_FLOAT, [5], float_val=[1.0])
    expected["bert/encoder/ones_splat"] = np.ones(5, np.float32)
    _const(g, "bert/encoder/partial_list", DT_FLOAT, [2, 3], float_val=[1.5, -2.5])   # last value repeats
    expected["bert/encoder/partial_list"] = np.array([1.5, -2.5, -2.5, -2.5, -2.5, -2.5], np.float32)
    _const(g, "bert/encoder/half_splat", DT_HALF, [3], half_val=[0.5])
    expected["bert/encoder/half_splat"] = np.full(3, 0.5, np.float32)
    _const(g, "loss/one_element_bias", DT_FLOAT, [1], float_val=[0.125])
    expected["loss/one_element_bias"] = np.array([0.125], np.float32)
    _const(g, "bert/encoder/empty", DT_FLOAT, [0])
    expected["bert/encoder/empty"] = np.zeros(0, np.float32)
    # an all-zero tensor after TensorFlow's tensor compression: a shape, no tensor_content and no value list
    _const(g, "bert/encoder/zeros_compressed", DT_FLOAT, [2, 3])
    expected["bert/encoder/zeros_compressed"] = np.zeros(6, np.float32)
    _const(g, "bert/encoder/zeros_compressed_half", DT_HALF, [4])
    expected["bert/encoder/zeros_compressed_half"] = np.zeros(4, np.float32)

    # a repeated name: the later node wins
    _const(g, "repeated/name", DT_FLOAT, [2], content=np.array([1, 2], np.float32).tobytes())
    _const(g, "repeated/name", DT_FLOAT, [3], content=np.array([7, 8, 9], np.float32).tobytes())
    expected["repeated/name"] = np.array([7, 8, 9], np.float32)

    # a function library holding a Const named like a weight: not a GraphDef.node
    fn = g.library.function.add()
    fn.signature.name = "cond_true_17"
    inner = fn.node_def.add(name="bert/embeddings/LayerNorm/beta", op="Const")
    inner.attr["dtype"].type = DT_FLOAT
    inner.attr["value"].tensor.dtype = DT_FLOAT
    _set_shape(inner.attr["value"].tensor, [TINY["hidden"]])
    inner.attr["value"].tensor.tensor_content = np.full(TINY["hidden"], 99.0, np.float32).tobytes()
    fn.ret["out"] = "bert/embeddings/LayerNorm/beta:output:0"
    g.library.gradient.add(function_name="cond_true_17", gradient_func="cond_true_17_grad")

    # the same kinds of scalar, unpacked: one tag per element
    U = _messages("tensorflow_unpacked", packed=False)
    u = U["GraphDef"]()
    _const(u, "bert/encoder/layer_0/output/LayerNorm/batchnorm/add/y", DT_FLOAT, [], float_val=[1e-12])
    expected["bert/encoder/layer_0/output/LayerNorm/batchnorm/add/y"] = np.array([1e-12], np.float32)
    _const(u, "bert/encoder/unpacked_list", DT_FLOAT, [4], float_val=[0.25, 0.5, 0.75, 1.0])
    expected["bert/encoder/unpacked_list"] = np.array([0.25, 0.5, 0.75, 1.0], np.float32)
    _const(u, "bert/encoder/unpacked_half", DT_HALF, [2], half_val=[-10000.0, 3.0])
    expected["bert/encoder/unpacked_half"] = np.array([-10000.0, 3.0], np.float32)
    _const(u, "bert/encoder/unpacked_int", DT_INT32, [2], int_val=[4, 5])

    # concatenated serialisations of one message type parse as their merge: node lists append
    data = g.SerializeToString() + u.SerializeToString()
    absent = ["input_ids", "bert/encoder/Reshape/shape", "bert/encoder/strided_slice/stack",
              "bert/embeddings/ExpandDims/dim", "bert/embeddings/Slice/hints", "bert/encoder/unpacked_int",
              "bert/encoder/layer_0/attention/self/query/MatMul", "bert/embeddings/word_embeddings/read"]
    return data, expected, absent


def main():
    data, expected, absent = build()
    with open(os.path.join(HERE, "tf_style_graphdef.pb"), "wb") as f:
        f.write(data)
    arrays = {"w%03d" % i: v for i, v in enumerate(expected.values())}
    np.savez_compressed(os.path.join(HERE, "tf_style_graphdef_expected.npz"),
                        names=np.array(list(expected.keys())), absent=np.array(absent), **arrays)
    print("wrote %d bytes, %d expected tensors" % (len(data), len(expected)))


if __name__ == "__main__":
    main()
