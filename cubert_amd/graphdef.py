"""Writes (and reads back) the frozen TensorFlow GraphDef files cuBERT_open loads.

Only what the loader looks at is produced: one `Const` NodeDef per weight with
attr "dtype" and attr "value" = TensorProto{dtype, tensor_shape, tensor_content}
(field numbers from tensorflow/core/framework/{graph,node_def,attr_value,tensor,
tensor_shape,types}.proto).  This lets a random-init model go through the real
`cuBERT_open(model_file, ...)` path without TensorFlow.
"""
import numpy as np

DT_FLOAT = 1
DT_HALF = 19


def _varint(n):
    out = bytearray()
    n &= (1 << 64) - 1
    while True:
        b = n & 0x7F
        n >>= 7
        if n:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _field(number, wire, payload):
    return _varint((number << 3) | wire) + payload


def _bytes_field(number, data):
    return _field(number, 2, _varint(len(data)) + data)


def _tensor_proto(array):
    array = np.require(array, requirements="C")  # keeps 0-d arrays 0-d
    if array.dtype == np.float32:
        dtype = DT_FLOAT
    elif array.dtype == np.float16:
        dtype = DT_HALF
    else:
        raise TypeError("float32 or float16 expected")
    shape = b"".join(_bytes_field(2, _field(1, 0, _varint(d))) for d in array.shape)
    return (_field(1, 0, _varint(dtype)) + _bytes_field(2, shape) + _bytes_field(4, array.tobytes())), dtype


def _node(name, array):
    tensor, dtype = _tensor_proto(array)
    attr_dtype = _bytes_field(1, b"dtype") + _bytes_field(2, _field(6, 0, _varint(dtype)))
    attr_value = _bytes_field(1, b"value") + _bytes_field(2, _bytes_field(8, tensor))
    return (_bytes_field(1, name.encode()) + _bytes_field(2, b"Const") + _bytes_field(5, attr_dtype)
            + _bytes_field(5, attr_value))


def write_graphdef(path, weights):
    """weights: {variable name: float32/float16 ndarray}."""
    with open(path, "wb") as f:
        for name, array in weights.items():
            f.write(_bytes_field(1, _node(name, array)))
        f.write(_bytes_field(4, _field(1, 0, _varint(27))))  # versions { producer: 27 }
    return path


# ---- reader (used to check the writer; the library has its own in C++) ----

def _read_varint(buf, pos):
    shift = 0
    value = 0
    while True:
        b = buf[pos]
        pos += 1
        value |= (b & 0x7F) << shift
        if not b & 0x80:
            return value, pos
        shift += 7


def _fields(buf):
    pos = 0
    end = len(buf)
    while pos < end:
        tag, pos = _read_varint(buf, pos)
        number, wire = tag >> 3, tag & 7
        if wire == 0:
            value, pos = _read_varint(buf, pos)
        elif wire == 2:
            n, pos = _read_varint(buf, pos)
            value = buf[pos:pos + n]
            pos += n
        elif wire == 1:
            value = buf[pos:pos + 8]
            pos += 8
        elif wire == 5:
            value = buf[pos:pos + 4]
            pos += 4
        else:
            raise ValueError("unsupported wire type %d" % wire)
        yield number, wire, value


def read_graphdef(path):
    with open(path, "rb") as f:
        buf = memoryview(f.read())
    out = {}
    for number, wire, node in _fields(buf):
        if number != 1 or wire != 2:
            continue
        name, tensor = None, None
        for nf, nw, nv in _fields(node):
            if nf == 1:
                name = bytes(nv).decode()
            elif nf == 5:
                key, val = None, None
                for ef, ew, ev in _fields(nv):
                    if ef == 1:
                        key = bytes(ev)
                    elif ef == 2:
                        val = ev
                if key == b"value" and val is not None:
                    for af, aw, av in _fields(val):
                        if af == 8:
                            tensor = av
        if tensor is None:
            continue
        dtype, dims, content = None, [], b""
        for tf_, tw, tv in _fields(tensor):
            if tf_ == 1:
                dtype = tv
            elif tf_ == 2:
                for sf, sw, sv in _fields(tv):
                    if sf == 2:
                        size = 0
                        for df, dw, dv in _fields(sv):
                            if df == 1:
                                size = dv
                        dims.append(size)
            elif tf_ == 4:
                content = tv
        np_dtype = {DT_FLOAT: np.float32, DT_HALF: np.float16}.get(dtype)
        if np_dtype is None:
            continue
        out[name] = np.frombuffer(bytes(content), dtype=np_dtype).reshape(dims)
    return out
