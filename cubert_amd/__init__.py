"""Host-side Python interface of the library, mirroring the reference's Python
binding (python/cuBERT.pyx: get_gpu_count, ComputeType, OutputType, Output,
Model.compute / compute_m) on top of the C ABI of include/cuBERT.h, plus `Bert`,
the reference's C++ host class of the same name, constructed from named weights.

Argument errors raise the exceptions Cython's `except +` would produce from the
reference's C++ exceptions: std::invalid_argument -> ValueError,
std::out_of_range -> IndexError.  Device errors terminate the process, as in the
reference.
"""
import ctypes
import os

import numpy as np

from ._lib import cuBERT_Output, lib

__all__ = ["get_gpu_count", "ComputeType", "OutputType", "Output", "Model", "Bert"]


class ComputeType(object):
    FLOAT = 0
    HALF = 1


class OutputType(object):
    LOGITS = 0
    POOLED_OUTPUT = 1
    SEQUENCE_OUTPUT = 2
    EMBEDDING_OUTPUT = 3
    PROBS = 4


_FIELDS = {OutputType.LOGITS: "logits", OutputType.POOLED_OUTPUT: "pooled_output",
           OutputType.SEQUENCE_OUTPUT: "sequence_output", OutputType.EMBEDDING_OUTPUT: "embedding_output",
           OutputType.PROBS: "probs"}


def get_gpu_count():
    return lib().cuBERT_get_gpu_count()


def _raise(rc):
    if rc == 0:
        return
    msg = lib().cubert_last_error().decode()
    if rc == 1:
        raise ValueError(msg)
    if rc == 2:
        raise IndexError(msg)
    raise RuntimeError(msg)


class Output(object):
    """Any subset of the five outputs; assign numpy arrays to the fields wanted."""

    def __init__(self, output=None, output_type=OutputType.LOGITS):
        self._c = cuBERT_Output()
        self._keep = {}
        if output is not None:
            setattr(self, _FIELDS[output_type], output)

    def _set(self, name, value):
        if not isinstance(value, np.ndarray) or not value.flags["C_CONTIGUOUS"]:
            raise ValueError("numpy array should be C_CONTIGUOUS")
        self._keep[name] = value
        setattr(self._c, name, value.ctypes.data)

    logits = property(lambda s: s._keep.get("logits"), lambda s, v: s._set("logits", v))
    pooled_output = property(lambda s: s._keep.get("pooled_output"), lambda s, v: s._set("pooled_output", v))
    sequence_output = property(lambda s: s._keep.get("sequence_output"), lambda s, v: s._set("sequence_output", v))
    embedding_output = property(lambda s: s._keep.get("embedding_output"), lambda s, v: s._set("embedding_output", v))
    probs = property(lambda s: s._keep.get("probs"), lambda s, v: s._set("probs", v))


def _check_inputs(input_ids, input_mask, segment_ids):
    for a, dt in ((input_ids, np.int32), (input_mask, np.int8), (segment_ids, np.int8)):
        if not isinstance(a, np.ndarray) or a.dtype != dt or a.ndim != 2:
            raise TypeError("inputs must be 2-d numpy arrays: int32 ids, int8 mask, int8 segment ids")
        if not a.flags["C_CONTIGUOUS"]:
            raise ValueError("numpy array should be C_CONTIGUOUS")
    if input_ids.shape[0] != input_mask.shape[0] or input_ids.shape[0] != segment_ids.shape[0]:
        raise ValueError("numpy shape mismatch")
    return input_ids.shape[0]


def _text_array(texts):
    """list of str/bytes -> (const char*[]) with the bytes objects kept alive by the returned pair."""
    if texts is None:
        return None, None
    keep = [t.encode("utf8") if isinstance(t, str) else bytes(t) for t in texts]
    return (ctypes.c_char_p * len(keep))(*keep), keep


class Tokenizer(object):
    """The text front end alone (CPU): the reference's FullTokenizer (src/cuBERT/tokenization.h:112-152), or with
    vocab_file=None its BasicTokenizer."""

    def __init__(self, vocab_file=None, do_lower_case=True):
        self._h = None
        self.do_lower_case = bool(do_lower_case)
        if vocab_file is not None:
            handle = ctypes.c_void_p()
            _raise(lib().cubert_try_open_tokenizer(os.fsencode(vocab_file), int(self.do_lower_case),
                                                   ctypes.byref(handle)))
            self._h = handle

    def close(self):
        if self._h is not None:
            lib().cuBERT_close_tokenizer(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _tokens(call):
        n, needed = ctypes.c_int(), ctypes.c_size_t()
        _raise(call(None, 0, ctypes.byref(n), ctypes.byref(needed)))
        buf = ctypes.create_string_buffer(needed.value)
        _raise(call(buf, needed.value, ctypes.byref(n), ctypes.byref(needed)))
        return buf.value.decode("utf8").split("\n") if n.value else []

    def tokenize(self, text, max_length=1 << 20):
        """Word pieces of `text` (basic tokens when there is no vocabulary)."""
        raw = text.encode("utf8") if isinstance(text, str) else bytes(text)
        return self._tokens(lambda out, cap, n, needed: lib().cubert_tokenizer_tokenize(
            self._h, int(self.do_lower_case), raw, max_length, out, cap, n, needed))

    def wordpiece(self, token):
        raw = token.encode("utf8") if isinstance(token, str) else bytes(token)
        return self._tokens(lambda out, cap, n, needed: lib().cubert_tokenizer_wordpiece(self._h, raw, out, cap, n,
                                                                                          needed))

    def convert_tokens_to_ids(self, tokens):
        return [int(lib().cubert_tokenizer_token_id(self._h, t.encode("utf8"))) for t in tokens]

    def convert_example(self, max_seq_length, text_a, text_b=None):
        """(input_ids int32, input_mask int8, segment_ids int8), each of max_seq_length entries."""
        ids = np.zeros(max_seq_length, np.int32)
        mask = np.zeros(max_seq_length, np.int8)
        seg = np.zeros(max_seq_length, np.int8)
        _raise(lib().cubert_tokenizer_convert_example(
            self._h, max_seq_length, text_a.encode("utf8"), None if text_b is None else text_b.encode("utf8"),
            ids.ctypes.data, mask.ctypes.data, seg.ctypes.data))
        return ids, mask, seg


def nfd(text):
    """Canonical decomposition of a string by the library's own tables."""
    raw = text.encode("utf8")
    needed = ctypes.c_size_t()
    _raise(lib().cubert_tokenizer_nfd(raw, None, 0, ctypes.byref(needed)))
    buf = ctypes.create_string_buffer(needed.value)
    _raise(lib().cubert_tokenizer_nfd(raw, buf, needed.value, ctypes.byref(needed)))
    return buf.value.decode("utf8")


class Graph(object):
    """The float / binary16 constants of a frozen GraphDef file as the library's loader sees them (the C++ class
    Graph<T>, reference src/cuBERT/tensorflow/Graph.h:10-23).  CPU only."""

    def __init__(self, model_file, compute_type=ComputeType.FLOAT):
        self._h = None
        self.compute_type = compute_type
        handle = ctypes.c_void_p()
        _raise(lib().cubert_graph_open(os.fsencode(model_file), compute_type, ctypes.byref(handle)))
        self._h = handle
        sizes = (ctypes.c_size_t * 5)()
        _raise(lib().cubert_graph_sizes(handle, compute_type, sizes))
        (self.vocab_size, self.type_vocab_size, self.hidden_size, self.intermediate_size,
         self.num_labels) = (int(v) for v in sizes)

    def __len__(self):
        return int(lib().cubert_graph_count(self._h, self.compute_type))

    def var(self, name):
        """A copy of var[name] (flat) and its declared shape, or None for a name the graph does not hold."""
        n = ctypes.c_size_t()
        dims = (ctypes.c_longlong * 8)()
        rank = ctypes.c_int()
        ptr = lib().cubert_graph_var(self._h, self.compute_type, name.encode(), ctypes.byref(n), dims, 8,
                                     ctypes.byref(rank))
        if not ptr:
            return None
        dtype = np.float32 if self.compute_type == ComputeType.FLOAT else np.float16
        data = np.empty(n.value, dtype)
        if n.value:
            ctypes.memmove(data.ctypes.data, ptr, data.nbytes)
        return data, tuple(int(d) for d in dims[:min(rank.value, 8)])

    def close(self):
        if self._h is not None:
            _raise(lib().cubert_graph_close(self._h, self.compute_type))
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Model(object):
    """A model opened from a frozen GraphDef file (cuBERT_open), one replica per visible GPU; with a vocabulary
    file also the tokenizer (cuBERT_open_tokenizer), as python/cuBERT.pyx:116-139 of the reference."""

    def __init__(self, model_file, max_batch_size, seq_length, num_hidden_layers, num_attention_heads,
                 compute_type=ComputeType.FLOAT, vocab_file=None, do_lower_case=1):
        self._c_model = None
        self._c_tokenizer = None
        self._c_compute_type = compute_type
        if vocab_file:
            handle = ctypes.c_void_p()
            _raise(lib().cubert_try_open_tokenizer(os.fsencode(vocab_file), int(do_lower_case), ctypes.byref(handle)))
            self._c_tokenizer = handle
        if isinstance(model_file, str):
            model_file = model_file.encode("utf8")
        handle = ctypes.c_void_p()
        _raise(lib().cubert_try_open(model_file, max_batch_size, seq_length, num_hidden_layers, num_attention_heads,
                                     compute_type, ctypes.byref(handle)))
        self._c_model = handle
        h, l, s = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _raise(lib().cubert_model_info(handle, compute_type, ctypes.byref(h), ctypes.byref(l), ctypes.byref(s)))
        self.hidden_size, self.num_labels, self.seq_length = h.value, l.value, s.value

    def close(self):
        if self._c_model is not None:
            _raise(lib().cubert_try_close(self._c_model, self._c_compute_type))
            self._c_model = None
        if self._c_tokenizer is not None:
            lib().cuBERT_close_tokenizer(self._c_tokenizer)
            self._c_tokenizer = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def dtype(self):
        return np.float32 if self._c_compute_type == ComputeType.FLOAT else np.float16

    def compute(self, input_ids, input_mask, segment_ids, output, output_type=OutputType.LOGITS):
        batch = _check_inputs(input_ids, input_mask, segment_ids)
        if not isinstance(output, np.ndarray) or not output.flags["C_CONTIGUOUS"]:
            raise ValueError("numpy array should be C_CONTIGUOUS")
        _raise(lib().cubert_try_compute(self._c_model, batch, input_ids.ctypes.data, input_mask.ctypes.data,
                                        segment_ids.ctypes.data, output.ctypes.data, output_type, self._c_compute_type))

    def compute_m(self, input_ids, input_mask, segment_ids, output, output_to_float=False):
        batch = _check_inputs(input_ids, input_mask, segment_ids)
        _raise(lib().cubert_try_compute_m(self._c_model, batch, input_ids.ctypes.data, input_mask.ctypes.data,
                                          segment_ids.ctypes.data, ctypes.byref(output._c), self._c_compute_type,
                                          int(bool(output_to_float))))


    def tokenize_compute(self, text_a, text_b, output, output_type=OutputType.LOGITS):
        """Texts in, one output array out (python/cuBERT.pyx:181-189)."""
        if self._c_tokenizer is None:
            raise ValueError("the model was opened without a vocab_file")
        if text_b is not None and len(text_a) != len(text_b):
            raise ValueError("text_a and text_b differ in length")
        if not isinstance(output, np.ndarray) or not output.flags["C_CONTIGUOUS"]:
            raise ValueError("numpy array should be C_CONTIGUOUS")
        a, keep_a = _text_array(text_a)
        b, keep_b = _text_array(text_b)
        _raise(lib().cubert_try_tokenize_compute(self._c_model, self._c_tokenizer, len(keep_a), a, b,
                                                 output.ctypes.data, output_type, self._c_compute_type))

    def tokenize_compute_m(self, text_a, text_b, output, output_to_float=False):
        """Texts in, several outputs out (python/cuBERT.pyx:191-208)."""
        if self._c_tokenizer is None:
            raise ValueError("the model was opened without a vocab_file")
        if text_b is not None and len(text_a) != len(text_b):
            raise ValueError("text_a and text_b differ in length")
        a, keep_a = _text_array(text_a)
        b, keep_b = _text_array(text_b)
        _raise(lib().cubert_try_tokenize_compute_m(self._c_model, self._c_tokenizer, len(keep_a), a, b,
                                                   ctypes.byref(output._c), self._c_compute_type,
                                                   int(bool(output_to_float))))


class Bert(object):
    """One model on the current GPU built from named numpy weights: the reference's
    C++ class cuBERT::Bert<T> (Bert.h:17-44), whose constructor takes the same
    name -> array map.  Shapes come from the arrays as the reference's graph
    loader infers them (tensorflow/Graph.cpp:68-78)."""

    def __init__(self, weights, max_batch_size, seq_length, num_hidden_layers, num_attention_heads,
                 compute_type=ComputeType.FLOAT):
        self._h = None
        self.compute_type = compute_type
        dt = np.float32 if compute_type == ComputeType.FLOAT else np.float16
        self.dtype = dt
        # arrays of the other type are converted here (float -> half rounds to nearest even)
        keep = {k: np.ascontiguousarray(v, dtype=dt) for k, v in weights.items()}
        word = keep["bert/embeddings/word_embeddings"]
        self.vocab_size, self.hidden_size = word.shape
        self.type_vocab_size = keep["bert/embeddings/token_type_embeddings"].shape[0]
        self.intermediate_size = keep["bert/encoder/layer_0/intermediate/dense/bias"].shape[0] \
            if "bert/encoder/layer_0/intermediate/dense/bias" in keep else 4 * self.hidden_size
        self.num_labels = keep["output_weights"].shape[0] if "output_weights" in keep else 1
        self.has_classifier = "output_weights" in keep
        self.max_batch_size, self.seq_length = max_batch_size, seq_length
        names = list(keep.keys())
        c_names = (ctypes.c_char_p * len(names))(*[n.encode() for n in names])
        c_data = (ctypes.c_void_p * len(names))(*[keep[n].ctypes.data for n in names])
        handle = ctypes.c_void_p()
        _raise(lib().cubert_bert_create(compute_type, len(names), c_names, c_data, max_batch_size, seq_length,
                                        self.vocab_size, self.type_vocab_size, self.hidden_size, num_hidden_layers,
                                        num_attention_heads, self.intermediate_size, self.num_labels,
                                        ctypes.byref(handle)))
        self._h = handle

    def close(self):
        if self._h is not None:
            _raise(lib().cubert_bert_destroy(self._h, self.compute_type))
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def stream(self):
        return lib().cubert_bert_stream(self._h, self.compute_type)

    def compute(self, input_ids, input_mask, segment_ids):
        """Enqueue one forward pass (asynchronous; `output` waits for it)."""
        batch = _check_inputs(input_ids, input_mask, segment_ids)
        _raise(lib().cubert_bert_compute(self._h, self.compute_type, batch, input_ids.ctypes.data,
                                         input_mask.ctypes.data, segment_ids.ctypes.data))
        return batch

    def compute_resident(self, batch):
        """The forward pass again on the inputs the last compute() left on the device (asynchronous)."""
        _raise(lib().cubert_bert_compute_resident(self._h, self.compute_type, batch))

    def synchronize(self):
        rc = lib().cubert_stream_synchronize(self.stream)
        if rc:
            raise RuntimeError("stream synchronize failed: %d" % rc)

    KINDS = ("embed_ln", "bias_res_ln", "bias_gelu", "mask_scale_softmax", "bias_tanh", "mean_pool", "row_softmax",
             "dense_gemm", "attention_gemm", "attention_fused", "classifier_head", "dense_split",
             "dense_qkv", "dense_attention_output", "dense_intermediate", "dense_output", "dense_pooler")
    # a Dense launch is timed under its own kind when that kind is on and under "dense_gemm" otherwise
    DENSE_KINDS = ("dense_qkv", "dense_attention_output", "dense_intermediate", "dense_output", "dense_pooler")

    def profile(self, kinds):
        """Switch per-kernel event timing on for the named kinds (empty = off)."""
        mask = 0
        for k in kinds:
            mask |= 1 << self.KINDS.index(k)
        _raise(lib().cubert_bert_profile(self._h, self.compute_type, mask))

    def profile_read(self):
        """{kind: (total milliseconds, launches)} since the last read; synchronises the stream."""
        n = len(self.KINDS)
        ms = (ctypes.c_double * n)()
        cnt = (ctypes.c_int * n)()
        _raise(lib().cubert_bert_profile_read(self._h, self.compute_type, ms, cnt, n))
        return {k: (ms[i], cnt[i]) for i, k in enumerate(self.KINDS) if cnt[i]}

    def output(self, batch, output, output_to_float=False):
        _raise(lib().cubert_bert_output(self._h, self.compute_type, batch, ctypes.byref(output._c),
                                        int(bool(output_to_float))))

    def forward(self, input_ids, input_mask, segment_ids, to_float=True):
        """compute + all outputs as a dict of numpy arrays (float32 when to_float)."""
        batch = self.compute(input_ids, input_mask, segment_ids)
        dt = np.float32 if (to_float or self.compute_type == ComputeType.FLOAT) else np.float16
        S, H = self.seq_length, self.hidden_size
        o = Output()
        o.embedding_output = np.empty((batch, S, H), dt)
        o.sequence_output = np.empty((batch, S, H), dt)
        o.pooled_output = np.empty((batch, H), dt)
        if self.has_classifier:
            o.logits = np.empty((batch, self.num_labels), dt)
            o.probs = np.empty((batch, self.num_labels), dt)
        self.output(batch, o, output_to_float=to_float)
        return dict(o._keep)


def transformer_run(weights, prefix, x, mask, num_hidden_layers, num_attention_heads, intermediate_size,
                    compute_type=ComputeType.FLOAT):
    """The encoder stack alone (the reference's Transformer<T>::compute) on host arrays."""
    dt = np.float32 if compute_type == ComputeType.FLOAT else np.float16
    keep = {k: np.ascontiguousarray(v, dtype=dt) for k, v in weights.items()}
    x = np.ascontiguousarray(x, dtype=dt)
    mask = np.ascontiguousarray(mask, dtype=np.int8)
    batch, seq, hidden = x.shape
    names = list(keep.keys())
    c_names = (ctypes.c_char_p * len(names))(*[n.encode() for n in names])
    c_data = (ctypes.c_void_p * len(names))(*[keep[n].ctypes.data for n in names])
    out = np.empty_like(x)
    _raise(lib().cubert_transformer_run(compute_type, prefix.encode(), len(names), c_names, c_data, batch, seq, hidden,
                                        num_hidden_layers, num_attention_heads, intermediate_size, x.ctypes.data,
                                        mask.ctypes.data, out.ctypes.data))
    return out
