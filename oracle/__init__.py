"""ctypes access to the CPU oracle (oracle/liboracle.so) and, when it was built,
to the reference's own CPU op launchers (oracle/_ref/libref_ops.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg.  The shipped library never touches this package.
"""
import ctypes
import glob
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None

c_float_p = ctypes.POINTER(ctypes.c_float)


def build():
    """Compile liboracle.so (and _ref/libref_ops.so when the reference is mounted)."""
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def _fp(a):
    return a.ctypes.data_as(c_float_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        L.oracle_blas_name.restype = ctypes.c_char_p
        L.oracle_use_cblas.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
        L.oracle_half_bits_to_float.restype = ctypes.c_float
        L.oracle_half_bits_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_float_to_half_bits.restype = ctypes.c_uint16
        L.oracle_float_to_half_bits.argtypes = [ctypes.c_float]
        _LIB = L
        use_best_blas()
    return _LIB


def ref_ops():
    """The reference's CPU launchers, or None where they were not built."""
    global _REF
    if _REF is None:
        path = os.path.join(_HERE, "_ref", "libref_ops.so")
        if not os.path.exists(path):
            return None
        _REF = ctypes.CDLL(path)
    return _REF


def find_openblas():
    """Path of the OpenBLAS that ships inside the scipy wheel, or None."""
    try:
        import scipy
    except ImportError:
        return None
    root = os.path.join(os.path.dirname(os.path.dirname(scipy.__file__)), "scipy.libs")
    hits = sorted(glob.glob(os.path.join(root, "libscipy_openblas-*.so")))
    return hits[0] if hits else None


def use_best_blas():
    """OpenBLAS from scipy when present, else the oracle's own loop."""
    path = find_openblas()
    if path and lib_raw().oracle_use_cblas(path.encode(), b"scipy_cblas_sgemm") == 0:
        return blas_name()
    lib_raw().oracle_use_builtin_gemm()
    return blas_name()


def lib_raw():
    return _LIB if _LIB is not None else lib()


def use_builtin_gemm():
    lib().oracle_use_builtin_gemm()


def blas_name():
    return lib().oracle_blas_name().decode()


def set_blas_threads(n):
    """Thread count of the scipy OpenBLAS (no effect on the builtin loop, which follows OMP_NUM_THREADS)."""
    path = find_openblas()
    if not path:
        return False
    ob = ctypes.CDLL(path)
    try:
        ob.scipy_openblas_set_num_threads(int(n))
    except AttributeError:
        return False
    return True


def set_batch_parallel(on):
    """Batched attention GEMMs as an OpenMP loop around single-threaded BLAS calls (default) or one multi-threaded
    call per problem."""
    lib().oracle_set_batch_parallel(int(bool(on)))


PROFILE_PARTS = ("dense_gemm", "attention_batch_gemm", "row_kernels", "other")


def profile_reset():
    lib().oracle_profile_reset()


def profile_read():
    """Seconds per part of the forward passes since the last reset."""
    out = (ctypes.c_double * len(PROFILE_PARTS))()
    lib().oracle_profile_read(out)
    return dict(zip(PROFILE_PARTS, (float(v) for v in out)))


def threads_in_use():
    """What the host and the libraries report about themselves: logical CPUs, CPUs this process may run on, the
    OpenMP team size of the oracle's loops and the thread count of the loaded BLAS."""
    info = {"nproc": os.cpu_count(), "OMP_NUM_THREADS": os.environ.get("OMP_NUM_THREADS"),
            "blas_threads": int(lib().oracle_blas_threads())}
    try:
        info["sched_affinity"] = len(os.sched_getaffinity(0))
    except AttributeError:
        info["sched_affinity"] = None
    try:
        with open("/sys/fs/cgroup/cpu.max") as f:  # "<quota> <period>" in microseconds, or "max <period>"
            quota, period = f.read().split()[:2]
        info["cgroup_cpu_share"] = None if quota == "max" else round(int(quota) / int(period), 2)
    except (OSError, ValueError):
        info["cgroup_cpu_share"] = None
    try:
        info["omp_max_threads"] = int(ctypes.CDLL("libgomp.so.1").omp_get_max_threads())
    except OSError:
        info["omp_max_threads"] = None
    return info


class Vars(object):
    """Named fp32 weights in the form the C oracle takes them (names + pointers)."""

    def __init__(self, weights):
        self.keep = {k: _f32(v) for k, v in weights.items()}
        names = list(self.keep.keys())
        self._names = (ctypes.c_char_p * len(names))(*[n.encode() for n in names])
        self._ptrs = (c_float_p * len(names))(*[_fp(self.keep[n]) for n in names])

        class S(ctypes.Structure):
            _fields_ = [("n", ctypes.c_int), ("names", ctypes.POINTER(ctypes.c_char_p)),
                        ("data", ctypes.POINTER(c_float_p))]

        self.struct = S(len(names), self._names, self._ptrs)

    def ref(self):
        return ctypes.byref(self.struct)


# ----------------------------------------------------------------- primitives

def _pick(use_ref):
    if use_ref:
        r = ref_ops()
        if r is None:
            raise RuntimeError("oracle/_ref/libref_ops.so was not built")
        return r, "ref_"
    return lib(), "oracle_"


def embedding(ids, table, use_ref=False):
    L, p = _pick(use_ref)
    table = _f32(table)
    width = table.shape[1]
    if np.asarray(ids).dtype == np.int8:
        ids = np.ascontiguousarray(ids, dtype=np.int8)
        fn, ptr = getattr(L, p + "embedding_i8"), ids.ctypes.data_as(ctypes.POINTER(ctypes.c_int8))
    else:
        ids = np.ascontiguousarray(ids, dtype=np.int32)
        fn, ptr = getattr(L, p + "embedding"), ids.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
    out = np.empty((ids.size, width), np.float32)
    fn(ptr, ctypes.c_int(ids.size), _fp(table), ctypes.c_int(width), _fp(out))
    return out


def layer_norm_(inp, inout, beta, gamma, use_ref=False):
    """Returns LN(inout + inp); inputs are [rows, C]."""
    L, p = _pick(use_ref)
    inp, out = _f32(inp), _f32(inout).copy()
    rows, C = out.shape
    beta, gamma = _f32(beta), _f32(gamma)
    getattr(L, p + "layer_norm_")(_fp(inp), _fp(out), ctypes.c_int(rows), ctypes.c_int(C), _fp(beta), _fp(gamma))
    return out


def softmax_(x, use_ref=False):
    L, p = _pick(use_ref)
    x = _f32(x).copy()
    rows, C = x.shape
    out = np.empty_like(x)
    getattr(L, p + "softmax_")(_fp(x), _fp(out), ctypes.c_int(rows), ctypes.c_int(C))
    return out


def gelu(x, use_ref=False):
    L, p = _pick(use_ref)
    out = _f32(x).copy()
    getattr(L, p + "gelu")(ctypes.c_size_t(out.size), _fp(out))
    return out


def not_(mask, use_ref=False):
    L, p = _pick(use_ref)
    mask = np.ascontiguousarray(mask, dtype=np.int8)
    out = np.empty(mask.shape, np.float32)
    getattr(L, p + "not")(mask.ctypes.data_as(ctypes.POINTER(ctypes.c_int8)), _fp(out), ctypes.c_int(mask.size))
    return out


def tanh_(x, use_ref=False):
    L, p = _pick(use_ref)
    out = _f32(x).copy()
    getattr(L, p + "tanh_")(_fp(out), ctypes.c_int(out.size))
    return out


def reduce_mean_1(x, use_ref=False):
    L, p = _pick(use_ref)
    x = _f32(x)
    B, S, H = x.shape
    out = np.empty((B, H), np.float32)
    getattr(L, p + "reduce_mean_1")(_fp(x), _fp(out), ctypes.c_int(B), ctypes.c_int(S), ctypes.c_int(H))
    return out


# ----------------------------------------------------------------- composites

def sgemm(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc):
    """Column-major sgemm on flat fp32 arrays; C is updated in place."""
    lib().oracle_sgemm(int(transA), int(transB), M, N, K, ctypes.c_float(alpha), _fp(A), lda, _fp(B), ldb,
                       ctypes.c_float(beta), _fp(C), ldc)
    return C


def dense(x, kernel, bias):
    x, kernel, bias = _f32(x), _f32(kernel), _f32(bias)
    rows, inputs = x.shape
    units = kernel.shape[1]
    out = np.empty((rows, units), np.float32)
    lib().oracle_dense(rows, inputs, units, _fp(kernel), _fp(bias), _fp(x), _fp(out))
    return out


def attention_mask(mask, heads):
    mask = np.ascontiguousarray(mask, dtype=np.int8)
    B, S = mask.shape
    out = np.empty((B, heads * S, S), np.float32)
    lib().oracle_attention_mask(B, S, heads, mask.ctypes.data_as(ctypes.POINTER(ctypes.c_int8)), _fp(out))
    return out


def att_q_k(query, key, batch, S, A, d, alpha=1.0, beta=0.0, scores=None):
    query, key = _f32(query), _f32(key)
    out = np.zeros((batch, S, A, S), np.float32) if scores is None else _f32(scores).copy()
    lib().oracle_att_q_k(batch, S, A, d, _fp(query), _fp(key), _fp(out), ctypes.c_float(alpha), ctypes.c_float(beta))
    return out


def att_qk_v(qk, value, batch, S, A, d, alpha=1.0, beta=0.0):
    qk, value = _f32(qk), _f32(value)
    out = np.zeros((batch, S, A, d), np.float32)
    lib().oracle_att_qk_v(batch, S, A, d, _fp(qk), _fp(value), _fp(out), ctypes.c_float(alpha), ctypes.c_float(beta))
    return out


def attention_self(weights, prefix, x, neg_mask, batch, S, A, d):
    v = Vars(weights)
    x, neg_mask = _f32(x), _f32(neg_mask)
    out = np.empty((batch * S, A * d), np.float32)
    rc = lib().oracle_attention_self(v.ref(), prefix.encode(), batch, S, A, d, _fp(x), _fp(neg_mask), _fp(out))
    if rc:
        raise KeyError("missing weight under " + prefix)
    return out


def transformer(weights, prefix, x, mask, batch, S, H, layers, heads, intermediate):
    v = Vars(weights)
    x = _f32(x)
    mask = np.ascontiguousarray(mask, dtype=np.int8)
    out = np.empty((batch * S, H), np.float32)
    rc = lib().oracle_transformer(v.ref(), prefix.encode(), batch, S, H, layers, heads, intermediate, _fp(x),
                                  mask.ctypes.data_as(ctypes.POINTER(ctypes.c_int8)), _fp(out))
    if rc:
        raise KeyError("missing weight under " + prefix)
    return out


def bert_embeddings(weights, ids, segments, batch, S, H):
    v = Vars(weights)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    segments = np.ascontiguousarray(segments, dtype=np.int8)
    out = np.empty((batch * S, H), np.float32)
    rc = lib().oracle_bert_embeddings(v.ref(), batch, S, H, ids.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)),
                                      segments.ctypes.data_as(ctypes.POINTER(ctypes.c_int8)), _fp(out))
    if rc:
        raise KeyError("missing embedding weight")
    return out


def bert_pooler(kernel, bias, x):
    x, kernel, bias = _f32(x), _f32(kernel), _f32(bias)
    B, S, H = x.shape
    out = np.empty((B, H), np.float32)
    lib().oracle_bert_pooler(B, S, H, _fp(kernel), _fp(bias), _fp(x), _fp(out))
    return out


def mean_pooler(x):
    x = _f32(x)
    B, S, H = x.shape
    out = np.empty((B, H), np.float32)
    lib().oracle_mean_pooler(B, S, H, _fp(x), _fp(out))
    return out


def classifier(weights, bias, x, want_probs=True):
    x, weights = _f32(x), _f32(weights)
    B, H = x.shape
    labels = weights.shape[0]
    logits = np.empty((B, labels), np.float32)
    probs = np.empty((B, labels), np.float32) if want_probs else None
    b = _f32(bias) if bias is not None else None
    lib().oracle_classifier(B, H, labels, _fp(weights), _fp(b) if b is not None else None, _fp(x), _fp(logits),
                            _fp(probs) if probs is not None else None)
    return logits, probs


def bert_forward(weights, ids, mask, segments, layers, heads, vars_obj=None):
    """Full forward pass.  Shapes are inferred from the weights the way the
    reference's graph loader does (tensorflow/Graph.cpp:68-78).  Returns a dict
    with embedding_output, sequence_output, pooled_output and, when the model
    has a classifier, logits and probs."""
    v = vars_obj or Vars(weights)
    w = v.keep
    H = w["bert/embeddings/word_embeddings"].shape[1]
    I = w["bert/encoder/layer_0/intermediate/dense/bias"].shape[0]
    has_cls = "output_weights" in w
    labels = w["output_weights"].shape[0] if has_cls else 1
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    mask = np.ascontiguousarray(mask, dtype=np.int8)
    segments = np.ascontiguousarray(segments, dtype=np.int8)
    B, S = ids.shape
    out = {
        "embedding_output": np.empty((B, S, H), np.float32),
        "sequence_output": np.empty((B, S, H), np.float32),
        "pooled_output": np.empty((B, H), np.float32),
    }
    if has_cls:
        out["logits"] = np.empty((B, labels), np.float32)
        out["probs"] = np.empty((B, labels), np.float32)
    i8p = ctypes.POINTER(ctypes.c_int8)
    rc = lib().oracle_bert_forward(
        v.ref(), B, S, H, layers, heads, I, labels, ids.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)),
        mask.ctypes.data_as(i8p), segments.ctypes.data_as(i8p), _fp(out["embedding_output"]),
        _fp(out["sequence_output"]), _fp(out["pooled_output"]),
        _fp(out["logits"]) if has_cls else None, _fp(out["probs"]) if has_cls else None)
    if rc:
        raise KeyError("missing weight")
    return out


def round_to_half(x):
    x = _f32(x)
    out = np.empty_like(x)
    lib().oracle_round_to_half(_fp(x), _fp(out), ctypes.c_size_t(x.size))
    return out
