"""The reference's own benchmark client (benchmark/benchmark_cu.cpp), compiled unmodified against the
reference's own cuBERT.h and linked with this repository's libcuBERT.so (oracle/Makefile -> oracle/_ref/
benchmark_cu), run on a BERT-base GraphDef file written here: the drop-in check of the public C ABI.

The client draws its inputs from std::default_random_engine(0) with std::uniform_int_distribution; both are
replayed here (libstdc++'s algorithms, stated below) so that what the client wrote to cuBERT.txt can be checked
against the CPU oracle on the same inputs.

The reference's Cython extension is built the same way, as a link check in the build container only."""
import glob
import os
import re
import subprocess

import numpy as np
import pytest

import oracle
from util import assert_close

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLIENT = os.path.join(ROOT, "oracle", "_ref", "benchmark_cu")
PY_EXTENSION = glob.glob(os.path.join(ROOT, "oracle", "_ref", "cuBERT.*.so"))

BATCH, SEQ, HIDDEN, CALLS = 128, 32, 768, 20  # constants of the client (benchmark_cu.cpp:15-18,66-77)


class MinstdRand0(object):
    """std::default_random_engine of libstdc++: x <- 16807 x mod (2^31 - 1); seed 0 is taken as 1."""

    def __init__(self, seed):
        self.x = seed % 2147483647 or 1

    def __call__(self):
        self.x = self.x * 16807 % 2147483647
        return self.x


def uniform_int(engine, a, b):
    """libstdc++ std::uniform_int_distribution<int>(a, b) on an engine with range [1, 2^31 - 2]: scale down by
    integer division, rejecting the incomplete last bucket."""
    urng_range = 2147483646 - 1
    buckets = b - a + 1
    scaling = urng_range // buckets
    past = buckets * scaling
    while True:
        r = engine() - 1
        if r < past:
            return a + r // scaling


def client_inputs(calls):
    """Inputs of the client's `calls`-th cuBERT_compute (benchmark_cu.cpp:25-34)."""
    e = MinstdRand0(0)
    ids = np.zeros(BATCH * SEQ, np.int32)
    mask = np.zeros(BATCH * SEQ, np.int8)
    seg = np.zeros(BATCH * SEQ, np.int8)
    for _ in range(calls):
        for i in range(BATCH * SEQ):
            ids[i] = uniform_int(e, 0, 21120)
            mask[i] = uniform_int(e, 0, 1)
            seg[i] = uniform_int(e, 0, 1)
    return ids.reshape(BATCH, SEQ), mask.reshape(BATCH, SEQ), seg.reshape(BATCH, SEQ)


def test_engine_replay_known_values():
    """minstd_rand0's 10000th value from seed 1 is 1043618065 (C++ standard, [rand.predef]); seed 0 acts as 1."""
    e = MinstdRand0(0)
    for _ in range(9999):
        e()
    assert e() == 1043618065


@pytest.mark.gpu
@pytest.mark.skipif(not os.path.exists(CLIENT), reason="oracle/_ref/benchmark_cu is built where the reference is mounted")
def test_reference_benchmark_client_runs_against_this_library(tmp_path):
    from cubert_amd.graphdef import write_graphdef
    from cubert_amd.testing import CONFIGS, config_weights
    w = config_weights("C1", seed=0)
    write_graphdef(str(tmp_path / "bert_frozen_seq32.pb"), w)
    r = subprocess.run([CLIENT], cwd=str(tmp_path), stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stdout[-2000:]
    times = [int(t) for t in re.findall(r"cuBERT: (\d+)ms", r.stdout)]
    assert len(times) == CALLS, r.stdout[-2000:]
    print("reference client, batch 128 seq 32 POOLED_OUTPUT, host arrays in and out: warm-up %s ms, timed %s ms"
          % (times[:10], times[10:]))
    out = np.loadtxt(str(tmp_path / "cuBERT.txt"), dtype=np.float32)
    assert out.size == CALLS * BATCH * HIDDEN
    last = out.reshape(CALLS, BATCH, HIDDEN)[-1]
    assert np.abs(last).max() <= 1.0  # tanh pooler
    ids, mask, seg = client_inputs(CALLS)
    m = CONFIGS["C1"]["model"]
    rows = 16  # sequences are independent: the oracle runs a prefix of the batch
    want = oracle.bert_forward(w, ids[:rows], mask[:rows], seg[:rows], m["layers"], m["heads"])["pooled_output"]
    # the client prints 6 significant digits
    assert_close(last[:rows], want, 2e-5, "pooled output written by the reference client")


@pytest.mark.skipif(not PY_EXTENSION, reason="oracle/_ref/cuBERT.*.so is built where the reference is mounted")
def test_reference_python_extension_links_against_this_library():
    """The reference's Cython extension (python/cuBERT.pyx + _cuBERT.pxd), translated and compiled unmodified by
    oracle/Makefile, needs nothing from libcuBERT.so that the library does not export: every cuBERT_* symbol it
    leaves undefined is defined there, and the dynamic linker resolves the rest.  A link check in the build
    container only: the extension is neither imported here nor carried to the GPU box."""
    from cubert_amd._lib import LIB_PATH

    def symbols(path, flag):
        out = subprocess.check_output(["nm", "-D", flag, path], text=True)
        return set(l.split()[-1].split("@")[0] for l in out.splitlines() if l.strip())

    wanted = set(n for n in symbols(PY_EXTENSION[0], "--undefined-only") if n.startswith("cuBERT_"))
    # the nine entry points python/cuBERT.pyx calls (its compute and tokenize_compute go through the _m variants)
    assert wanted == {"cuBERT_initialize", "cuBERT_finalize", "cuBERT_get_gpu_count", "cuBERT_open",
                      "cuBERT_compute_m", "cuBERT_close", "cuBERT_open_tokenizer", "cuBERT_close_tokenizer",
                      "cuBERT_tokenize_compute_m"}, sorted(wanted)
    assert wanted <= symbols(LIB_PATH, "--defined-only")
    r = subprocess.run(["ldd", "-r", PY_EXTENSION[0]], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    unresolved = [l for l in r.stdout.splitlines() if "undefined symbol" in l and "Py" not in l and "_Py" not in l]
    assert not unresolved, unresolved


@pytest.mark.gpu
@pytest.mark.parametrize("compute_type", [0, 1])
def test_public_symbols_driven_the_way_the_reference_python_binding_drives_them(tmp_path, compute_type):
    """The calls python/cuBERT.pyx makes, in its order, on the exported cuBERT_* symbols themselves (not the
    exception-free cubert_try_* forms the package uses): cuBERT_initialize at import (cuBERT.pyx:9),
    cuBERT_open then cuBERT_open_tokenizer (:121-138), cuBERT_compute_m and cuBERT_tokenize_compute_m with a
    cuBERT_Output whose five pointers sit in the header's order and of which only some are set (:41-114,171-177,
    202-208), cuBERT_close then cuBERT_close_tokenizer (:140-143), cuBERT_finalize (:10).  Outputs carry the
    model's element type (half for a half model).  The argument-error paths are C++ exceptions there (`except +`
    in _cuBERT.pxd) and cannot cross ctypes; they are covered through cubert_try_* in the model tests."""
    import ctypes
    from cubert_amd._lib import LIB_PATH, cuBERT_Output
    from cubert_amd.graphdef import write_graphdef
    from cubert_amd.testing import random_bert_weights, random_inputs
    from oracle import tokenizer as otok
    cfg = dict(vocab=211, hidden=128, layers=3, heads=4, intermediate=512, max_position=64, type_vocab=2)
    w = random_bert_weights(seed=5, labels=2, ln_random=True, **cfg)
    write_graphdef(str(tmp_path / "model.pb"), w)
    lines = ["[PAD]", "[UNK]", "[CLS]", "[SEP]"] + list("abcdefghijklmnopqrstuvwxyz") + ["##" + c for c in "abcdefgh"]
    (tmp_path / "vocab.txt").write_text("\n".join(lines) + "\n", encoding="utf8")

    L = ctypes.CDLL(LIB_PATH)  # a second handle on the same library, with the signatures of _cuBERT.pxd only
    vp, ci = ctypes.c_void_p, ctypes.c_int
    L.cuBERT_open.restype, L.cuBERT_open.argtypes = vp, [ctypes.c_char_p, ci, ci, ci, ci, ci]
    L.cuBERT_open_tokenizer.restype, L.cuBERT_open_tokenizer.argtypes = vp, [ctypes.c_char_p, ci]
    L.cuBERT_compute_m.restype = None
    L.cuBERT_compute_m.argtypes = [vp, ci, vp, vp, vp, ctypes.POINTER(cuBERT_Output), ci, ci]
    L.cuBERT_tokenize_compute_m.restype = None
    L.cuBERT_tokenize_compute_m.argtypes = [vp, vp, ci, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(ctypes.c_char_p),
                                            ctypes.POINTER(cuBERT_Output), ci, ci]
    L.cuBERT_close.restype, L.cuBERT_close.argtypes = None, [vp, ci]
    L.cuBERT_close_tokenizer.restype, L.cuBERT_close_tokenizer.argtypes = None, [vp]
    L.cuBERT_get_gpu_count.restype = ci

    assert [name for name, _ in cuBERT_Output._fields_] == ["logits", "pooled_output", "sequence_output",
                                                            "embedding_output", "probs"]
    assert ctypes.sizeof(cuBERT_Output) == 5 * ctypes.sizeof(vp)

    half = compute_type == 1
    dt = np.float16 if half else np.float32
    tol = 1e-2 if half else 1e-5
    wf = {k: oracle.round_to_half(v) for k, v in w.items()} if half else w

    L.cuBERT_initialize()
    assert L.cuBERT_get_gpu_count() >= 1
    model = L.cuBERT_open(str(tmp_path / "model.pb").encode(), 4, 32, cfg["layers"], cfg["heads"], compute_type)
    tokenizer = L.cuBERT_open_tokenizer(str(tmp_path / "vocab.txt").encode(), 1)
    assert model and tokenizer

    ids, mask, seg = random_inputs(seed=6, batch=3, seq_length=32, vocab=cfg["vocab"], min_valid=4, segment_split=9)
    want = oracle.bert_forward(wf, ids, mask, seg, cfg["layers"], cfg["heads"])
    pooled, probs = np.full((3, 128), np.nan, dt), np.full((3, 2), np.nan, dt)
    out = cuBERT_Output(None, pooled.ctypes.data, None, None, probs.ctypes.data)   # Output(pooled_output=..., probs=...)
    L.cuBERT_compute_m(model, 3, ids.ctypes.data, mask.ctypes.data, seg.ctypes.data, ctypes.byref(out), compute_type, 0)
    assert_close(pooled.astype(np.float32), want["pooled_output"], tol, "pooled_output")
    assert_close(probs.astype(np.float32), want["probs"], tol, "probs")

    # Output(sequence_output) alone, the way compute() wraps one array (cuBERT.pyx:147-156)
    sequence = np.full((3, 32, 128), np.nan, dt)
    out = cuBERT_Output(None, None, sequence.ctypes.data, None, None)
    L.cuBERT_compute_m(model, 3, ids.ctypes.data, mask.ctypes.data, seg.ctypes.data, ctypes.byref(out), compute_type, 0)
    if half:   # token-level bound of the model tests: 1e-2 * max(1, |x|)
        assert np.all(np.abs(sequence.astype(np.float32) - want["sequence_output"]) <=
                      1e-2 * np.maximum(1.0, np.abs(want["sequence_output"])))
    else:
        assert_close(sequence, want["sequence_output"], tol, "sequence_output")

    text_a, text_b = ["abc def", "hello again", "x"], ["gh", "", "zzz yx"]
    vocab = otok.load_vocab(lines)
    feats = [otok.convert_single_example(vocab, 32, a, b) for a, b in zip(text_a, text_b)]
    t_ids = np.array([f[0] for f in feats], np.int32)
    t_mask = np.array([f[1] for f in feats], np.int8)
    t_seg = np.array([f[2] for f in feats], np.int8)
    want = oracle.bert_forward(wf, t_ids, t_mask, t_seg, cfg["layers"], cfg["heads"])
    arr_a = (ctypes.c_char_p * 3)(*[s.encode() for s in text_a])
    arr_b = (ctypes.c_char_p * 3)(*[s.encode() for s in text_b])
    logits = np.full((3, 2), np.nan, dt)
    out = cuBERT_Output(logits.ctypes.data, None, None, None, None)
    L.cuBERT_tokenize_compute_m(model, tokenizer, 3, arr_a, arr_b, ctypes.byref(out), compute_type, 0)
    assert_close(logits.astype(np.float32), want["logits"], tol, "logits from texts")

    L.cuBERT_close(model, compute_type)
    L.cuBERT_close_tokenizer(tokenizer)
    L.cuBERT_finalize()
