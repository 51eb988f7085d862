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
