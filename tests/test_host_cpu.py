"""CPU-side checks: the shared library loads and exports exactly what include/*.h declares, the
GraphDef writer produces files its reader (and the wire format) agree on, and the synthetic
weight/input generators are deterministic.  No device call is made here."""
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")


def declared_functions():
    names = set()
    for header in ("cuBERT.h", "cubert_kernels.h", "cubert_host.h"):
        text = open(os.path.join(INCLUDE, header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        names.update(re.findall(r"\b(cuBERT_\w+|cubert_\w+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    from cubert_amd._lib import LIB_PATH, SIGNATURES, lib
    assert os.path.exists(LIB_PATH), "build the library first: python -m cubert_amd.build"
    declared = declared_functions()
    assert len(declared) > 50
    exported = set(l.split()[-1] for l in subprocess.check_output(["nm", "-D", "--defined-only", LIB_PATH],
                                                                   text=True).splitlines())
    assert declared <= exported, sorted(declared - exported)
    assert declared == set(SIGNATURES), sorted(declared ^ set(SIGNATURES))
    lib()  # resolves every symbol through ctypes


def test_public_header_is_valid_c_and_abi_constants():
    """cuBERT.h must stay usable from C callers and keep the reference's enum values / field order."""
    src = '#include "cuBERT.h"\n#include "cubert_kernels.h"\n#include "cubert_host.h"\n' \
          '#include <stddef.h>\n' \
          '_Static_assert(cuBERT_COMPUTE_FLOAT == 0 && cuBERT_COMPUTE_HALF == 1, "compute type");\n' \
          '_Static_assert(cuBERT_LOGITS == 0 && cuBERT_POOLED_OUTPUT == 1 && cuBERT_SEQUENCE_OUTPUT == 2 && ' \
          'cuBERT_EMBEDDING_OUTPUT == 3 && cuBERT_PROBS == 4, "output type");\n' \
          '_Static_assert(offsetof(cuBERT_Output, logits) == 0 && offsetof(cuBERT_Output, pooled_output) == 8 && ' \
          'offsetof(cuBERT_Output, sequence_output) == 16 && offsetof(cuBERT_Output, embedding_output) == 24 && ' \
          'offsetof(cuBERT_Output, probs) == 32, "output struct");\nint main(void) { return 0; }\n'
    subprocess.run(["gcc", "-std=c11", "-fsyntax-only", "-I", INCLUDE, "-x", "c", "-"], input=src, text=True, check=True)
    from cubert_amd._lib import cuBERT_Output
    assert [f[0] for f in cuBERT_Output._fields_] == ["logits", "pooled_output", "sequence_output", "embedding_output",
                                                      "probs"]


def test_no_gpu_reports_zero_devices_or_more():
    from cubert_amd import get_gpu_count
    assert get_gpu_count() >= 0


def test_graphdef_round_trip(tmp_path):
    from cubert_amd.graphdef import read_graphdef, write_graphdef
    rng = np.random.default_rng(0)
    w = {"bert/embeddings/word_embeddings": rng.normal(size=(300, 24)).astype(np.float32),
         "output_weights": rng.normal(size=(3, 24)).astype(np.float16),
         "output_bias": rng.normal(size=3).astype(np.float32),
         "a/scalar": np.float32(2.5).reshape(())}
    path = write_graphdef(str(tmp_path / "m.pb"), w)
    back = read_graphdef(path)
    assert set(back) == set(w)
    for k in w:
        assert back[k].dtype == w[k].dtype and back[k].shape == w[k].shape
        assert np.array_equal(back[k], w[k])


def test_graphdef_wire_format_matches_protobuf_library(tmp_path):
    """Decode the written bytes with google.protobuf's own wire decoder (no TensorFlow schema needed):
    field numbers GraphDef.node=1, NodeDef.name=1/op=2/attr=5, AttrValue.tensor=8, TensorProto.dtype=1/
    tensor_shape=2/tensor_content=4."""
    decoder = pytest.importorskip("google.protobuf.internal.decoder")
    from cubert_amd.graphdef import write_graphdef
    w = {"x": np.arange(6, dtype=np.float32).reshape(2, 3)}
    buf = open(write_graphdef(str(tmp_path / "m.pb"), w), "rb").read()

    def fields(b):
        pos, out = 0, []
        while pos < len(b):
            tag, pos = decoder._DecodeVarint(b, pos)
            num, wire = tag >> 3, tag & 7
            if wire == 0:
                v, pos = decoder._DecodeVarint(b, pos)
            else:
                assert wire == 2
                n, pos = decoder._DecodeVarint(b, pos)
                v, pos = b[pos:pos + n], pos + n
            out.append((num, v))
        return out

    node = dict(fields(buf))[1]
    nf = fields(node)
    assert (1, b"x") in nf and (2, b"Const") in nf
    attrs = {dict(fields(v))[1]: dict(fields(v))[2] for n, v in nf if n == 5}
    tensor = dict(fields(dict(fields(attrs[b"value"]))[8]))
    assert tensor[1] == 1  # DT_FLOAT
    dims = [dict(fields(v))[1] for n, v in fields(tensor[2]) if n == 2]
    assert dims == [2, 3]
    assert np.array_equal(np.frombuffer(tensor[4], np.float32), np.arange(6, dtype=np.float32))


from util import tf_style_fixture


@pytest.mark.parametrize("compute_type", [0, 1])
def test_loader_reads_a_graphdef_written_the_way_tensorflow_writes_one(compute_type):
    """Scalars and splats in float_val / half_val (packed and unpacked), a weight stored as DT_HALF, non-Const
    nodes, a fixed32 attr, int32 Consts, versions and a function library, a repeated name: every float / half
    constant arrives bit-exact (after conversion to the model's type), nothing else does, nothing throws."""
    import cubert_amd
    path, expected, absent = tf_style_fixture()
    g = cubert_amd.Graph(path, compute_type)
    assert (g.vocab_size, g.type_vocab_size, g.hidden_size, g.intermediate_size, g.num_labels) == (37, 2, 16, 32, 3)
    assert len(g) == len(expected)
    for name, want in expected.items():
        got = g.var(name)
        assert got is not None, name
        data, shape = got
        want = want.astype(np.float32 if compute_type == 0 else np.float16)
        assert data.shape == (want.size,), (name, data.shape, want.shape)
        assert np.array_equal(data.view(np.uint32 if compute_type == 0 else np.uint16),
                              want.reshape(-1).view(np.uint32 if compute_type == 0 else np.uint16)), name
    assert g.var("bert/embeddings/word_embeddings")[1] == (37, 16)
    assert g.var("bert/embeddings/LayerNorm/batchnorm/add/y")[1] == ()
    # the function library's Const of the same name did not replace the weight
    assert not np.any(g.var("bert/embeddings/LayerNorm/beta")[0] == 99)
    for name in absent:
        assert g.var(name) is None, name
    g.close()


def test_loader_keeps_what_the_file_holds_when_the_declared_shape_disagrees(tmp_path):
    """The element count of a constant is the length of its tensor_content, whatever its shape says (reference
    tensorflow/Graph.cpp:50-56); a model whose tensors do not fit is refused where it is built, by name."""
    import cubert_amd
    from cubert_amd.graphdef import _bytes_field, _field, _varint
    content = np.arange(5, dtype=np.float32).tobytes()
    shape = _bytes_field(2, _field(1, 0, _varint(2))) + _bytes_field(2, _field(1, 0, _varint(3)))   # says [2, 3]
    tensor = _field(1, 0, _varint(1)) + _bytes_field(2, shape) + _bytes_field(4, content)
    # AttrValue with the tensor first and another member of the oneof after it: the later member is the one set
    overwritten = _bytes_field(8, tensor) + _field(3, 0, _varint(7))
    nodes = b""
    for name, attr in (("odd/shape", _bytes_field(8, tensor)), ("odd/oneof", overwritten)):
        entry = _bytes_field(1, b"value") + _bytes_field(2, attr)
        nodes += _bytes_field(1, _bytes_field(1, name.encode()) + _bytes_field(2, b"Const") + _bytes_field(5, entry))
    path = tmp_path / "odd.pb"
    path.write_bytes(nodes)
    g = cubert_amd.Graph(str(path))
    data, shape = g.var("odd/shape")
    assert shape == (2, 3) and np.array_equal(data, np.arange(5, dtype=np.float32))
    assert g.var("odd/oneof") is None and len(g) == 1
    g.close()
    # truncated in the middle of a node: an error, not a crash
    (tmp_path / "cut.pb").write_bytes(nodes[:len(nodes) - 9])
    with pytest.raises(ValueError, match="model file invalid"):
        cubert_amd.Graph(str(tmp_path / "cut.pb"))
    with pytest.raises(ValueError, match="model file not found"):
        cubert_amd.Graph(str(tmp_path / "missing.pb"))


def test_open_accepts_the_tensorflow_style_file_up_to_the_device_check():
    """cuBERT_open on the fixture: the loader and the size checks pass (seq_length 8 of 12 positions), and without a
    GPU the call ends at the device count like the reference's (BertM.cpp:20-22)."""
    import cubert_amd
    path, _, _ = tf_style_fixture()
    if cubert_amd.get_gpu_count() == 0:
        with pytest.raises(ValueError, match="No GPU device detected"):
            cubert_amd.Model(path, 4, 8, 2, 2)
    with pytest.raises(ValueError, match="position_embeddings holds 192 elements, the model needs 256"):
        cubert_amd.Model(path, 4, 16, 2, 2)


def test_generators_are_deterministic_and_follow_the_configs():
    from cubert_amd.testing import CONFIGS, config_inputs, random_bert_weights
    small = dict(vocab=50, hidden=16, layers=2, heads=2, intermediate=32, max_position=8, type_vocab=2)
    a = random_bert_weights(seed=1, **small)
    b = random_bert_weights(seed=1, **small)
    assert all(np.array_equal(a[k], b[k]) for k in a)
    assert a["bert/embeddings/word_embeddings"].shape == (50, 16)
    assert a["bert/encoder/layer_1/intermediate/dense/kernel"].shape == (16, 32)
    assert a["output_weights"].shape == (2, 16)
    assert abs(a["bert/embeddings/word_embeddings"].std() - 0.02) < 0.003
    assert (a["bert/encoder/layer_0/output/LayerNorm/gamma"] == 1).all()
    ids, mask, seg = config_inputs("C1")
    assert ids.shape == (128, 32) and ids.dtype == np.int32 and mask.dtype == np.int8 and seg.dtype == np.int8
    assert ids.min() >= 0 and ids.max() < 21128
    valid = mask.sum(1)
    assert valid.min() >= 8 and valid.max() <= 32 and (np.diff(mask.astype(int), axis=1) <= 0).all()
    assert (seg[:, :16] == 0).all() and (seg[:, 16:] == 1).all()
    ids3, mask3, _ = config_inputs("C3")
    assert ids3.shape == (64, 512) and mask3.sum(1).min() >= 16
    _, mask4, seg4 = config_inputs("C4")
    assert mask4.all() and (seg4[:, 0] == 0).all() and (seg4[:, -1] == 1).all()
    assert set(CONFIGS) == {"C0", "C1", "C2", "C3", "C4"}


def test_open_rejects_files_whose_tensors_do_not_fit_the_model(tmp_path):
    """cuBERT_open checks every tensor's element count against the sizes in the file and its own arguments before
    anything is copied (the reference trusts the file); this happens before the GPU is looked for, so it runs
    here.  A consistent file gets as far as the device count."""
    import cubert_amd
    from cubert_amd.graphdef import write_graphdef
    from cubert_amd.testing import random_bert_weights
    small = dict(vocab=50, hidden=32, layers=2, heads=4, intermediate=64, max_position=16, type_vocab=2)
    w = random_bert_weights(seed=1, labels=2, **small)

    def open_(weights, seq_length=16, layers=2):
        path = write_graphdef(str(tmp_path / "m.pb"), weights)
        model = cubert_amd.Model(path, 2, seq_length, layers, 4)
        model.close()

    with pytest.raises(ValueError, match="position_embeddings holds 512 elements, the model needs 1024"):
        open_(w, seq_length=32)                      # longer sequences than the position table has rows
    bad = dict(w)
    bad["bert/encoder/layer_1/intermediate/dense/kernel"] = w["bert/encoder/layer_1/intermediate/dense/kernel"][:, :60]
    with pytest.raises(ValueError, match="layer_1/intermediate/dense/kernel holds 1920 elements, the model needs 2048"):
        open_(bad)
    bad = dict(w)
    bad["output_bias"] = np.zeros(3, np.float32)
    with pytest.raises(ValueError, match="output_bias holds 3 elements"):
        open_(bad)
    if cubert_amd.get_gpu_count() == 0:
        with pytest.raises(ValueError, match="No GPU device detected"):
            open_(w)
    else:
        open_(w)


def test_input_range_check():
    """What Bert<T>::compute checks before it enqueues anything: ids in [0, vocab), segment ids in [0, types)."""
    from cubert_amd._lib import lib
    L = lib()
    ids = np.array([0, 5, 20, 99, 3], np.int32)
    seg = np.array([0, 1, 0, 1, 1], np.int8)

    def check(i, s, vocab, types):
        rc = L.cubert_check_input_range(i.ctypes.data, s.ctypes.data, i.size, vocab, types)
        return rc, L.cubert_last_error().decode()

    assert check(ids, seg, 100, 2) == (0, "")
    assert check(ids[:0], seg[:0], 100, 2) == (0, "")
    assert check(ids, seg, 99, 2) == (1, "input id out of range: input_ids[3] = 99, vocab_size = 99")
    neg = ids.copy()
    neg[1] = -7
    assert check(neg, seg, 100, 2) == (1, "input id out of range: input_ids[1] = -7, vocab_size = 100")
    assert check(ids, seg, 100, 1) == (1, "segment id out of range: segment_ids[1] = 1, type_vocab_size = 1")
    bad = seg.copy()
    bad[4] = -1
    assert check(ids, bad, 100, 2) == (1, "segment id out of range: segment_ids[4] = -1, type_vocab_size = 2")
    big = np.arange(1 << 15, dtype=np.int32)
    assert check(big, np.zeros(big.size, np.int8), 1 << 15, 2)[0] == 0
    assert check(big, np.zeros(big.size, np.int8), (1 << 15) - 1, 2)[0] == 1


def test_open_warmup_batch_list():
    """CUBERT_OPEN_WARMUP as a model reads it when it is opened: unset = the maximum batch (what the reference
    prepares, src/cuBERT/Bert.cpp:62-64), "0" = nothing, else a list of batch sizes with "max" for the maximum."""
    import ctypes
    from cubert_amd._lib import lib
    L = lib()

    def batches(setting, max_batch):
        out = (ctypes.c_size_t * 16)()
        n = L.cubert_open_warmup_batches(None if setting is None else setting.encode(), max_batch, out, 16)
        return [out[i] for i in range(min(n, 16))]

    assert batches(None, 128) == [128]
    assert batches("0", 128) == []
    assert batches("", 128) == []
    assert batches("1,8,32", 128) == [1, 8, 32]
    assert batches(" 8 , max,1,8", 128) == [8, 128, 1]          # order kept, repeats dropped
    assert batches("1", 128) == [1]
    assert batches("max", 4) == [4]
    assert batches("1,129,0,x,-3,16", 128) == [1, 16]           # the others are named on stderr and skipped
    assert batches("99999999999999999999999", 128) == []


def test_bench_refuses_more_than_one_gpu():
    """This build measures one GPU: `bench.py --gpus N` with N > 1 exits with a message instead of a number."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_bench_algorithmic_bytes_follow_the_published_formulas():
    """Per-launch algorithmic bytes of the fused kernels at the benchmark shapes (every operand once)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    from cubert_amd.testing import CONFIGS
    os.environ.pop("CUBERT_FP32_DENSE", None)
    mb = {name: {k: v / 1e6 for k, v in bench.algorithmic_bytes(CONFIGS[name]).items()} for name in CONFIGS}
    # bias+GELU 2*M*I*e + I*e, bias+residual+LN 3*M*H*e + 3*H*e, mask+softmax 2*B*A*S^2*e + B*S, embed+LN
    for name, gelu, ln, softmax, embed in (("C1", 100.7, 37.8, 12.6, 25.3), ("C3", 402.7, 151.0, 805.3, 101.6),
                                           ("C4", 536.9, 201.3, 268.5, 134.7)):
        assert abs(mb[name]["bias_gelu"] - gelu) < 0.06 and abs(mb[name]["bias_res_ln"] - ln) < 0.06
        assert abs(mb[name]["mask_scale_softmax"] - softmax) < 0.06 and abs(mb[name]["embed_ln"] - embed) < 0.06
    os.environ["CUBERT_FP32_DENSE"] = "f16x3"
    try:
        two_term = bench.algorithmic_bytes(CONFIGS["C1"])
        half_model = bench.algorithmic_bytes(CONFIGS["C3"])
    finally:
        del os.environ["CUBERT_FP32_DENSE"]
    assert two_term["bias_gelu"] == 4096 * 3072 * 10 + 3072 * 4 and two_term["dense_split"] == 4096 * 768 * 10
    assert half_model["bias_gelu"] == bench.algorithmic_bytes(CONFIGS["C3"])["bias_gelu"]  # fp16 models: unchanged
