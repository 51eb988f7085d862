"""Run by test_reference_client_gpu.py in a process of its own: drives the reference's Cython extension
(python/cuBERT.pyx, built unmodified into oracle/_ref/ and linked with this repository's libcuBERT.so) the way
the reference's python/cuBERT_test.py does, and saves what it returned.

    python reference_python_client.py <dir with cuBERT.*.so> <model.pb> <vocab.txt> <inputs.npz> <out.npz>
"""
import sys

import numpy as np


def main(ext_dir, model_file, vocab_file, inputs_file, out_file):
    sys.path.insert(0, ext_dir)
    import cuBERT  # the reference's extension module; initialises the library on import
    assert cuBERT.__file__.startswith(ext_dir), cuBERT.__file__
    got = {"gpu_count": np.int64(cuBERT.get_gpu_count())}
    z = np.load(inputs_file)
    ids, mask, seg = z["ids"], z["mask"], z["seg"]
    layers, heads, hidden, labels = (int(v) for v in z["shape"])
    batch, seq = ids.shape
    text_a = [str(t) for t in z["text_a"]]
    text_b = [str(t) for t in z["text_b"]]

    model = cuBERT.Model(model_file, 8, seq, layers, heads, compute_type=cuBERT.ComputeType.FLOAT)
    for name, kind, shape in (("logits", cuBERT.OutputType.LOGITS, (batch, labels)),
                              ("probs", cuBERT.OutputType.PROBS, (batch, labels)),
                              ("pooled_output", cuBERT.OutputType.POOLED_OUTPUT, (batch, hidden)),
                              ("sequence_output", cuBERT.OutputType.SEQUENCE_OUTPUT, (batch, seq, hidden)),
                              ("embedding_output", cuBERT.OutputType.EMBEDDING_OUTPUT, (batch, seq, hidden))):
        out = np.zeros(shape, np.float32, order="C")
        model.compute(ids, mask, seg, out, output_type=kind)
        got["compute_" + name] = out
    o = cuBERT.Output()
    o.logits = np.zeros((batch, labels), np.float32)
    o.pooled_output = np.zeros((batch, hidden), np.float32)
    model.compute_m(ids, mask, seg, o)
    got["compute_m_logits"], got["compute_m_pooled_output"] = o.logits, o.pooled_output
    del model

    half = cuBERT.Model(model_file, 8, seq, layers, heads, compute_type=cuBERT.ComputeType.HALF)
    out = np.zeros((batch, labels), np.float16)
    half.compute(ids, mask, seg, out, output_type=cuBERT.OutputType.LOGITS)
    got["half_logits"] = out
    del half

    model = cuBERT.Model(model_file, 8, seq, layers, heads, vocab_file=vocab_file)
    out = np.zeros((len(text_a), labels), np.float32)
    model.tokenize_compute(text_a, text_b, out, output_type=cuBERT.OutputType.LOGITS)
    got["tokenize_logits"] = out
    o = cuBERT.Output()
    o.probs = np.zeros((len(text_a), labels), np.float32)
    model.tokenize_compute_m(text_a, None, o)
    got["tokenize_single_probs"] = o.probs
    try:  # errors cross the C boundary as C++ exceptions, which the extension turns into Python ones
        model.compute(np.zeros((9, seq), np.int32), np.zeros((9, seq), np.int8), np.zeros((9, seq), np.int8),
                      np.zeros((9, labels), np.float32))
        got["too_large_batch"] = np.array("no error")
    except Exception as e:  # noqa: BLE001
        got["too_large_batch"] = np.array("%s: %s" % (type(e).__name__, e))
    del model
    np.savez(out_file, **got)
    print("reference python client done", flush=True)


if __name__ == "__main__":
    main(*sys.argv[1:6])
