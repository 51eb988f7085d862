"""Seeded synthetic BERT weights and inputs.

The reference never generates a model (it only loads a frozen TensorFlow
GraphDef), so benchmarks and parity tests need their own deterministic source:
numpy's PCG64 with a fixed seed, one child stream per tensor name, so a tensor's
values do not depend on which other tensors were asked for.
"""
import zlib

import numpy as np

BERT_BASE = dict(vocab=21128, hidden=768, layers=12, heads=12, intermediate=3072, max_position=512, type_vocab=2)
BERT_LARGE = dict(vocab=30522, hidden=1024, layers=24, heads=16, intermediate=4096, max_position=512, type_vocab=2)


def _stream(seed, name):
    return np.random.Generator(np.random.PCG64([seed, zlib.crc32(name.encode())]))


def random_bert_weights(seed=0, vocab=21128, hidden=768, layers=12, heads=12, intermediate=3072, max_position=512,
                        type_vocab=2, labels=2, pooler=True, classifier=True, classifier_bias=True, ln_random=False,
                        stddev=0.02):
    """Weights keyed by the TensorFlow variable names the reference looks up
    (BertEmbeddings.cpp:19-27, AttentionSelf.cpp:27-44, Transformer.cpp:54-101,
    Bert.cpp:34-46).  Kernels, embeddings and biases ~ N(0, stddev); LayerNorm
    gamma = 1, beta = 0 unless ln_random (then gamma ~ N(1, .1), beta ~ N(0, .1)
    so that the affine part of LayerNorm is exercised)."""
    del heads
    w = {}

    def normal(name, *shape):
        w[name] = _stream(seed, name).standard_normal(shape, dtype=np.float32) * np.float32(stddev)

    def layer_norm(prefix):
        if ln_random:
            w[prefix + "/gamma"] = (1 + 0.1 * _stream(seed, prefix + "/gamma").standard_normal(hidden)).astype(np.float32)
            w[prefix + "/beta"] = (0.1 * _stream(seed, prefix + "/beta").standard_normal(hidden)).astype(np.float32)
        else:
            w[prefix + "/gamma"] = np.ones(hidden, np.float32)
            w[prefix + "/beta"] = np.zeros(hidden, np.float32)

    normal("bert/embeddings/word_embeddings", vocab, hidden)
    normal("bert/embeddings/token_type_embeddings", type_vocab, hidden)
    normal("bert/embeddings/position_embeddings", max_position, hidden)
    layer_norm("bert/embeddings/LayerNorm")
    for l in range(layers):
        p = "bert/encoder/layer_%d" % l
        for n in ("query", "key", "value"):
            normal("%s/attention/self/%s/kernel" % (p, n), hidden, hidden)
            normal("%s/attention/self/%s/bias" % (p, n), hidden)
        normal(p + "/attention/output/dense/kernel", hidden, hidden)
        normal(p + "/attention/output/dense/bias", hidden)
        layer_norm(p + "/attention/output/LayerNorm")
        normal(p + "/intermediate/dense/kernel", hidden, intermediate)
        normal(p + "/intermediate/dense/bias", intermediate)
        normal(p + "/output/dense/kernel", intermediate, hidden)
        normal(p + "/output/dense/bias", hidden)
        layer_norm(p + "/output/LayerNorm")
    if pooler:
        normal("bert/pooler/dense/kernel", hidden, hidden)
        normal("bert/pooler/dense/bias", hidden)
    if classifier:
        normal("output_weights", labels, hidden)
        if classifier_bias:
            normal("output_bias", labels)
    return w


def random_inputs(seed, batch, seq_length, vocab, min_valid=None, max_valid=None, segment_split=None,
                  scattered_mask=False, valid_lengths=None):
    """input_ids ~ U[0, vocab); input_mask = 1 on a prefix whose length is
    U{min_valid..max_valid} per row (all ones when min_valid is None), or an
    arbitrary 0/1 pattern when scattered_mask (the reference's BertTest uses
    such masks: any non-zero byte keeps the key).  segment_ids: 0 before
    `segment_split` and 1 after; segment_split may be an int, "random" (U{1..S-1}
    per row) or None (all 0)."""
    rng = np.random.Generator(np.random.PCG64([seed, 0xC0FFEE]))
    S = seq_length
    ids = rng.integers(0, vocab, (batch, S), dtype=np.int32)
    pos = np.arange(S)[None, :]
    if valid_lengths is not None:
        mask = (pos < np.asarray(valid_lengths)[:, None]).astype(np.int8)
    elif scattered_mask:
        mask = (rng.random((batch, S)) < 0.6).astype(np.int8)
        mask[:, 0] |= (mask.sum(1) == 0)  # keep at least one key per row
        mask *= rng.integers(1, 4, (batch, S), dtype=np.int8)  # non-zero values other than 1 also mean "keep"
    elif min_valid is None:
        mask = np.ones((batch, S), np.int8)
    else:
        hi = S if max_valid is None else max_valid
        mask = (pos < rng.integers(min_valid, hi + 1, (batch, 1))).astype(np.int8)
    if segment_split is None:
        seg = np.zeros((batch, S), np.int8)
    elif segment_split == "random":
        seg = (pos >= rng.integers(1, S, (batch, 1))).astype(np.int8)
    else:
        seg = np.broadcast_to(pos >= segment_split, (batch, S)).astype(np.int8)
    return ids, mask, np.ascontiguousarray(seg)


# The five workloads of the benchmark definition (sizes, input statistics, outputs).
CONFIGS = {
    "C0": dict(model=BERT_BASE, dtype="f32", batch=1, seq_length=32, labels=2, pooler=True,
               inputs=dict(min_valid=None, segment_split=None)),
    "C1": dict(model=BERT_BASE, dtype="f32", batch=128, seq_length=32, labels=2, pooler=True,
               inputs=dict(min_valid=8, max_valid=32, segment_split=16)),
    "C2": dict(model=BERT_BASE, dtype="f16", batch=32, seq_length=128, labels=2, pooler=False,
               inputs=dict(min_valid=16, max_valid=128, segment_split=None)),
    "C3": dict(model=BERT_BASE, dtype="f16", batch=64, seq_length=512, labels=2, pooler=True,
               inputs=dict(valid="exp", segment_split=None)),
    "C4": dict(model=BERT_LARGE, dtype="f16", batch=256, seq_length=128, labels=3, pooler=True,
               inputs=dict(min_valid=None, segment_split="random")),
}


def config_inputs(name, seed=0, batch=None):
    c = CONFIGS[name]
    B = batch or c["batch"]
    S = c["seq_length"]
    kw = dict(c["inputs"])
    if kw.pop("valid", None) == "exp":
        # heavy padding: valid length = min(S, 16 + Exp(mean 96))
        rng = np.random.Generator(np.random.PCG64([seed, 0xE4B]))
        kw["valid_lengths"] = np.minimum(S, 16 + np.floor(rng.exponential(96.0, B))).astype(np.int64)
    return random_inputs(seed, B, S, c["model"]["vocab"], **kw)


def config_weights(name, seed=0):
    c = CONFIGS[name]
    return random_bert_weights(seed=seed, labels=c["labels"], pooler=c["pooler"], classifier=True, **c["model"])
