"""Pins the CPU oracle (oracle/cubert_oracle.c) before anything is compared with it:
 1. every known-answer vector the reference's own gtest files hold for this path,
 2. the reference's own CPU launchers compiled from /root/reference (bit-exact,
    where oracle/_ref was built),
 3. textbook float64 formulations (numpy / scipy), chosen so that a dropped term,
    a wrong sign/index or a transposed operand fails.
"""
import math

import numpy as np
import pytest

import oracle

T = "test/cuBERT/"


# ---------------------------------------------------------------- 1. reference vectors

def test_embedding_vector(case):
    c = case(T + "op/EmbeddingTest.cpp", "embedding")
    table = np.array(c.arrays["embedding_table"], np.float32).reshape(4, 3)
    out = oracle.embedding(np.array(c.arrays["input_ids"], np.int32), table)
    assert c.check(out) == 9


def test_dense_vector(case):
    c = case(T + "op/DenseTest.cpp", "dense")
    out = oracle.dense(np.array(c.arrays["input"]).reshape(3, 2), np.array(c.arrays["kernel"]).reshape(2, 3),
                       c.arrays["bias"])
    assert c.check(out) == 9


def test_gelu_vector(case):
    c = case(T + "op/GELUTest.cpp", "gelu")
    x = np.array(c.arrays["inout"], np.float32)
    out = oracle.gelu(x)
    c.check(out, closed_form=lambda i: x[i] * 0.5 * (1.0 + math.erf(x[i] / math.sqrt(2.0))))


def test_layer_norm_vector(case):
    c = case(T + "op/LayerNormTest.cpp", "layer_norm_ext")
    out = oracle.layer_norm_(np.array(c.arrays["in"]).reshape(2, 3), np.array(c.arrays["inout"]).reshape(2, 3),
                             c.arrays["beta"], c.arrays["gamma"])
    assert c.check(out) == 6


def test_softmax_vector(case):
    c = case(T + "op/SoftmaxTest.cpp", "softmax_")
    out = oracle.softmax_(np.array(c.arrays["inout"]).reshape(2, 3))
    assert c.check(out) == 6


def test_attention_mask_vector(case):
    c = case(T + "op_att/AttentionMaskTest.cpp", "attention_mask")
    out = oracle.attention_mask(np.array(c.arrays["in"], np.int8).reshape(2, 2), heads=3)
    assert c.check(out) == 24


@pytest.mark.parametrize("blas,batch_parallel", [("builtin", True), ("best", True), ("best", False)])
def test_batch_matmul_vectors(case, blas, batch_parallel):
    """The pointer-array batch (one cblas_sgemm_batch group in the reference) with the builtin loop, as an OpenMP
    loop around single-threaded BLAS calls, and as one multi-threaded BLAS call per problem."""
    oracle.use_builtin_gemm() if blas == "builtin" else oracle.use_best_blas()
    oracle.set_batch_parallel(batch_parallel)
    try:
        c = case(T + "op_att/BatchMatMulTest.cpp", "q_k")
        out = oracle.att_q_k(c.arrays["query"], c.arrays["key"], 2, 2, 4, 3)
        assert c.check(out) == 32
        c = case(T + "op_att/BatchMatMulTest.cpp", "qk_v")
        out = oracle.att_qk_v(c.arrays["qk"], c.arrays["value"], 2, 2, 4, 3)
        assert c.check(out) == 48
        # the two batch modes are the same sgemm per problem: equal bits at a BERT-base head shape
        rng = np.random.default_rng(3)
        q, k = (rng.normal(size=(3 * 32 * 12 * 64)).astype(np.float32) for _ in range(2))
        a = oracle.att_q_k(q, k, 3, 32, 12, 64, alpha=0.125)
        oracle.set_batch_parallel(not batch_parallel)
        b = oracle.att_q_k(q, k, 3, 32, 12, 64, alpha=0.125)
        assert np.array_equal(a, b)
    finally:
        oracle.set_batch_parallel(True)
        oracle.use_best_blas()


def test_attention_self_vector(case):
    c = case(T + "op_att/AttentionSelfTest.cpp", "attention_self")
    w = {"attention/self/%s/%s" % (n, k): c.arrays["%s_%s" % (n, k)]
         for n in ("query", "key", "value") for k in ("kernel", "bias")}
    neg = np.zeros(64, np.float32)
    neg[0] = 1  # the test hands over an already-broadcast negative mask with one masked key
    out = oracle.attention_self(w, "attention/self", np.array(c.arrays["tensor"]).reshape(8, 6), neg, 2, 4, 2, 3)
    assert c.check(out) == 12


def transformer_weights(c, layers):
    names = {
        "attention/self/query/kernel": "query_kernel", "attention/self/query/bias": "query_bias",
        "attention/self/key/kernel": "key_kernel", "attention/self/key/bias": "key_bias",
        "attention/self/value/kernel": "value_kernel", "attention/self/value/bias": "value_bias",
        "attention/output/dense/kernel": "attention_output_kernel",
        "attention/output/dense/bias": "attention_output_bias",
        "attention/output/LayerNorm/beta": "attention_norm_beta",
        "attention/output/LayerNorm/gamma": "attention_norm_gamma",
        "intermediate/dense/kernel": "intermediate_kernel", "intermediate/dense/bias": "intermediate_bias",
        "output/dense/kernel": "output_kernel", "output/dense/bias": "output_bias",
        "output/LayerNorm/beta": "output_norm_beta", "output/LayerNorm/gamma": "output_norm_gamma",
    }
    return {"encoder/layer_%d/%s" % (l, k): np.array(c.arrays[v], np.float32)
            for l in range(layers) for k, v in names.items()}


@pytest.mark.parametrize("name,layers", [("transformer", 1), ("transformer_complex", 2)])
def test_transformer_vectors(case, name, layers):
    c = case(T + "op_att/TransformerTest.cpp", name)
    mask = np.ones((2, 4), np.int8)
    mask[0, 0] = 0
    for blas in ("builtin", "best"):
        oracle.use_builtin_gemm() if blas == "builtin" else oracle.use_best_blas()
        out = oracle.transformer(transformer_weights(c, layers), "encoder",
                                 np.array(c.arrays["tensor"]).reshape(8, 6), mask, 2, 4, 6, layers, 2, 5)
        assert c.check(out) == 12
    oracle.use_best_blas()


def test_bert_embeddings_vector(case):
    c = case(T + "op_bert/BertEmbeddingsTest.cpp", "bert_embedding")
    w = {"bert/embeddings/word_embeddings": np.array(c.arrays["word_embeddings"]).reshape(5, 3),
         "bert/embeddings/token_type_embeddings": np.array(c.arrays["token_type_embeddings"]).reshape(2, 3),
         "bert/embeddings/position_embeddings": np.array(c.arrays["position_embeddings"]).reshape(4, 3),
         "bert/embeddings/LayerNorm/beta": c.arrays["beta"], "bert/embeddings/LayerNorm/gamma": c.arrays["gamma"]}
    out = oracle.bert_embeddings(w, np.array(c.arrays["input_ids"]).reshape(2, 4),
                                 np.array(c.arrays["segment_ids"]).reshape(2, 4), 2, 4, 3)
    assert c.check(out) == 24


def test_pooler_vectors(case):
    c = case(T + "op_bert/BertPoolerTest.cpp", "bert_pooler")
    x = np.array(c.arrays["in"]).reshape(2, 3, 2)
    out = oracle.bert_pooler(np.array(c.arrays["kernel"]).reshape(2, 2), c.arrays["bias"], x)
    assert c.check(out) == 4
    c = case(T + "op_bert/BertPoolerTest.cpp", "mean_pooler")
    assert c.check(oracle.mean_pooler(np.array(c.arrays["in"]).reshape(2, 3, 2))) == 4


def test_classifier_vector(case):
    c = case(T + "op_out/AdditionalOutputLayerTest.cpp", "additional_output")
    logits, _ = oracle.classifier(np.array(c.arrays["output_weights"]).reshape(1, 3), None,
                                  np.array(c.arrays["in"]).reshape(2, 3), want_probs=False)
    assert c.check(logits) == 2


# ---------------------------------------------------------------- 2. reference launchers, bit for bit

needs_ref = pytest.mark.skipif(oracle.ref_ops() is None, reason="oracle/_ref not built (no reference checkout)")


@needs_ref
def test_primitives_match_reference_build_bitwise():
    rng = np.random.default_rng(7)
    x = rng.normal(0, 3, (37, 768)).astype(np.float32)
    y = rng.normal(0, 1, (37, 768)).astype(np.float32)
    beta = rng.normal(0, 1, 768).astype(np.float32)
    gamma = rng.normal(1, 0.1, 768).astype(np.float32)
    assert np.array_equal(oracle.layer_norm_(x, y, beta, gamma), oracle.layer_norm_(x, y, beta, gamma, use_ref=True))
    s = rng.normal(0, 4, (129, 33)).astype(np.float32)
    s[:, 5] -= 10000.0
    assert np.array_equal(oracle.softmax_(s), oracle.softmax_(s, use_ref=True))
    assert np.array_equal(oracle.gelu(x), oracle.gelu(x, use_ref=True))
    assert np.array_equal(oracle.tanh_(x), oracle.tanh_(x, use_ref=True))
    m = rng.integers(-2, 3, 500).astype(np.int8)
    assert np.array_equal(oracle.not_(m), oracle.not_(m, use_ref=True))
    z = rng.normal(0, 1, (5, 17, 24)).astype(np.float32)
    assert np.array_equal(oracle.reduce_mean_1(z), oracle.reduce_mean_1(z, use_ref=True))
    table = rng.normal(0, 1, (50, 24)).astype(np.float32)
    ids = rng.integers(0, 50, 99).astype(np.int32)
    assert np.array_equal(oracle.embedding(ids, table), oracle.embedding(ids, table, use_ref=True))
    seg = rng.integers(0, 2, 99).astype(np.int8)
    assert np.array_equal(oracle.embedding(seg, table), oracle.embedding(seg, table, use_ref=True))


@needs_ref
def test_reference_build_reproduces_its_own_vectors(case):
    c = case(T + "op/LayerNormTest.cpp", "layer_norm_ext")
    out = oracle.layer_norm_(np.array(c.arrays["in"]).reshape(2, 3), np.array(c.arrays["inout"]).reshape(2, 3),
                             c.arrays["beta"], c.arrays["gamma"], use_ref=True)
    c.check(out)
    c = case(T + "op/SoftmaxTest.cpp", "softmax_")
    c.check(oracle.softmax_(np.array(c.arrays["inout"]).reshape(2, 3), use_ref=True))


# ---------------------------------------------------------------- 3. what the mathematics fixes

def ln64(x, beta, gamma):
    x = x.astype(np.float64)
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + 1e-12) * gamma + beta


def gelu64(x):
    from scipy.special import erf
    return x * 0.5 * (1.0 + erf(x / np.sqrt(2.0)))


def softmax64(x):
    from scipy.special import softmax
    return softmax(x.astype(np.float64), axis=-1)


def test_sgemm_against_float64_all_transposes():
    rng = np.random.default_rng(3)
    M, N, K = 7, 5, 11
    for blas in ("builtin", "best"):
        oracle.use_builtin_gemm() if blas == "builtin" else oracle.use_best_blas()
        for ta in (0, 1):
            for tb in (0, 1):
                # column-major storage: A is (M x K) or (K x M) with padding in the leading dimension
                lda, ldb, ldc = (K if ta else M) + 2, (N if tb else K) + 3, M + 1
                A = rng.normal(size=lda * (M if ta else K)).astype(np.float32)
                B = rng.normal(size=ldb * (K if tb else N)).astype(np.float32)
                C = rng.normal(size=ldc * N).astype(np.float32)
                Am = A.reshape(-1, lda).T[: (K if ta else M)]
                Bm = B.reshape(-1, ldb).T[: (N if tb else K)]
                opA = Am.T if ta else Am
                opB = Bm.T if tb else Bm
                want = 0.5 * opA.astype(np.float64) @ opB.astype(np.float64) + 2.0 * C.reshape(N, ldc).T[:M]
                got = oracle.sgemm(ta, tb, M, N, K, 0.5, A, lda, B, ldb, 2.0, C.copy(), ldc).reshape(N, ldc).T[:M]
                np.testing.assert_allclose(got, want, rtol=0, atol=2e-5)
    oracle.use_best_blas()


def test_layer_norm_textbook():
    rng = np.random.default_rng(0)
    a = rng.normal(0.3, 2, (64, 768)).astype(np.float32)
    b = rng.normal(0, 1, (64, 768)).astype(np.float32)
    beta = rng.normal(0, 1, 768).astype(np.float32)
    gamma = rng.normal(1, 0.2, 768).astype(np.float32)
    got = oracle.layer_norm_(a, b, beta, gamma)
    want = ln64(a.astype(np.float64) + b, beta, gamma)
    np.testing.assert_allclose(got, want, atol=2e-5, rtol=0)
    # gamma = 1: the output row mean is mean(beta)
    got1 = oracle.layer_norm_(a, b, beta, np.ones(768))
    np.testing.assert_allclose(got1.mean(-1), beta.mean(), atol=1e-5)


def test_softmax_gelu_textbook():
    rng = np.random.default_rng(1)
    x = rng.normal(0, 5, (100, 77)).astype(np.float32)
    got = oracle.softmax_(x)
    np.testing.assert_allclose(got, softmax64(x), atol=1e-6)
    np.testing.assert_allclose(got.sum(-1), 1.0, atol=1e-5)
    g = rng.normal(0, 3, 10000).astype(np.float32)
    np.testing.assert_allclose(oracle.gelu(g), gelu64(g.astype(np.float64)), atol=1e-6)


def np_bert64(w, ids, mask, seg, layers, heads):
    """Independent float64 BERT written from the textbook (row-major matmuls, einsum attention)."""
    f = lambda k: np.asarray(w[k], np.float64)
    B, S = ids.shape
    H = f("bert/embeddings/word_embeddings").shape[1]
    d = H // heads
    x = (f("bert/embeddings/word_embeddings")[ids] + f("bert/embeddings/position_embeddings")[:S][None]
         + f("bert/embeddings/token_type_embeddings")[seg])
    x = ln64(x, f("bert/embeddings/LayerNorm/beta"), f("bert/embeddings/LayerNorm/gamma"))
    emb = x
    adder = (mask == 0)[:, None, None, :] * -10000.0
    for l in range(layers):
        p = "bert/encoder/layer_%d/" % l
        q = (x @ f(p + "attention/self/query/kernel") + f(p + "attention/self/query/bias")).reshape(B, S, heads, d)
        k = (x @ f(p + "attention/self/key/kernel") + f(p + "attention/self/key/bias")).reshape(B, S, heads, d)
        v = (x @ f(p + "attention/self/value/kernel") + f(p + "attention/self/value/bias")).reshape(B, S, heads, d)
        s = np.einsum("bqhd,bkhd->bhqk", q, k) / math.sqrt(d) + adder
        pr = softmax64(s)
        ctx = np.einsum("bhqk,bkhd->bqhd", pr, v).reshape(B, S, H)
        a = ctx @ f(p + "attention/output/dense/kernel") + f(p + "attention/output/dense/bias")
        a = ln64(a + x, f(p + "attention/output/LayerNorm/beta"), f(p + "attention/output/LayerNorm/gamma"))
        i = gelu64(a @ f(p + "intermediate/dense/kernel") + f(p + "intermediate/dense/bias"))
        o = i @ f(p + "output/dense/kernel") + f(p + "output/dense/bias")
        x = ln64(o + a, f(p + "output/LayerNorm/beta"), f(p + "output/LayerNorm/gamma"))
    out = {"embedding_output": emb, "sequence_output": x}
    if "bert/pooler/dense/kernel" in w:
        out["pooled_output"] = np.tanh(x[:, 0] @ f("bert/pooler/dense/kernel") + f("bert/pooler/dense/bias"))
    else:
        out["pooled_output"] = x.mean(1)
    if "output_weights" in w:
        lg = out["pooled_output"] @ f("output_weights").T
        if "output_bias" in w:
            lg = lg + f("output_bias")
        out["logits"] = lg
        out["probs"] = softmax64(lg)
    return out


@pytest.mark.parametrize("pooler,bias", [(True, True), (False, False), (True, False)])
def test_bert_forward_against_float64_textbook(pooler, bias):
    from cubert_amd.testing import random_bert_weights, random_inputs
    cfg = dict(vocab=97, hidden=48, layers=3, heads=4, intermediate=80, max_position=40, type_vocab=2, labels=3)
    w = random_bert_weights(seed=11, pooler=pooler, classifier=True, classifier_bias=bias, ln_random=True, **cfg)
    ids, mask, seg = random_inputs(seed=5, batch=5, seq_length=24, vocab=97, min_valid=3, scattered_mask=True)
    got = oracle.bert_forward(w, ids, mask, seg, layers=3, heads=4)
    want = np_bert64(w, ids, mask, seg, 3, 4)
    for k in want:
        np.testing.assert_allclose(got[k], want[k], atol=3e-5, rtol=0, err_msg=k)


def test_half_rounding_matches_numpy():
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.normal(0, 0.02, 5000), rng.normal(0, 300, 2000), [0.0, -0.0, 65504, 65519.9, 65520, 1e-8,
                        2.0 ** -25, 2.0 ** -24, 6e-8, 6.1e-5, 1 + 2.0 ** -11, 1 + 3 * 2.0 ** -11]]).astype(np.float32)
    want = x.astype(np.float16).astype(np.float32)
    np.testing.assert_array_equal(oracle.round_to_half(x), want)
