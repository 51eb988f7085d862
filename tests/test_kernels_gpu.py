"""Parity of every fused kernel, called through the C ABI (include/cubert_kernels.h),
against the CPU oracle on the same seeded inputs, plus the known-answer vectors of the
reference's unit tests and the edge cases it covers.  fp32: 1e-5 relative (norm-wise);
fp16 storage: compared with the oracle run on the fp16-rounded inputs, within fp16
output rounding (2e-3 relative)."""
import math

import numpy as np
import pytest

import oracle
from util import FP32_TOL, assert_close

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
T = "test/cuBERT/"
F16_KERNEL_TOL = 2e-3


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.fail("no GPU visible: the -m gpu tests must run on the MI355X box")
    from cubert_amd import kernels
    return kernels


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def host(t):
    torch.cuda.synchronize()
    return t.float().cpu().numpy()


def tdt(name):
    return torch.float32 if name == "f32" else torch.float16


def q(a, name):
    """The values the kernel actually sees: fp32, or fp32 rounded to fp16 and back."""
    a = np.asarray(a, np.float32)
    return a if name == "f32" else oracle.round_to_half(a)


def tol(name):
    return FP32_TOL if name == "f32" else F16_KERNEL_TOL


# ------------------------------------------------------------------ reference vectors

def test_layer_norm_reference_vector(K, case):
    c = case(T + "op/LayerNormTest.cpp", "layer_norm_ext")
    inout = dev(np.array(c.arrays["inout"], np.float32).reshape(2, 3))
    K.bias_res_ln_(inout, dev(np.array(c.arrays["in"], np.float32).reshape(2, 3)), None,
                   dev(np.array(c.arrays["beta"], np.float32)), dev(np.array(c.arrays["gamma"], np.float32)))
    c.check(host(inout))


def test_softmax_reference_vector(K, case):
    c = case(T + "op/SoftmaxTest.cpp", "softmax_")
    x = dev(np.array(c.arrays["inout"], np.float32).reshape(2, 3))
    c.check(host(K.row_softmax(x)))
    # the same rows through the attention kernel (square score matrix, no mask, scale 1)
    s3 = torch.zeros((1, 1, 3, 3), device="cuda")
    s3[0, 0, :2] = x
    K.mask_scale_softmax_(s3, None, 1.0)
    c.check(host(s3)[0, 0, :2])


def test_gelu_reference_vector(K, case):
    c = case(T + "op/GELUTest.cpp", "gelu")
    x = np.array(c.arrays["inout"], np.float32)
    y = dev(x.reshape(1, 5).copy())
    K.bias_gelu_(y, None)
    c.check(host(y), closed_form=lambda i: x[i] * 0.5 * (1.0 + math.erf(x[i] / math.sqrt(2.0))))


def test_embedding_reference_vector(K, case):
    c = case(T + "op/EmbeddingTest.cpp", "embedding")
    out = K.gather(dev(np.array(c.arrays["input_ids"], np.int32)),
                   dev(np.array(c.arrays["embedding_table"], np.float32).reshape(4, 3)))
    c.check(host(out))


def test_bert_embeddings_reference_vector(K, case):
    c = case(T + "op_bert/BertEmbeddingsTest.cpp", "bert_embedding")
    f = lambda k, *s: dev(np.array(c.arrays[k], np.float32).reshape(*s))
    out = K.embed_ln(dev(np.array(c.arrays["input_ids"], np.int32).reshape(2, 4)),
                     dev(np.array(c.arrays["segment_ids"], np.int8).reshape(2, 4)),
                     f("word_embeddings", 5, 3), f("position_embeddings", 4, 3), f("token_type_embeddings", 2, 3),
                     f("beta", 3), f("gamma", 3))
    c.check(host(out))


def test_pooler_reference_vectors(K, case):
    c = case(T + "op_bert/BertPoolerTest.cpp", "bert_pooler")
    x = dev(np.array(c.arrays["in"], np.float32).reshape(2, 3, 2))
    kernel = dev(np.array(c.arrays["kernel"], np.float32).reshape(2, 2))
    out = torch.zeros((2, 2), device="cuda")
    blas = K.Blas()
    # first token of each sequence: ldb = hidden * seq_length, as the reference's pooler GEMM
    blas.gemm(False, False, 2, 2, 2, 1.0, kernel, 2, x, 2 * 3, 0.0, out, 2)
    K.bias_tanh_(out, dev(np.array(c.arrays["bias"], np.float32)))
    c.check(host(out))
    c = case(T + "op_bert/BertPoolerTest.cpp", "mean_pooler")
    c.check(host(K.mean_pool(dev(np.array(c.arrays["in"], np.float32).reshape(2, 3, 2)))))


def test_dense_reference_vector(K, case):
    c = case(T + "op/DenseTest.cpp", "dense")
    kernel = dev(np.array(c.arrays["kernel"], np.float32))
    x = dev(np.array(c.arrays["input"], np.float32))
    out = torch.zeros(9, device="cuda")
    K.Blas().gemm(False, False, 3, 3, 2, 1.0, kernel, 3, x, 2, 0.0, out, 3, bias=dev(np.array(c.arrays["bias"], np.float32)))
    c.check(host(out))


def test_attention_mask_reference_vector(K, case):
    """AttentionMaskTest pins neg = !mask broadcast over heads and queries.  The fused kernel never
    materialises that tensor; what it must reproduce is its effect: with all scores zero, keys with
    neg = 1 get the -10000 addend, i.e. probability exp(-10000) = 0 unless every key of the row is masked."""
    c = case(T + "op_att/AttentionMaskTest.cpp", "attention_mask")
    mask = np.array(c.arrays["in"], np.int8).reshape(2, 2)
    neg = np.array([v for _, _, v, _ in c.expect], np.float32).reshape(2, 3, 2, 2)  # [b, a, q, k]
    scores = torch.zeros((2, 3, 2, 2), device="cuda")
    K.mask_scale_softmax_(scores, dev(mask), 1.0)
    want = oracle.softmax_((-10000.0 * neg).reshape(-1, 2)).reshape(2, 3, 2, 2)
    np.testing.assert_allclose(host(scores), want, atol=1e-7)
    assert host(scores)[0, :, :, 0].min() == 1.0 and host(scores)[0, :, :, 1].max() == 0.0
    np.testing.assert_allclose(host(scores)[1], 0.5)  # fully masked rows stay uniform


def test_batch_matmul_reference_vectors(K, case):
    """QK^T and PV layouts of BatchMatMulTest through the strided-batched GEMM, both loop orders."""
    blas = K.Blas()
    S, A, d, B = 2, 4, 3, 2
    H = A * d
    c = case(T + "op_att/BatchMatMulTest.cpp", "q_k")
    qh, kh = np.array(c.arrays["query"], np.float32), np.array(c.arrays["key"], np.float32)
    want = oracle.att_q_k(qh, kh, B, S, A, d)  # [B, S_q, A, S_k], pinned by the oracle test
    c.check(want)
    q_, k_ = dev(qh), dev(kh)
    for loop_heads in (True, False):
        out = torch.zeros(B * A * S * S, device="cuda")  # [B, A, S_q, S_k]
        if loop_heads:
            for a in range(A):
                blas.gemm_strided_batch(True, False, S, S, d, 1.0, k_[a * d:], H, S * H, q_[a * d:], H, S * H, 0.0,
                                        out[a * S * S:], S, A * S * S, B)
        else:
            for b in range(B):
                blas.gemm_strided_batch(True, False, S, S, d, 1.0, k_[b * S * H:], H, d, q_[b * S * H:], H, d, 0.0,
                                        out[b * A * S * S:], S, S * S, A)
        got = host(out).reshape(B, A, S, S).transpose(0, 2, 1, 3)
        np.testing.assert_array_equal(got, want)
    c = case(T + "op_att/BatchMatMulTest.cpp", "qk_v")
    p_h, v_h = np.array(c.arrays["qk"], np.float32), np.array(c.arrays["value"], np.float32)
    want = oracle.att_qk_v(p_h, v_h, B, S, A, d)
    c.check(want)
    p_ = dev(np.ascontiguousarray(p_h.reshape(B, S, A, S).transpose(0, 2, 1, 3)))  # ours: [B, A, S_q, S_k]
    v_ = dev(v_h)
    out = torch.zeros(B * S * H, device="cuda")
    for a in range(A):
        blas.gemm_strided_batch(False, False, d, S, S, 1.0, v_[a * d:], H, S * H, p_.reshape(-1)[a * S * S:], S,
                                A * S * S, 0.0, out[a * d:], H, S * H, B)
    np.testing.assert_array_equal(host(out).reshape(B, S, A, d), want)


def test_batch_matmul_reference_vectors_pointer_arrays(K, case):
    """The same vectors through blas_gemm_batch's interface, called as the reference's Att_Q_K / Att_QK_V call it
    (src/cuBERT/op_att/BatchMatMul.cpp:31-38,57-68,103-110,129-140): one pointer per (batch, head) into the
    [B, S, A, d] operands, scores laid out [B, S_q, A, S_k] as in the reference."""
    blas = K.Blas()
    S, A, d, B = 2, 4, 3, 2
    H = A * d
    c = case(T + "op_att/BatchMatMulTest.cpp", "q_k")
    q_, k_ = dev(np.array(c.arrays["query"], np.float32)), dev(np.array(c.arrays["key"], np.float32))
    out = torch.full((B * S * A * S,), 7.0, device="cuda")
    problems = [(b, h) for b in range(B) for h in range(A)]
    idx = lambda b, h: b * S * d * A + d * h
    blas.gemm_batch(True, False, S, S, d, 1.0, [k_[idx(b, h):] for b, h in problems], H,
                    [q_[idx(b, h):] for b, h in problems], H, 0.0,
                    [out[b * S * S * A + S * h:] for b, h in problems], S * A)
    c.check(host(out))
    c = case(T + "op_att/BatchMatMulTest.cpp", "qk_v")
    p_, v_ = dev(np.array(c.arrays["qk"], np.float32)), dev(np.array(c.arrays["value"], np.float32))
    out = torch.full((B * S * H,), 7.0, device="cuda")
    blas.gemm_batch(False, False, d, S, S, 1.0, [v_[idx(b, h):] for b, h in problems], H,
                    [p_[b * S * S * A + S * h:] for b, h in problems], S * A, 0.0,
                    [out[idx(b, h):] for b, h in problems], H)
    c.check(host(out))


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("M,N,K_,batch", [(32, 32, 64, 24), (64, 128, 128, 5), (70, 65, 19, 3), (1, 1, 1, 2),
                                          (128, 128, 64, 7), (5, 200, 33, 4)])
@pytest.mark.parametrize("padded", [True, False])
def test_gemm_batch_against_oracle_sgemm(K, name, ta, tb, M, N, K_, batch, padded):
    """blas_gemm_batch (arrays of pointers, column-major, all transposes, alpha / beta, tile edges) against the
    oracle's sgemm problem by problem; leading dimensions padded by odd amounts (element accesses) and exact (the
    16-byte accesses of the matrix-core kernel that shapes of whole 32 x 32 x 32 tiles take)."""
    rng = np.random.default_rng(M * 31 + N * 7 + K_ + batch + 2 * ta + tb)
    lda, ldb, ldc = (K_ if ta else M), (N if tb else K_), M
    if padded:
        lda, ldb, ldc = lda + 3, ldb + 2, ldc + 1
    a_cols, b_cols = (M if ta else K_), (K_ if tb else N)
    As = [q(rng.normal(0, 1, lda * a_cols), name) for _ in range(batch)]
    Bs = [q(rng.normal(0, 1, ldb * b_cols), name) for _ in range(batch)]
    C0 = [q(rng.normal(0, 1, ldc * N), name) for _ in range(batch)]
    blas = K.Blas()
    dA, dB = [dev(a, tdt(name)) for a in As], [dev(b, tdt(name)) for b in Bs]
    for alpha, beta in ((1.0, 0.0), (0.5, 1.0), (1.0, -0.25)):
        dC = [dev(c0, tdt(name)) for c0 in C0]
        blas.gemm_batch(ta, tb, M, N, K_, alpha, dA, lda, dB, ldb, beta, dC, ldc)
        for z in range(batch):
            want = oracle.sgemm(ta, tb, M, N, K_, alpha, As[z], lda, Bs[z], ldb, beta, C0[z].copy(), ldc)
            got = host(dC[z])
            live = (np.arange(ldc * N) % ldc) < M  # the padding rows of C are not written
            np.testing.assert_array_equal(got[~live], C0[z][~live])
            assert_close(got[live], want[live], 2e-5 if name == "f32" else 2e-3,
                         "gemm_batch %s problem %d alpha=%g beta=%g" % (name, z, alpha, beta))


# ------------------------------------------------------------------ seeded parity with the oracle

@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("rows,hidden", [(4096, 768), (1000, 1024), (37, 768), (5, 256), (64, 1280), (3, 6), (9, 100),
                                         (2, 4096), (7, 384), (1, 768), (2, 768)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_bias_res_ln(K, name, rows, hidden, with_bias):
    rng = np.random.default_rng(rows * 7 + hidden)
    x = q(rng.normal(0.2, 1.5, (rows, hidden)), name)
    res = q(rng.normal(0, 1, (rows, hidden)), name)
    bias = q(rng.normal(0, 0.5, hidden), name)
    beta = q(rng.normal(0, 0.3, hidden), name)
    gamma = q(rng.normal(1, 0.2, hidden), name)
    inout = dev(x, tdt(name))
    K.bias_res_ln_(inout, dev(res, tdt(name)), dev(bias, tdt(name)) if with_bias else None, dev(beta, tdt(name)),
                   dev(gamma, tdt(name)))
    # the reference adds the bias into the GEMM output first, then LayerNorm adds the residual
    pre = x + bias if with_bias else x
    want = oracle.layer_norm_(res, pre, beta, gamma)
    assert_close(host(inout), want, tol(name), "bias_res_ln %s" % name)


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("batch,seq,hidden,vocab", [(128, 32, 768, 21128), (3, 128, 1024, 3000), (2, 4, 6, 11),
                                                    (1, 512, 768, 21128), (5, 7, 100, 50), (5, 7, 768, 50),
                                                    (3, 3, 384, 20), (1, 1, 768, 9)])
def test_embed_ln(K, name, batch, seq, hidden, vocab):
    rng = np.random.default_rng(batch + seq + hidden)
    w = {"bert/embeddings/word_embeddings": q(rng.normal(0, 0.02, (vocab, hidden)), name),
         "bert/embeddings/token_type_embeddings": q(rng.normal(0, 0.02, (2, hidden)), name),
         "bert/embeddings/position_embeddings": q(rng.normal(0, 0.02, (seq, hidden)), name),
         "bert/embeddings/LayerNorm/beta": q(rng.normal(0, 0.1, hidden), name),
         "bert/embeddings/LayerNorm/gamma": q(rng.normal(1, 0.1, hidden), name)}
    ids = rng.integers(0, vocab, (batch, seq), dtype=np.int32)
    ids[0, 0], ids[-1, -1] = 0, vocab - 1
    seg = rng.integers(0, 2, (batch, seq)).astype(np.int8)
    d = lambda k: dev(w["bert/embeddings/" + k], tdt(name))
    out = K.embed_ln(dev(ids), dev(seg), d("word_embeddings"), d("position_embeddings"), d("token_type_embeddings"),
                     d("LayerNorm/beta"), d("LayerNorm/gamma"))
    want = oracle.bert_embeddings(w, ids, seg, batch, seq, hidden).reshape(batch, seq, hidden)
    assert_close(host(out), want, tol(name), "embed_ln %s" % name)


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("rows,width", [(4096, 3072), (512, 4096), (3, 3072), (7, 5), (33, 72), (1, 8)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_bias_gelu(K, name, rows, width, with_bias):
    rng = np.random.default_rng(rows + width)
    x = q(rng.normal(0, 2.5, (rows, width)), name)
    x.ravel()[:6] = q(np.array([-12, -6, -0.0, 0.0, 6, 12]), name)[: min(6, x.size)]
    bias = q(rng.normal(0, 0.5, width), name)
    y = dev(x, tdt(name))
    K.bias_gelu_(y, dev(bias, tdt(name)) if with_bias else None)
    want = oracle.gelu(x + bias if with_bias else x)
    assert_close(host(y), want, tol(name), "bias_gelu %s" % name)


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("batch,heads,seq", [(128, 12, 32), (8, 12, 128), (2, 12, 512), (2, 2, 4), (3, 5, 7),
                                             (2, 3, 384), (1, 16, 64), (2, 4, 8), (2, 2, 1024), (1, 2, 100)])
def test_mask_scale_softmax(K, name, batch, heads, seq):
    rng = np.random.default_rng(batch * 131 + heads * 17 + seq)
    raw = q(rng.normal(0, 6, (batch, heads, seq, seq)), name)
    valid = rng.integers(1, seq + 1, batch)
    mask = (np.arange(seq)[None, :] < valid[:, None]).astype(np.int8)
    mask[0] = (rng.random(seq) < 0.5)  # a scattered pattern, and values other than 1
    mask[0, rng.integers(0, seq)] = 3
    scale = 0.125
    s = dev(raw, tdt(name))
    K.mask_scale_softmax_(s, dev(mask), scale)
    neg = oracle.not_(mask)  # 1.0 where the key is masked
    logits = raw * np.float32(scale) + np.float32(-10000.0) * neg[:, None, None, :]
    want = oracle.softmax_(logits.reshape(-1, seq)).reshape(raw.shape)
    got = host(s)
    assert_close(got, want, tol(name), "mask_scale_softmax %s" % name)
    np.testing.assert_allclose(got.sum(-1), 1.0, atol=1e-5 if name == "f32" else 4e-3)
    assert got[0][:, :, mask[0] == 0].max() == 0.0  # masked keys get exactly zero probability


@pytest.mark.parametrize("name", ["f32", "f16"])
def test_mask_special_cases(K, name):
    rng = np.random.default_rng(0)
    raw = q(rng.normal(0, 3, (2, 2, 32, 32)), name)
    ones = np.ones((2, 32), np.int8)
    plain = oracle.softmax_(raw.reshape(-1, 32)).reshape(raw.shape)
    a = dev(raw, tdt(name)); K.mask_scale_softmax_(a, dev(ones), 1.0)      # all kept = plain softmax
    b = dev(raw, tdt(name)); K.mask_scale_softmax_(b, None, 1.0)           # no mask at all
    assert_close(host(a), plain, tol(name))
    assert np.array_equal(host(a), host(b))
    # every key masked: the -10000 shift cancels up to fp32 rounding at magnitude 1e4
    z = dev(raw, tdt(name)); K.mask_scale_softmax_(z, dev(np.zeros((2, 32), np.int8)), 1.0)
    want = oracle.softmax_((raw - np.float32(10000.0)).reshape(-1, 32)).reshape(raw.shape)
    assert_close(host(z), want, tol(name))


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("rows,channel", [(128, 2), (256, 3), (1, 1), (77, 16), (40, 33), (5, 1000)])
def test_row_softmax(K, name, rows, channel):
    rng = np.random.default_rng(rows + channel)
    x = q(rng.normal(0, 4, (rows, channel)), name)
    got = host(K.row_softmax(dev(x, tdt(name))))
    assert_close(got, oracle.softmax_(x), tol(name), "row_softmax")


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("rows,width", [(128, 768), (256, 1024), (1, 768), (3, 5)])
def test_bias_tanh(K, name, rows, width):
    rng = np.random.default_rng(rows + width)
    x = q(rng.normal(0, 2, (rows, width)), name)
    bias = q(rng.normal(0, 0.5, width), name)
    y = dev(x, tdt(name))
    K.bias_tanh_(y, dev(bias, tdt(name)))
    assert_close(host(y), oracle.tanh_(x + bias), tol(name), "bias_tanh")


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("batch,seq,hidden", [(32, 128, 768), (4, 512, 1024), (2, 3, 2), (3, 5, 100), (1, 1, 768)])
def test_mean_pool(K, name, batch, seq, hidden):
    rng = np.random.default_rng(batch + seq + hidden)
    x = q(rng.normal(0.1, 1, (batch, seq, hidden)), name)
    got = host(K.mean_pool(dev(x, tdt(name))))
    assert_close(got, oracle.reduce_mean_1(x), tol(name), "mean_pool")


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("idt", [np.int32, np.int8])
def test_gather(K, name, idt):
    rng = np.random.default_rng(1)
    table = q(rng.normal(0, 1, (100, 768)), name)
    ids = rng.integers(0, 100, 333).astype(idt)
    got = host(K.gather(dev(ids), dev(table, tdt(name))))
    assert np.array_equal(got, oracle.embedding(ids, table))  # a copy: bit exact


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("batch,hidden,labels,tanh,bias", [(1, 768, 2, True, True), (128, 768, 2, True, True),
                                                          (5, 1024, 3, False, True), (7, 100, 1, True, False),
                                                          (3, 768, 64, True, True)])
def test_classifier_head(K, name, batch, hidden, labels, tanh, bias):
    """Pooler bias + tanh, classifier and softmax in one launch against the oracle's tanh_, sgemm (W^T) and
    softmax_ and against this library's three separate kernels."""
    rng = np.random.default_rng(batch + hidden + labels)
    dt = tdt(name)
    x = q(rng.normal(0, 1, (batch, hidden)), name)
    pb = q(rng.normal(0, 0.5, hidden), name)
    W = q(rng.normal(0, 0.1, (labels, hidden)), name)
    ob = q(rng.normal(0, 1, labels), name) if bias else None
    pooled = dev(x, dt)
    out = K.classifier_head_(pooled, dev(pb, dt) if tanh else None, dev(W, dt), None if ob is None else dev(ob, dt))
    assert out is not None
    logits, probs = out
    want_pooled = np.tanh((x + pb[None, :]).astype(np.float32)) if tanh else x
    if name == "f16":
        want_pooled = oracle.round_to_half(want_pooled)
    t = tol(name)
    assert_close(host(pooled), want_pooled, t, "pooled")
    want_logits = host(pooled) @ W.T + (0 if ob is None else ob[None, :])
    if name == "f16":
        want_logits = oracle.round_to_half(want_logits.astype(np.float32))
    assert_close(host(logits), want_logits, 2e-5 if name == "f32" else 2e-3, "logits")
    want_probs = oracle.softmax_(np.ascontiguousarray(host(logits), dtype=np.float32))
    assert_close(host(probs), want_probs, 2e-5 if name == "f32" else 2e-3, "probs")
    np.testing.assert_allclose(host(probs).sum(-1), 1.0, atol=1e-5 if name == "f32" else 2e-3)
    # the three separate kernels
    p3 = dev(x, dt)
    if tanh:
        K.bias_tanh_(p3, dev(pb, dt))
    assert_close(host(pooled), host(p3), 1e-6 if name == "f32" else 1e-3, "pooled vs bias_tanh")
    s3 = K.row_softmax(logits)
    assert_close(host(probs), host(s3), 1e-6 if name == "f32" else 1e-3, "probs vs row_softmax")


def test_classifier_head_declines_many_labels(K):
    z = torch.zeros
    assert K.classifier_head_(z((2, 64), device="cuda"), None, z((65, 64), device="cuda"), None) is None


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("rows,cols", [(768, 2304), (3072, 768), (33, 65), (1, 7), (100, 1), (32, 32)])
def test_transpose(K, name, rows, cols):
    x = q(np.random.default_rng(rows + cols).normal(0, 1, (rows, cols)), name)
    got = host(K.transpose(dev(x, tdt(name))))
    assert got.shape == (cols, rows) and np.array_equal(got, x.T)  # a copy: bit exact


# ------------------------------------------------------------------ fp32 Dense on the fp16 matrix cores (opt-in form)

def two_terms(x):
    """numpy's statement of the split: hi = fp16(x), lo = fp16(x - hi), both round-to-nearest-even."""
    x = np.asarray(x, np.float32)
    hi = x.astype(np.float16)
    lo = (x - hi.astype(np.float32)).astype(np.float16)
    return hi, lo


@pytest.mark.parametrize("rows,width", [(64, 768), (33, 3072), (5, 24), (3, 7), (1, 1), (16, 8)])
@pytest.mark.parametrize("lo_in_middle", [False, True])
def test_split3_bit_exact(K, rows, width, lo_in_middle):
    rng = np.random.default_rng(rows * 7 + width)
    x = rng.normal(0, 1, (rows, width)).astype(np.float32)
    x.flat[::5] *= 1e-4   # lo parts in the fp16 subnormals
    x.flat[::7] *= 300.0
    x.flat[0] = 70000.0   # beyond fp16: hi saturates at 65504, lo carries the rest
    scale = 4.0
    got = K.split3(dev(x), scale, lo_in_middle)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    clipped = np.clip(x * np.float32(scale), -65504, 65504)
    hi = clipped.astype(np.float16)
    lo = np.clip(x * np.float32(scale) - hi.astype(np.float32), -65504, 65504).astype(np.float16)
    parts = [hi, lo, hi] if lo_in_middle else [hi, hi, lo]
    assert got.dtype == np.float16 and got.shape == (rows, 3 * width)
    for i, part in enumerate(parts):
        assert np.array_equal(got[:, i * width:(i + 1) * width].view(np.uint16), part.view(np.uint16)), i
    # the two terms carry the value to 2^-22 relative (2^-25 absolute once lo is subnormal)
    back = hi.astype(np.float64) + lo.astype(np.float64)
    want = (x * np.float32(scale)).astype(np.float64)
    ok = np.abs(want) <= 65504
    assert np.all(np.abs(back - want)[ok] <= np.maximum(np.abs(want)[ok] * 2.0 ** -22, 2.0 ** -25))


@pytest.mark.parametrize("rows,width", [(40, 3072), (7, 512), (3, 20), (2, 5)])
def test_bias_gelu_split3_against_oracle(K, rows, width):
    rng = np.random.default_rng(width)
    x = (rng.normal(0, 2, (rows, width))).astype(np.float32)
    b = rng.normal(0, 0.5, width).astype(np.float32)
    got = K.bias_gelu_split3(dev(x), dev(b), 16.0)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert np.array_equal(got[:, :width].view(np.uint16), got[:, width:2 * width].view(np.uint16))
    value = (got[:, :width].astype(np.float64) + got[:, 2 * width:].astype(np.float64)) / 16
    want = oracle.gelu(x + b)
    assert_close(value, want, FP32_TOL, "two-term GELU")
    # and against the in-place kernel, to the resolution of the two terms
    inplace = host(K.bias_gelu_(dev(x), dev(b))).astype(np.float64)
    assert np.all(np.abs(value - inplace) <= np.maximum(np.abs(inplace) * 2.0 ** -21, 2.0 ** -24))


@pytest.mark.parametrize("rows,hidden,with_bias", [(37, 768, True), (5, 1024, False), (4, 256, True), (3, 2048, True)])
def test_bias_res_ln_split3_equals_ln_then_split(K, rows, hidden, with_bias):
    rng = np.random.default_rng(hidden + rows)
    x = rng.normal(0, 1, (rows, hidden)).astype(np.float32)
    res = rng.normal(0, 1, (rows, hidden)).astype(np.float32)
    bias = rng.normal(0, 0.1, hidden).astype(np.float32) if with_bias else None
    beta = rng.normal(0, 0.1, hidden).astype(np.float32)
    gamma = rng.normal(1, 0.1, hidden).astype(np.float32)
    args = [dev(res), None if bias is None else dev(bias), dev(beta), dev(gamma)]
    plain = K.bias_res_ln_(dev(x), *args)
    want_split = K.split3(plain, 16.0)
    inout = dev(x)
    got_split = K.bias_res_ln_split3_(inout, *args, scale=16.0)
    assert got_split is not None
    torch.cuda.synchronize()
    assert torch.equal(inout, plain)             # the fp32 result is the plain kernel's, bit for bit
    assert torch.equal(got_split, want_split)    # and its two-term rows are those of the split kernel
    assert_close(host(inout), oracle.layer_norm_(res, x + (0 if bias is None else bias), beta, gamma), FP32_TOL, "LN")


@pytest.mark.parametrize("batch,heads,seq,d", [(1, 12, 32, 64), (24, 12, 32, 64), (3, 4, 128, 64), (2, 3, 64, 32),
                                               (1, 2, 256, 64), (2, 2, 96, 128), (1, 2, 512, 64)])
def test_attention_fused_split3_equals_attention_then_split(K, batch, heads, seq, d):
    rng = np.random.default_rng(batch + heads + seq + d)
    H = heads * d
    qkv = dev(rng.normal(0, 1, (batch * seq, 3 * H)).astype(np.float32))
    mask = (rng.random((batch, seq)) < 0.7).astype(np.int8)
    mask[:, 0] = 1
    mask = dev(mask)
    alpha = 1.0 / math.sqrt(d)
    plain = K.attention_fused(qkv, mask, batch, heads, seq, d, alpha)
    assert plain is not None
    got = K.attention_fused_split3(qkv, mask, batch, heads, seq, d, alpha, scale=16.0)
    assert got is not None
    torch.cuda.synchronize()
    assert torch.equal(got, K.split3(plain, 16.0))  # the same context values, written in the other form


def test_two_term_kernels_raise_the_overflow_flag(K):
    """A value whose scaled form is beyond the fp16 range (or is not a number) cannot be written as two fp16 terms:
    each of the four kernels that write two-term rows stores 1 to the caller's flag then, and leaves it alone
    otherwise (the host classes recompute such a request with the fp32 GEMMs)."""
    rng = np.random.default_rng(5)
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")

    def raised():
        torch.cuda.synchronize()
        v = int(flag.item())
        flag.zero_()
        return v

    # plain rows: vector path (width 768) and element path (width 7)
    for width in (768, 7):
        x = rng.normal(0, 1, (9, width)).astype(np.float32)
        K.split3(dev(x), 16.0, overflow=flag)
        assert raised() == 0
        x[4, width - 2] = 4094.1                      # 16 x = 65505.6 > 65504
        K.split3(dev(x), 16.0, overflow=flag)
        assert raised() == 1
        x[4, width - 2] = -4093.9                     # 16 x = -65502.4: still representable
        K.split3(dev(x), 16.0, overflow=flag)
        assert raised() == 0
        x[0, 0] = np.nan
        K.split3(dev(x), 16.0, overflow=flag)
        assert raised() == 1
        K.split3(dev(x), 16.0)                        # no flag wanted: nothing to write to
    # bias + GELU
    x = rng.normal(0, 1, (5, 768)).astype(np.float32)
    b = rng.normal(0, 1, 768).astype(np.float32)
    K.bias_gelu_split3(dev(x), dev(b), 16.0, overflow=flag)
    assert raised() == 0
    x[2, 100] = 5000.0                                # GELU(5000 + b) = 5000 + b
    K.bias_gelu_split3(dev(x), dev(b), 16.0, overflow=flag)
    assert raised() == 1
    x[2, 100] = -5000.0                               # GELU of a large negative number is 0
    K.bias_gelu_split3(dev(x), dev(b), 16.0, overflow=flag)
    assert raised() == 0
    # bias + residual + LayerNorm: outputs are gamma * (unit variance) + beta
    x = rng.normal(0, 1, (6, 768)).astype(np.float32)
    res = rng.normal(0, 1, (6, 768)).astype(np.float32)
    gamma, beta = np.ones(768, np.float32), np.zeros(768, np.float32)
    assert K.bias_res_ln_split3_(dev(x), dev(res), None, dev(beta), dev(gamma), 16.0, overflow=flag) is not None
    assert raised() == 0
    gamma[17] = 30000.0
    assert K.bias_res_ln_split3_(dev(x), dev(res), None, dev(beta), dev(gamma), 16.0, overflow=flag) is not None
    assert raised() == 1
    # attention: the context is an average of V rows, so a large V column carries through
    batch, heads, seq, d = 3, 4, 32, 64
    hidden = heads * d
    qkv = rng.normal(0, 1, (batch * seq, 3 * hidden)).astype(np.float32)
    mask = torch.ones((batch, seq), dtype=torch.int8, device="cuda")
    assert K.attention_fused_split3(dev(qkv), mask, batch, heads, seq, d, 0.125, scale=16.0, overflow=flag) is not None
    assert raised() == 0
    qkv[:, 2 * hidden + 5] = 6000.0
    assert K.attention_fused_split3(dev(qkv), mask, batch, heads, seq, d, 0.125, scale=16.0, overflow=flag) is not None
    assert raised() == 1


def test_bias_res_ln_split3_declines_other_hidden_sizes(K):
    x = dev(np.zeros((2, 100), np.float32))
    v = dev(np.ones(100, np.float32))
    assert K.bias_res_ln_split3_(x, x.clone(), None, v, v) is None


@pytest.mark.parametrize("tokens,in_features,out_features,magnitude", [(4096, 768, 2304, 1.0), (200, 3072, 768, 1.0),
                                                                       (64, 128, 512, 1.0), (33, 40, 24, 1.0),
                                                                       # the ends of the range the host classes'
                                                                       # activation scale of 16 is meant for
                                                                       (256, 768, 768, 0.01), (256, 768, 768, 500.0)])
def test_two_term_dense_matches_fp32_dense(K, tokens, in_features, out_features, magnitude):
    """Dense(x) = x W + b with both operands in two-term fp16 form on the mixed GEMM, against float64 and against
    the fp32 GEMM: the error of the form is that of fp32 arithmetic (accumulation rounding dominates both)."""
    rng = np.random.default_rng(tokens + in_features)
    x = (rng.normal(0, 1, (tokens, in_features)) * magnitude).astype(np.float32)
    w = rng.normal(0, 0.02, (in_features, out_features)).astype(np.float32)
    b = rng.normal(0, 0.02, out_features).astype(np.float32)
    want = x.astype(np.float64) @ w.astype(np.float64) + b
    blas = K.Blas()
    dx, dw, db = dev(x), dev(w), dev(b)
    plain = torch.empty((tokens, out_features), dtype=torch.float32, device="cuda")
    blas.gemm(False, False, out_features, tokens, in_features, 1.0, dw, out_features, dx, in_features, 0.0, plain,
              out_features, db)
    exponent = 10 - math.frexp(float(np.abs(w).max()))[1]
    w3 = K.split3(K.transpose(dw), 2.0 ** exponent, True)       # [out, 3 in]: hi | lo | hi
    x3 = K.split3(dx, 16.0)                                     # [tokens, 3 in]: hi | hi | lo of 16 x
    out = torch.empty((tokens, out_features), dtype=torch.float32, device="cuda")
    blas.gemm_f16_f32(True, False, out_features, tokens, 3 * in_features, 2.0 ** -exponent / 16, w3, 3 * in_features, x3,
                      3 * in_features, 0.0, out, out_features, db)
    plain, out = host(plain), host(out)
    blas.close()
    err_plain = np.linalg.norm(plain - want) / np.linalg.norm(want)
    err_two_term = np.linalg.norm(out - want) / np.linalg.norm(want)
    print("\nrelative error vs float64: fp32 GEMM %.2e, two-term fp16 GEMM %.2e" % (err_plain, err_two_term))
    assert err_two_term < 2e-6
    assert err_two_term < 2 * err_plain + 2e-7
    assert_close(out, plain, FP32_TOL, "two-term Dense vs fp32 Dense")


# ------------------------------------------------------------------ attention contractions (matrix-core kernels)

@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("batch,heads,seq,d", [(3, 12, 32, 64), (2, 4, 128, 64), (1, 2, 512, 64), (2, 3, 64, 32),
                                               (1, 2, 96, 128), (2, 16, 128, 64), (5, 1, 32, 64), (1, 2, 256, 64),
                                               # partial 128 x 128 tiles of the LDS-tiled scores kernel
                                               (1, 2, 160, 64), (1, 3, 384, 64), (2, 2, 224, 32), (1, 1, 128, 128)])
def test_attention_scores_and_context(K, name, batch, heads, seq, d):
    rng = np.random.default_rng(batch * 1000 + heads * 100 + seq + d)
    H = heads * d
    qkv = q(rng.normal(0, 1, (batch * seq, 3 * H)), name)
    qh, kh, vh = qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:]
    alpha = 1.0 / math.sqrt(d)
    dqkv = dev(qkv, tdt(name))
    scores = K.attention_scores(dqkv, batch, heads, seq, d, alpha)
    assert scores is not None
    # the oracle (pinned by the reference's BatchMatMulTest vectors) lays scores out [B, S_q, A, S_k]
    want = oracle.att_q_k(np.ascontiguousarray(qh), np.ascontiguousarray(kh), batch, seq, heads, d, alpha=alpha)
    want = want.transpose(0, 2, 1, 3)
    assert_close(host(scores), want, 2e-5 if name == "f32" else 2e-3, "attention_scores %s" % name)
    # context from row-stochastic P (what the softmax hands over)
    p = rng.random((batch, heads, seq, seq)).astype(np.float32)
    p = q(p / p.sum(-1, keepdims=True), name)
    ctx = K.attention_context(dev(p, tdt(name)), dqkv, batch, heads, seq, d)
    assert ctx is not None
    want_ctx = oracle.att_qk_v(np.ascontiguousarray(p.transpose(0, 2, 1, 3)), np.ascontiguousarray(vh), batch, seq,
                               heads, d).reshape(batch * seq, H)
    assert_close(host(ctx), want_ctx, 2e-5 if name == "f32" else 2e-3, "attention_context %s" % name)


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("batch,heads,seq,d", [(3, 12, 32, 64), (2, 4, 128, 64), (2, 3, 64, 32), (1, 2, 96, 128),
                                               (2, 16, 128, 64), (5, 1, 32, 64), (7, 3, 64, 64),
                                               # seq 32, head size 64: four wavefronts per problem up to 2048
                                               # problems, one wavefront per problem beyond and at head size 32
                                               (1, 12, 32, 64), (24, 12, 32, 64), (180, 12, 32, 64), (2, 2, 32, 32),
                                               # longer than 128: the online-softmax kernels (chunks of 64 keys;
                                               # seq 512 stages the keys in groups, the others the whole head)
                                               (1, 2, 512, 64), (2, 3, 256, 64), (2, 2, 160, 64), (1, 1, 384, 32),
                                               (2, 3, 512, 32)])
@pytest.mark.parametrize("masked", [True, False])
def test_attention_fused_against_oracle(K, name, batch, heads, seq, d, masked):
    """One-launch attention core vs the oracle's attention_self pieces (att_q_k -> mask -> softmax -> att_qk_v),
    with an arbitrary 0/1 mask pattern (not only prefixes) and one fully masked sequence."""
    rng = np.random.default_rng(batch * 1000 + heads * 100 + seq + d)
    H = heads * d
    qkv = q(rng.normal(0, 1, (batch * seq, 3 * H)), name)
    qh, kh, vh = (np.ascontiguousarray(x) for x in (qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:]))
    mask = (rng.random((batch, seq)) < 0.7).astype(np.int8)
    mask[0, :] = 0
    alpha = 1.0 / math.sqrt(d)
    ctx = K.attention_fused(dev(qkv, tdt(name)), dev(mask) if masked else None, batch, heads, seq, d, alpha)
    if ctx is None:  # K and V of one head must fit 160 KB of LDS, except at seq 512 (keys staged in groups)
        assert seq * (d + 4) * 4 + d * (seq + 4) * 4 + 2 * seq * 4 > 160 * 1024 and name == "f32" and seq != 512
        return
    scores = oracle.att_q_k(qh, kh, batch, seq, heads, d, alpha=alpha)  # [B, S_q, A, S_k]
    if name == "f16":
        scores = oracle.round_to_half(scores)  # the scaled scores are what is stored; the mask is added in fp32
    if masked:
        scores = scores + (-10000.0 * (1.0 - mask.astype(np.float32)))[:, None, None, :]
    p = oracle.softmax_(np.ascontiguousarray(scores.reshape(-1, seq), dtype=np.float32)).reshape(scores.shape)
    if name == "f16":
        p = oracle.round_to_half(p)
    want = oracle.att_qk_v(np.ascontiguousarray(p, dtype=np.float32), vh, batch, seq, heads, d).reshape(batch * seq, H)
    # Sequence 0 is fully masked: every score sits at -10000, where fp32 resolves 1e-3, so a last-bit difference
    # in a score moves its probability by 1e-3 relative.  It gets the fp16 tolerance; the others the tight one.
    tol = 2e-5 if name == "f32" else 2e-3
    first = seq if masked else 0
    if first < batch * seq:
        assert_close(host(ctx)[first:], want[first:], tol, "attention_fused %s" % name)
    assert_close(host(ctx)[:seq], want[:seq], 2e-3, "attention_fused %s, fully masked sequence" % name)
    # and against the three-kernel sequence of this library
    s3 = K.attention_scores(dev(qkv, tdt(name)), batch, heads, seq, d, alpha)
    K.mask_scale_softmax_(s3, dev(mask) if masked else None, 1.0)
    c3 = K.attention_context(s3, dev(qkv, tdt(name)), batch, heads, seq, d)
    if first < batch * seq:
        assert_close(host(ctx)[first:], host(c3)[first:], 1e-5 if name == "f32" else 2e-3,
                     "fused vs three kernels %s" % name)
    assert_close(host(ctx)[:seq], host(c3)[:seq], 2e-3, "fused vs three kernels %s, fully masked sequence" % name)


@pytest.mark.parametrize("batch,heads,seq,d", [(64, 16, 128, 64), (128, 8, 32, 64), (86, 12, 64, 32), (70, 16, 96, 128)])
@pytest.mark.parametrize("masked", [True, False])
def test_attention_fused_many_problems_fp16(K, batch, heads, seq, d, masked):
    """From 1024 (batch, head) problems up, fp16 sequences of at most 128 keys take the kernel that classifies key
    tiles from the mask words (left out / no mask term / general), takes the row sums from the matrix cores and
    reads V through transposing LDS loads.  Masks with every tile class: prefixes that end inside a tile and on a
    tile boundary, kept keys scattered over dead tiles, bytes other than 1, no masked key, one kept key in the last
    tile, a sequence with no kept key -- against the oracle, which computes every key."""
    name = "f16"
    rng = np.random.default_rng(batch + heads * 100 + seq + d)
    H = heads * d
    qkv = q(rng.normal(0, 1, (batch * seq, 3 * H)), name)
    qh, kh, vh = (np.ascontiguousarray(x) for x in (qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:]))
    valid = rng.integers(1, seq + 1, batch)
    mask = (np.arange(seq)[None, :] < valid[:, None]).astype(np.int8)
    mask[0, :] = 0                                      # no kept key: every tile, general path
    mask[1, :] = 1                                      # every key kept
    mask[2, :] = 0
    mask[2, seq - 1] = 1                                # one kept key, in the last tile
    mask[3, :] = (rng.random(seq) < 0.5).astype(np.int8)
    mask[3, :32] = 0                                    # a dead tile in front of mixed ones
    mask[4, :32] = 1                                    # prefix that ends on a tile boundary
    mask[4, 32:] = 0
    mask[5, :] = rng.integers(1, 4, seq).astype(np.int8) * (rng.random(seq) < 0.8)   # any non-zero byte keeps the key
    mask[6, :] = -1                                     # negative bytes keep it too
    alpha = 1.0 / math.sqrt(d)
    ctx = K.attention_fused(dev(qkv, tdt(name)), dev(mask) if masked else None, batch, heads, seq, d, alpha)
    assert ctx is not None
    scores = oracle.round_to_half(oracle.att_q_k(qh, kh, batch, seq, heads, d, alpha=alpha))
    if masked:
        scores = scores + (-10000.0 * (mask == 0).astype(np.float32))[:, None, None, :]
    p = oracle.softmax_(np.ascontiguousarray(scores.reshape(-1, seq), dtype=np.float32)).reshape(scores.shape)
    want = oracle.att_qk_v(np.ascontiguousarray(oracle.round_to_half(p), dtype=np.float32), vh, batch, seq, heads,
                           d).reshape(batch * seq, H)
    got = host(ctx)
    for b in range(batch):
        rows = slice(b * seq, (b + 1) * seq)
        assert_close(got[rows], want[rows], 2e-3, "attention, many problems, sequence %d (valid %d)" % (b, valid[b]))
    # the same call on a mask that cannot be read as 32-bit words takes the general kernel: same result to rounding
    if masked:
        shifted = torch.zeros(batch * seq + 1, dtype=torch.int8, device="cuda")
        shifted[1:] = dev(mask).reshape(-1)
        general = K.attention_fused(dev(qkv, tdt(name)), shifted[1:].reshape(batch, seq), batch, heads, seq, d, alpha)
        assert general is not None
        assert_close(got, host(general), 2e-3, "tile-classifying kernel vs general kernel")


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("heads,seq,d", [(2, 512, 64), (3, 256, 64), (2, 160, 64), (1, 384, 32), (2, 512, 32)])
def test_attention_long_sequences_with_padding(K, name, heads, seq, d):
    """The online-softmax kernel leaves out key tiles (32 keys) that are masked throughout.  Masks with whole tiles
    of zeros in every position (prefix padding, live tiles scattered between dead ones, a single unmasked key in
    the last tile, no padding, everything masked) against the oracle, which computes every key; and the same call
    on a mask that cannot be read as 32-bit words (all tiles computed) gives the same result."""
    batch = 6
    rng = np.random.default_rng(heads * 100 + seq + d)
    H = heads * d
    if name == "f32" and seq != 512 and seq * (d + 4) * 4 + d * (seq + 4) * 4 + 2 * seq * 4 > 160 * 1024:
        pytest.skip("K and V of one head do not fit the LDS in fp32")
    qkv = q(rng.normal(0, 1, (batch * seq, 3 * H)), name)
    qh, kh, vh = (np.ascontiguousarray(x) for x in (qkv[:, :H], qkv[:, H:2 * H], qkv[:, 2 * H:]))
    mask = np.zeros((batch, seq), np.int8)
    mask[0, :40] = 1                                    # prefix shorter than two tiles
    mask[1, 96:128] = rng.random(32) < 0.5              # live tiles between dead ones
    mask[1, seq - 64:seq - 32] = 1
    mask[1, 100] = 1
    mask[2, :] = 1                                      # no padding
    mask[3, seq - 1] = 1                                # one unmasked key, in the last tile
    mask[4, :] = 0                                      # everything masked: all tiles stay
    mask[5, :seq // 2 + 5] = 1
    alpha = 1.0 / math.sqrt(d)
    ctx = K.attention_fused(dev(qkv, tdt(name)), dev(mask), batch, heads, seq, d, alpha)
    assert ctx is not None
    scores = oracle.att_q_k(qh, kh, batch, seq, heads, d, alpha=alpha)
    if name == "f16":
        scores = oracle.round_to_half(scores)
    scores = scores + (-10000.0 * (1.0 - mask.astype(np.float32)))[:, None, None, :]
    p = oracle.softmax_(np.ascontiguousarray(scores.reshape(-1, seq), dtype=np.float32)).reshape(scores.shape)
    if name == "f16":
        p = oracle.round_to_half(p)
    want = oracle.att_qk_v(np.ascontiguousarray(p, dtype=np.float32), vh, batch, seq, heads, d).reshape(batch * seq, H)
    got = host(ctx)
    tol = 2e-5 if name == "f32" else 2e-3
    for b in range(batch):
        rows = slice(b * seq, (b + 1) * seq)
        assert_close(got[rows], want[rows], 2e-3 if b == 4 else tol, "padded attention %s, sequence %d" % (name, b))
    # a mask at an odd address: no tile is left out, the result agrees to rounding
    shifted = torch.zeros(batch * seq + 1, dtype=torch.int8, device="cuda")
    shifted[1:] = dev(mask).reshape(-1)
    plain = K.attention_fused(dev(qkv, tdt(name)), shifted[1:].reshape(batch, seq), batch, heads, seq, d, alpha)
    assert plain is not None
    assert_close(got, host(plain), 2e-3 if name == "f16" else 2e-5, "skipping vs not skipping masked tiles")
    # sequence 4 (fully masked) is ill-conditioned at fp32 resolution: compare it loosely
    keep = np.r_[0:4 * seq, 5 * seq:batch * seq]
    assert_close(got[keep], host(plain)[keep], 1e-6 if name == "f32" else 2e-3, "skipping vs not skipping, tight")


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("batch,heads,seq,d", [(37, 3, 512, 64), (9, 2, 256, 64), (5, 2, 160, 32)])
def test_attention_longest_sequences_first(K, name, batch, heads, seq, d):
    """cubert_attention_order sorts the sequences by falling number of live key tiles (a sequence without any kept
    key counts as full); the long-sequence kernels give bit for bit the same context whichever order they are handed."""
    rng = np.random.default_rng(batch + seq)
    H = heads * d
    if name == "f32" and seq != 512 and seq * (d + 4) * 4 + d * (seq + 4) * 4 + 2 * seq * 4 > 160 * 1024:
        pytest.skip("K and V of one head do not fit the LDS in fp32")
    valid = np.minimum(seq, 1 + np.floor(rng.exponential(seq / 5.0, batch))).astype(np.int64)
    mask = (np.arange(seq)[None, :] < valid[:, None]).astype(np.int8)
    mask[1, :] = 0                                     # no kept key: every tile is computed
    mask[2, :] = 0
    mask[2, seq - 3] = 1                               # a single live tile, the last one
    mask[3, ::37] = 1                                  # kept keys scattered over every tile
    dmask = dev(mask)
    order = K.attention_order(dmask)
    assert order is not None and order.numel() == 8 * batch
    host_order = order.cpu().numpy().astype(np.int64)
    got = host_order[:batch]
    assert sorted(got.tolist()) == list(range(batch))
    tile_live = (mask.reshape(batch, seq // 32, 32) != 0).any(-1)
    tile_live[~tile_live.any(-1)] = True               # no kept key at all: every tile
    live = tile_live.sum(-1)
    assert (np.diff(live[got]) <= 0).all(), live[got]
    # the record of each position: number of live tiles, their numbers 4 bits each, and as a bit mask
    records = host_order[4 * batch:].reshape(batch, 4)
    for position, b in enumerate(got):
        tiles = np.flatnonzero(tile_live[b])
        n, lo, hi, bits = (int(v) & 0xffffffff for v in records[position])
        listed = [((lo | (hi << 32)) >> (4 * i)) & 15 for i in range(n)]
        assert n == len(tiles) and listed == tiles.tolist() and bits == sum(1 << int(t) for t in tiles), (position, b)
    qkv = dev(q(rng.normal(0, 1, (batch * seq, 3 * H)), name), tdt(name))
    alpha = 1.0 / math.sqrt(d)
    plain = K.attention_fused(qkv, dmask, batch, heads, seq, d, alpha)
    ordered = K.attention_fused(qkv, dmask, batch, heads, seq, d, alpha, order=order)
    # any permutation of the positions that moves the records along with the indices
    flipped = torch.cat([order[:batch].flip(0), order[batch:4 * batch], order[4 * batch:].reshape(batch, 4).flip(0).reshape(-1)])
    backwards = K.attention_fused(qkv, dmask, batch, heads, seq, d, alpha, order=flipped.contiguous())
    assert plain is not None and ordered is not None and backwards is not None
    assert torch.equal(plain, ordered) and torch.equal(plain, backwards)
    # shapes and masks the sort declines
    assert K.attention_order(dev(np.ones((3, 40), np.int8))) is None
    odd = torch.zeros(batch * seq + 1, dtype=torch.int8, device="cuda")[1:].reshape(batch, seq)
    assert K.attention_order(odd) is None


def test_attention_unsupported_shapes_are_declined(K):
    """Shapes without a matrix-core kernel return CUBERT_UNSUPPORTED and launch nothing; the host classes then
    loop the strided-batched GEMM (covered by the encoder reference vectors, seq 4, head size 3)."""
    qkv = torch.zeros((2 * 4, 3 * 6), device="cuda")
    assert K.attention_scores(qkv, 2, 2, 4, 3, 1.0) is None
    assert K.attention_context(torch.zeros((2, 2, 4, 4), device="cuda"), qkv, 2, 2, 4, 3) is None
    qkv = torch.zeros((2 * 40, 3 * 128), device="cuda")
    assert K.attention_scores(qkv, 2, 2, 40, 64, 1.0) is None  # seq not a multiple of 32
    qkv = torch.zeros((544, 3 * 128), device="cuda")
    assert K.attention_fused(qkv, None, 1, 2, 544, 64, 1.0) is None   # more than 16 query tiles
    qkv = torch.zeros((256, 3 * 256), device="cuda")
    assert K.attention_fused(qkv, None, 1, 2, 256, 128, 1.0) is None  # long sequence with head size 128


# ------------------------------------------------------------------ GEMM convention

@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("M,N,K_", [(768, 4096, 768), (2, 128, 768), (5, 7, 11), (3072, 64, 768)])
def test_gemm_against_oracle_sgemm(K, name, ta, tb, M, N, K_):
    rng = np.random.default_rng(M + N + K_ + ta * 2 + tb)
    lda, ldb, ldc = (K_ if ta else M), (N if tb else K_), M
    A = q(rng.normal(0, 1, lda * (M if ta else K_)), name)
    B = q(rng.normal(0, 1, ldb * (K_ if tb else N)), name)
    C0 = q(rng.normal(0, 1, ldc * N), name)
    bias = q(rng.normal(0, 1, M), name)
    blas = K.Blas()
    for beta, use_bias in ((0.0, False), (1.0, False), (0.0, True)):
        C = dev(C0, tdt(name))
        blas.gemm(ta, tb, M, N, K_, 0.5, dev(A, tdt(name)), lda, dev(B, tdt(name)), ldb, beta, C, ldc,
                  bias=dev(bias, tdt(name)) if use_bias else None)
        want = oracle.sgemm(ta, tb, M, N, K_, 0.5, A, lda, B, ldb, beta, C0.copy(), ldc)
        if use_bias:
            want = (want.reshape(N, M) + bias[None, :]).ravel()
        # fp32: summation order differs between BLAS libraries; error grows like sqrt(K) * eps
        assert_close(host(C), want, 2e-5 if name == "f32" else 2e-3, "gemm %s beta=%g bias=%s" % (name, beta, use_bias))


# ------------------------------------------------------------------ few-token Dense GEMM

@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("M,N,K_", [(768, 32, 768), (2304, 32, 768), (3072, 32, 768), (768, 32, 3072), (768, 1, 768),
                                    (100, 7, 64), (33, 32, 16), (1024, 16, 4096), (2, 5, 768), (768, 32, 272),
                                    (768, 64, 768), (768, 33, 3072), (3072, 48, 768), (100, 50, 64), (1024, 64, 4096)])
def test_gemm_skinny_against_oracle_sgemm(K, name, M, N, K_):
    """Dense layer of a request with at most 64 tokens (column-major C[M,N] = A[M,K] B[K,N] + bias), K cut into
    1..16 slices; 30 launches in a row must give bit-identical results (slices are added in a fixed order and
    the arrival counters reset themselves)."""
    rng = np.random.default_rng(M + N + K_)
    ldb = K_ + 8  # a padded activation row pitch (multiple of 16 bytes), as a strided first-token view has
    A = q(rng.normal(0, 1, M * K_), name)
    Bs = [q(rng.normal(0, 1, N * ldb), name) for _ in range(2)]  # alternate: stale partial sums would show
    bias = q(rng.normal(0, 1, M), name)
    blas = K.Blas()
    dA, dBs, dbias = dev(A, tdt(name)), [dev(B, tdt(name)) for B in Bs], dev(bias, tdt(name))
    for alpha, use_bias in ((1.0, True), (0.5, False)):
        outs = [[], []]
        for it in range(30):
            C = torch.full((N * M,), 7.0, dtype=tdt(name), device="cuda")
            assert blas.gemm_skinny(M, N, K_, alpha, dA, M, dBs[it % 2], ldb, C, M,
                                    bias=dbias if use_bias else None) is not None
            outs[it % 2].append(C)
        for which in range(2):
            for other in outs[which][1:]:
                assert torch.equal(outs[which][0], other)
            want = oracle.sgemm(0, 0, M, N, K_, alpha, A, M, Bs[which], ldb, 0.0, np.zeros(N * M, np.float32), M)
            if use_bias:
                want = (want.reshape(N, M) + bias[None, :]).ravel()
            assert_close(host(outs[which][0]), want, 2e-5 if name == "f32" else 2e-3,
                         "gemm_skinny %s alpha=%g" % (name, alpha))
    B, dB = Bs[0], dBs[0]
    # Dense + bias + GELU in one launch against the oracle's GELU of the oracle's GEMM
    C = torch.zeros((N * M,), dtype=tdt(name), device="cuda")
    assert blas.gemm_skinny(M, N, K_, 1.0, dA, M, dB, ldb, C, M, bias=dbias, gelu=True) is not None
    pre = (oracle.sgemm(0, 0, M, N, K_, 1.0, A, M, B, ldb, 0.0, np.zeros(N * M, np.float32), M).reshape(N, M)
           + bias[None, :])
    assert_close(host(C), oracle.gelu(pre).ravel(), 2e-5 if name == "f32" else 2e-3, "gemm_skinny + gelu %s" % name)
    # the same on weights packed into the kernel's own order: bit-identical to the unpacked call where both cut the
    # reduction the same way (2-byte weights in the plain layout keep one pass per wavefront at every size)
    packed = blas.gemm_skinny_pack(dA, M, M, K_)
    for gelu in (False, True):
        C1 = torch.zeros((N * M,), dtype=tdt(name), device="cuda")
        C2 = torch.full((N * M,), 3.0, dtype=tdt(name), device="cuda")
        assert blas.gemm_skinny(M, N, K_, 1.0, dA, M, dB, ldb, C1, M, bias=dbias, gelu=gelu) is not None
        assert blas.gemm_skinny_packed(M, N, K_, 1.0, packed, dB, ldb, C2, M, bias=dbias, gelu=gelu) is not None
        if name == "f32":
            assert torch.equal(C1, C2)
        else:
            assert_close(host(C2), host(C1), 2e-3, "packed vs plain weights, gelu=%s" % gelu)
    # the general entry point takes the same path by itself (up to 32 tokens; beyond, the library: same numbers)
    C = torch.zeros((N * M,), dtype=tdt(name), device="cuda")
    blas.gemm(0, 0, M, N, K_, 1.0, dA, M, dB, ldb, 0.0, C, M, bias=dbias)
    want = (oracle.sgemm(0, 0, M, N, K_, 1.0, A, M, B, ldb, 0.0, np.zeros(N * M, np.float32), M).reshape(N, M)
            + bias[None, :]).ravel()
    assert_close(host(C), want, 2e-5 if name == "f32" else 2e-3, "gemm via skinny %s" % name)


def _slices_added(partials, name):
    """0.f + slice 0 + slice 1 + ... in fp32, rounded to the storage type: what the GEMM's last workgroup stores."""
    total = torch.zeros_like(partials[0])
    for s in range(partials.shape[0]):
        total = total + partials[s]
    return total.to(tdt(name))


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("M,N,K_", [(768, 32, 768), (2304, 32, 768), (768, 32, 3072), (768, 1, 768), (100, 7, 64),
                                    (1024, 16, 4096), (3072, 20, 1024), (33, 32, 16), (768, 64, 768), (768, 40, 3072),
                                    (1024, 64, 4096), (100, 33, 64)])
def test_gemm_skinny_partials_add_up_to_the_gemm(K, name, packed, M, N, K_):
    """The few-token Dense product left as K slices: added in slice order and rounded they are what
    cubert_gemm_skinny_* stores (alpha 1, no bias) up to the order of the additions, rows from N on are zero, and a
    second product into the same buffer leaves nothing of the first."""
    rng = np.random.default_rng(M * 3 + N * 5 + K_)
    ldb = K_ + 8
    A = q(rng.normal(0, 1, M * K_), name)
    blas = K.Blas()
    dA = dev(A, tdt(name))
    weights = blas.gemm_skinny_pack(dA, M, M, K_) if packed else dA
    for trial in range(2):
        B = q(rng.normal(0, 1, N * ldb), name)
        dB = dev(B, tdt(name))
        got = blas.gemm_skinny_partials(M, N, K_, weights, M, dB, ldb, packed=packed)
        assert got is not None
        partials, slices, pitch = got
        assert pitch >= M and pitch % 32 == 0 and slices >= 1 and partials.shape[1] == (N + 31) // 32 * 32
        C = torch.full((N * M,), 7.0, dtype=tdt(name), device="cuda")
        if packed:
            assert blas.gemm_skinny_packed(M, N, K_, 1.0, weights, dB, ldb, C, M) is not None
        else:
            assert blas.gemm_skinny(M, N, K_, 1.0, dA, M, dB, ldb, C, M) is not None
        added = _slices_added(partials, name)
        # the same product, added up in another order where the reduction is cut finer here
        assert_close(host(added[:N, :M]).ravel(), host(C), 2e-6 if name == "f32" else 1e-3, "slices against the GEMM")
        assert not partials[:, N:, :].any()
    want = oracle.sgemm(0, 0, M, N, K_, 1.0, A, M, B, ldb, 0.0, np.zeros(N * M, np.float32), M)
    assert_close(host(added[:N, :M]).ravel(), want, 2e-5 if name == "f32" else 2e-3, "partials %s" % name)


def test_gemm_skinny_partials_declines_what_it_cannot_do(K):
    blas = K.Blas()
    x = torch.zeros(64 * 1024, device="cuda")
    assert blas.gemm_skinny_partials(64, 65, 64, x, 64, x, 64) is None             # more than 64 tokens
    assert blas.gemm_skinny_partials(64, 8, 24, x, 64, x, 24) is None              # K not a multiple of 16
    assert blas.gemm_skinny_partials(64, 8, 32, x, 64, x[1:], 32) is None          # misaligned activations
    assert blas.gemm_skinny_partials(768, 8, 768, x, 768, x, 768, partial_floats=1000) is None  # buffer too small
    assert blas.gemm_skinny_partials(64, 8, 32, x, 64, x, 32, partial_floats=2048) is not None


@pytest.mark.parametrize("name", ["f32", "f16"])
@pytest.mark.parametrize("rows,hidden,in_features,with_bias", [(32, 768, 768, True), (32, 768, 3072, True),
                                                               (7, 768, 3072, False), (1, 1024, 4096, True),
                                                               (20, 256, 1024, True), (32, 512, 64, False),
                                                               (64, 768, 768, True), (33, 768, 3072, True),
                                                               (50, 1024, 4096, False)])
def test_bias_res_ln_from_partials_has_the_bits_of_layer_norm_of_the_added_slices(K, name, rows, hidden, in_features, with_bias):
    rng = np.random.default_rng(rows + hidden + in_features)
    blas = K.Blas()
    W = dev(q(rng.normal(0, 0.05, in_features * hidden), name), tdt(name))          # [in, out]
    X = dev(q(rng.normal(0, 1, rows * in_features), name), tdt(name))
    residual = dev(q(rng.normal(0, 1, (rows, hidden)), name), tdt(name))
    bias = dev(q(rng.normal(0, 1, hidden), name), tdt(name)) if with_bias else None
    beta, gamma = (dev(q(rng.normal(0, 1, hidden), name), tdt(name)) for _ in range(2))
    partials, slices, pitch = blas.gemm_skinny_partials(hidden, rows, in_features, W, hidden, X, in_features)
    # what a GEMM that adds its own slices would have stored: 0.f + slice 0 + slice 1 + ..., rounded
    C = _slices_added(partials, name)[:rows, :hidden].contiguous()
    dense_values = host(C)
    want = K.bias_res_ln_(C, residual, bias, beta, gamma)
    got = K.bias_res_ln_partials(partials, residual, bias, beta, gamma)
    assert got is not None
    if name == "f32":
        assert torch.equal(got, want)
    else:
        # half precision: the values that go into the LayerNorm are the same, but the two kernels are compiled
        # separately (a multiply-add fused in one and not in the other moves a result across an fp16 rounding boundary
        # now and then), and at 768 halves bias_res_ln takes its two-rows-per-wavefront kernel, whose row sums are
        # added in another order: the last bit of a few elements
        diff = (got.float() - want.float()).abs()
        assert (diff <= want.float().abs() * 2.0 ** -9 + 1e-6).all()
        assert (diff > 0).float().mean().item() < 0.01
        assert_close(host(got), host(want), 1e-3, "LayerNorm from partials against LayerNorm of the GEMM output")
    # and against the oracle's LayerNorm of the values the GEMM stored
    ref = oracle.layer_norm_(host(residual), dense_values + (host(bias) if with_bias else 0.0), host(beta), host(gamma))
    assert_close(host(got), ref, 2e-5 if name == "f32" else 4e-3, "LayerNorm from partials %s" % name)


def test_bias_res_ln_from_partials_declines_what_it_cannot_do(K):
    partials = torch.zeros((3, 32, 768), device="cuda")
    v = torch.zeros(768, device="cuda")
    assert K.bias_res_ln_partials(partials, torch.zeros((65, 768), device="cuda"), v, v, v) is None   # 65 rows
    narrow = torch.zeros((3, 32, 128), device="cuda")
    assert K.bias_res_ln_partials(narrow, torch.zeros((4, 100), device="cuda"), v[:100], v[:100], v[:100]) is None  # hidden 100
    assert K.bias_res_ln_partials(narrow, torch.zeros((4, 768), device="cuda"), v, v, v) is None  # rows narrower than hidden


def test_gemm_skinny_declines_what_it_cannot_do(K):
    blas = K.Blas()
    x = torch.zeros(64 * 1024, device="cuda")
    assert blas.gemm_skinny(64, 65, 64, 1.0, x, 64, x, 64, x, 64) is None      # more than 64 tokens
    assert blas.gemm_skinny(64, 8, 24, 1.0, x, 64, x, 24, x, 64) is None       # K not a multiple of 16
    assert blas.gemm_skinny(64, 8, 32, 1.0, x, 64, x[1:], 32, x, 64) is None   # misaligned activations
    assert blas.gemm_skinny(64, 8, 32, 1.0, x, 64, x, 34, x, 64) is None       # row pitch not 16-byte aligned


# ------------------------------------------------------------------ edge cases

def test_empty_and_bad_arguments(K):
    from cubert_amd._lib import lib
    L = lib()
    x = torch.zeros((4, 768), device="cuda")
    assert L.cubert_bias_res_ln_f32(x.data_ptr(), x.data_ptr(), None, x.data_ptr(), x.data_ptr(), 0, 768, None) == 0
    assert L.cubert_bias_gelu_f32(x.data_ptr(), None, 0, 768, None) == 0
    assert L.cubert_mask_scale_softmax_f32(x.data_ptr(), None, 1.0, 0, 12, 32, None) == 0
    assert L.cubert_bias_res_ln_f32(None, x.data_ptr(), None, x.data_ptr(), x.data_ptr(), 4, 768, None) == -1
    assert L.cubert_bias_gelu_f32(x.data_ptr(), None, 4, 0, None) == -1
    assert L.cubert_mask_scale_softmax_f32(x.data_ptr(), None, 1.0, 1, 0, 32, None) == -1
    assert L.cubert_mean_pool_f32(x.data_ptr(), x.data_ptr(), 1, 0, 768, None) == -1
    # the two-term operand kernels
    h = torch.zeros((4, 3 * 768), dtype=torch.float16, device="cuda")
    assert L.cubert_split3_f32(x.data_ptr(), 0, 768, 1.0, 0, h.data_ptr(), None, None) == 0
    assert L.cubert_split3_f32(x.data_ptr(), 4, 0, 1.0, 0, h.data_ptr(), None, None) == -1
    assert L.cubert_split3_f32(None, 4, 768, 1.0, 0, h.data_ptr(), None, None) == -1
    assert L.cubert_bias_gelu_split3_f32(x.data_ptr(), None, 0, 768, 1.0, h.data_ptr(), None, None) == 0
    assert L.cubert_bias_gelu_split3_f32(x.data_ptr(), None, 4, 768, 1.0, None, None, None) == -1
    assert L.cubert_bias_res_ln_split3_f32(x.data_ptr(), x.data_ptr(), None, x.data_ptr(), x.data_ptr(), 0, 768, 1.0,
                                           h.data_ptr(), None, None) == 0
    assert L.cubert_bias_res_ln_split3_f32(x.data_ptr(), x.data_ptr(), None, x.data_ptr(), x.data_ptr(), 4, 768, 1.0,
                                           None, None, None) == -1
    torch.cuda.synchronize()


def test_split3_unaligned_and_odd_widths_take_the_generic_path(K):
    rng = np.random.default_rng(11)
    base = torch.zeros(5 * 24 + 1, device="cuda")
    x = rng.normal(0, 1, (5, 24)).astype(np.float32)
    base[1:] = dev(x).reshape(-1)
    view = base[1:].view(5, 24)          # 4-byte aligned only
    assert torch.equal(K.split3(view, 2.0), K.split3(dev(x), 2.0))
    b = dev(rng.normal(0, 1, 24).astype(np.float32))
    assert torch.equal(K.bias_gelu_split3(view, b, 16.0), K.bias_gelu_split3(dev(x), b, 16.0))


def test_unaligned_views_take_the_generic_path(K):
    """Tensors offset by one element break 16-byte alignment; results must not change."""
    rng = np.random.default_rng(5)
    base = torch.zeros(4 * 768 + 1, device="cuda")
    x = rng.normal(0, 1, (4, 768)).astype(np.float32)
    base[1:] = dev(x).reshape(-1)
    view = base[1:].view(4, 768)
    res = dev(rng.normal(0, 1, (4, 768)).astype(np.float32))
    beta, gamma = dev(np.zeros(768, np.float32)), dev(np.ones(768, np.float32))
    K.bias_res_ln_(view, res, None, beta, gamma)
    want = oracle.layer_norm_(host(res), x, np.zeros(768), np.ones(768))
    assert_close(host(view), want, FP32_TOL)
