"""The fused layer kernels on torch tensors (torch is only the device allocator
and stream here): thin wrappers over the C ABI of include/cubert_kernels.h.
Tensors must be contiguous CUDA tensors of dtype float32 or float16; kernels run
on torch's current stream."""
import ctypes

import torch

from ._lib import lib


def _suffix(t):
    if t.dtype == torch.float32:
        return "f32"
    if t.dtype == torch.float16:
        return "f16"
    raise TypeError("float32 or float16 expected, got %s" % t.dtype)


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError("contiguous CUDA tensor expected")
    return t.data_ptr()


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _check(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed with code %d" % (what, rc))


def _call(name, ref, *args):
    fn = getattr(lib(), "%s_%s" % (name, _suffix(ref)))
    _check(fn(*args), fn.__name__)


def gather(ids, table):
    """out[i] = table[ids[i]]; ids int32 or int8."""
    out = torch.empty((ids.numel(), table.shape[1]), dtype=table.dtype, device=table.device)
    name = "cubert_gather_i8" if ids.dtype == torch.int8 else "cubert_gather"
    _call(name, table, _ptr(ids), ids.numel(), _ptr(table), table.shape[1], _ptr(out), _stream())
    return out


def embed_ln(ids, segments, word, pos, type_, beta, gamma):
    batch, seq = ids.shape
    hidden = word.shape[1]
    out = torch.empty((batch, seq, hidden), dtype=word.dtype, device=word.device)
    _call("cubert_embed_ln", word, _ptr(ids), _ptr(segments), _ptr(word), _ptr(pos), _ptr(type_), _ptr(beta),
          _ptr(gamma), _ptr(out), batch, seq, hidden, _stream())
    return out


def bias_res_ln_(inout, residual, bias, beta, gamma):
    rows, hidden = inout.numel() // inout.shape[-1], inout.shape[-1]
    _call("cubert_bias_res_ln", inout, _ptr(inout), _ptr(residual), _ptr(bias), _ptr(beta), _ptr(gamma), rows, hidden,
          _stream())
    return inout


def bias_res_ln_partials(partials, residual, bias, beta, gamma):
    """LayerNorm(storage type of (sum of the K slices partials[s, :rows, :hidden]) + bias + residual); None when the
    shape does not fit."""
    rows, hidden = residual.numel() // residual.shape[-1], residual.shape[-1]
    out = torch.empty_like(residual)
    fn = getattr(lib(), "cubert_bias_res_ln_partials_" + _suffix(residual))
    rc = fn(_ptr(out), _ptr(partials), partials.shape[0], partials.shape[2], _ptr(residual), _ptr(bias), _ptr(beta),
            _ptr(gamma), rows, hidden, _stream())
    if rc == -2:
        return None
    _check(rc, fn.__name__)
    return out


def bias_gelu_(inout, bias):
    rows, width = inout.numel() // inout.shape[-1], inout.shape[-1]
    _call("cubert_bias_gelu", inout, _ptr(inout), _ptr(bias), rows, width, _stream())
    return inout


def mask_scale_softmax_(scores, mask, scale=1.0):
    batch, heads, seq, seq2 = scores.shape
    assert seq == seq2
    _call("cubert_mask_scale_softmax", scores, _ptr(scores), _ptr(mask), float(scale), batch, heads, seq, _stream())
    return scores


def attention_scores(qkv, batch, heads, seq, head_size, alpha):
    """scores[B, A, S, S] = alpha * Q K^T from a packed [B*S, 3*H] projection (Q | K | V column blocks).
    Returns None when the shape has no matrix-core kernel."""
    hidden = heads * head_size
    flat = qkv.view(-1)
    scores = torch.empty((batch, heads, seq, seq), dtype=qkv.dtype, device=qkv.device)
    fn = getattr(lib(), "cubert_attention_scores_" + _suffix(qkv))
    rc = fn(_ptr(flat), _ptr(flat[hidden:]), 3 * hidden, _ptr(scores), float(alpha), batch, heads, seq, head_size,
            _stream())
    if rc == -2:
        return None
    _check(rc, fn.__name__)
    return scores


def attention_order(mask):
    """What cubert_attention_order writes, as an int32 tensor of 8 * batch: the sequence indices by falling number of
    key tiles (32 keys) with a kept key in [0, batch), and from 4 * batch on a record of 4 ints per position (live
    tiles: count, list, bit mask); None when the shape or the mask's alignment is not taken."""
    batch, seq = mask.shape
    order = torch.zeros(8 * batch, dtype=torch.int32, device=mask.device)
    rc = lib().cubert_attention_order(_ptr(mask), batch, seq, _ptr(order), _stream())
    if rc == -2:
        return None
    _check(rc, "cubert_attention_order")
    return order


def attention_fused(qkv, mask, batch, heads, seq, head_size, alpha, order=None):
    """ctx[B*S, H] = softmax(alpha Q K^T + mask) V in one launch (seq <= 512); None when the shape does not fit.
    `order` (from attention_order): the sequence each group of `heads` workgroups takes."""
    hidden = heads * head_size
    flat = qkv.view(-1)
    ctx = torch.empty((batch * seq, hidden), dtype=qkv.dtype, device=qkv.device)
    if order is not None:
        fn = getattr(lib(), "cubert_attention_fused_ordered_" + _suffix(qkv))
        rc = fn(_ptr(flat), _ptr(flat[hidden:]), _ptr(flat[2 * hidden:]), 3 * hidden, _ptr(mask), _ptr(order), _ptr(ctx),
                hidden, float(alpha), batch, heads, seq, head_size, _stream())
        if rc == -2:
            return None
        _check(rc, fn.__name__)
        return ctx
    fn = getattr(lib(), "cubert_attention_fused_" + _suffix(qkv))
    rc = fn(_ptr(flat), _ptr(flat[hidden:]), _ptr(flat[2 * hidden:]), 3 * hidden, _ptr(mask), _ptr(ctx), hidden,
            float(alpha), batch, heads, seq, head_size, _stream())
    if rc == -2:
        return None
    _check(rc, fn.__name__)
    return ctx


def attention_fused_split3(qkv, mask, batch, heads, seq, head_size, alpha, scale=1.0, overflow=None):
    """attention_fused of an fp32 projection with scale * context as fp16 rows [B*S, 3*H]: hi | hi | lo; None when
    the shape does not fit."""
    hidden = heads * head_size
    flat = qkv.view(-1)
    ctx = torch.empty((batch * seq, 3 * hidden), dtype=torch.float16, device=qkv.device)
    rc = lib().cubert_attention_fused_split3_f32(_ptr(flat), _ptr(flat[hidden:]), _ptr(flat[2 * hidden:]), 3 * hidden,
                                                 _ptr(mask), float(scale), _ptr(ctx), float(alpha), batch, heads, seq, head_size,
                                                 _ptr(overflow), _stream())
    if rc == -2:
        return None
    _check(rc, "cubert_attention_fused_split3_f32")
    return ctx


def attention_context(probs, qkv, batch, heads, seq, head_size):
    """ctx[B*S, H] = P V with V the third column block of the packed projection."""
    hidden = heads * head_size
    flat = qkv.view(-1)
    ctx = torch.empty((batch * seq, hidden), dtype=qkv.dtype, device=qkv.device)
    fn = getattr(lib(), "cubert_attention_context_" + _suffix(qkv))
    rc = fn(_ptr(probs), _ptr(flat[2 * hidden:]), 3 * hidden, _ptr(ctx), hidden, batch, heads, seq, head_size,
            _stream())
    if rc == -2:
        return None
    _check(rc, fn.__name__)
    return ctx


def row_softmax(x, out=None):
    out = torch.empty_like(x) if out is None else out
    _call("cubert_row_softmax", x, _ptr(x), _ptr(out), x.shape[0], x.shape[1], _stream())
    return out


def bias_tanh_(inout, bias):
    _call("cubert_bias_tanh", inout, _ptr(inout), _ptr(bias), inout.shape[0], inout.shape[1], _stream())
    return inout


def mean_pool(x):
    batch, seq, hidden = x.shape
    out = torch.empty((batch, hidden), dtype=x.dtype, device=x.device)
    _call("cubert_mean_pool", x, _ptr(x), _ptr(out), batch, seq, hidden, _stream())
    return out


def classifier_head_(pooled, pooler_bias, weights, out_bias):
    """tanh(pooled + pooler_bias) in place (skipped without pooler_bias), logits = pooled W^T + out_bias and their
    softmax in one launch; returns (logits, probs), or None beyond 64 labels."""
    batch, hidden = pooled.shape
    labels = weights.shape[0]
    logits = torch.empty((batch, labels), dtype=pooled.dtype, device=pooled.device)
    probs = torch.empty_like(logits)
    fn = getattr(lib(), "cubert_classifier_head_" + _suffix(pooled))
    rc = fn(_ptr(pooled), _ptr(pooler_bias), _ptr(weights), _ptr(out_bias), _ptr(logits), _ptr(probs), batch, hidden,
            labels, _stream())
    if rc == -2:
        return None
    _check(rc, fn.__name__)
    return logits, probs


def split3(x, scale=1.0, lo_in_middle=False, overflow=None):
    """fp32 rows [rows, width] as fp16 rows [rows, 3 * width]: hi | hi | lo (lo_in_middle: hi | lo | hi)."""
    rows, width = x.shape
    out = torch.empty((rows, 3 * width), dtype=torch.float16, device=x.device)
    _check(lib().cubert_split3_f32(_ptr(x), rows, width, float(scale), int(lo_in_middle), _ptr(out), _ptr(overflow),
                                   _stream()),
           "cubert_split3_f32")
    return out


def bias_gelu_split3(x, bias, scale=1.0, overflow=None):
    """scale * GELU(x + bias) of fp32 rows as fp16 rows [rows, 3 * width]: hi | hi | lo."""
    rows, width = x.shape
    out = torch.empty((rows, 3 * width), dtype=torch.float16, device=x.device)
    _check(lib().cubert_bias_gelu_split3_f32(_ptr(x), _ptr(bias), rows, width, float(scale), _ptr(out),
                                             _ptr(overflow), _stream()),
           "cubert_bias_gelu_split3_f32")
    return out


def bias_res_ln_split3_(inout, residual, bias, beta, gamma, scale=1.0, overflow=None):
    """bias_res_ln_ of fp32 rows plus scale * the result as fp16 rows [rows, 3 * hidden]: hi | hi | lo; None when declined."""
    rows, hidden = inout.shape
    out = torch.empty((rows, 3 * hidden), dtype=torch.float16, device=inout.device)
    rc = lib().cubert_bias_res_ln_split3_f32(_ptr(inout), _ptr(residual), _ptr(bias), _ptr(beta), _ptr(gamma), rows,
                                             hidden, float(scale), _ptr(out), _ptr(overflow), _stream())
    if rc == -2:
        return None
    _check(rc, "cubert_bias_res_ln_split3_f32")
    return out


def transpose(x):
    """The transpose of a row-major 2-D tensor, as a new contiguous tensor."""
    rows, cols = x.shape
    out = torch.empty((cols, rows), dtype=x.dtype, device=x.device)
    _call("cubert_transpose", x, _ptr(x), rows, cols, _ptr(out), _stream())
    return out


class Blas(object):
    """A BLAS context of the runtime bound to torch's current stream."""

    def __init__(self):
        self.handle = lib().cubert_blas_create()
        if not self.handle:
            raise RuntimeError("cubert_blas_create failed")
        _check(lib().cubert_blas_set_stream(self.handle, _stream()), "cubert_blas_set_stream")

    def close(self):
        if self.handle:
            lib().cubert_blas_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown: module globals may already be gone
            pass

    def gemm(self, transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, bias=None):
        """Column-major C = alpha op(A) op(B) + beta C (+ bias per row of C) on flat tensors."""
        _call("cubert_gemm", C, self.handle, int(transA), int(transB), M, N, K, float(alpha), _ptr(A), lda, _ptr(B),
              ldb, float(beta), _ptr(C), ldc, _ptr(bias))
        return C

    def gemm_f16_f32(self, transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, bias=None):
        """The same with fp16 A and B and fp32 C and bias."""
        _check(lib().cubert_gemm_f16_f32(self.handle, int(transA), int(transB), M, N, K, float(alpha), _ptr(A), lda,
                                         _ptr(B), ldb, float(beta), _ptr(C), ldc, _ptr(bias)), "cubert_gemm_f16_f32")
        return C

    def gemm_skinny(self, M, N, K, alpha, A, lda, B, ldb, C, ldc, bias=None, gelu=False):
        """C = [gelu](alpha A B (+ bias)) with the few-token kernel (N <= 64); None when the problem does not fit."""
        fn = getattr(lib(), "cubert_gemm_skinny_" + _suffix(C))
        rc = fn(self.handle, M, N, K, float(alpha), _ptr(A), lda, _ptr(B), ldb, _ptr(C), ldc, _ptr(bias), int(gelu))
        if rc == -2:
            return None
        _check(rc, fn.__name__)
        return C

    def gemm_skinny_pack(self, A, lda, M, K):
        """The weight matrix A (M x K column-major, i.e. [K, M] row-major) in the few-token kernel's own order."""
        packed = torch.empty(lib().cubert_gemm_skinny_packed_elements(M, K), dtype=A.dtype, device=A.device)
        fn = getattr(lib(), "cubert_gemm_skinny_pack_" + _suffix(A))
        _check(fn(self.handle, _ptr(A), lda, M, K, _ptr(packed)), fn.__name__)
        return packed

    def gemm_skinny_packed(self, M, N, K, alpha, packed, B, ldb, C, ldc, bias=None, gelu=False):
        fn = getattr(lib(), "cubert_gemm_skinny_packed_" + _suffix(C))
        rc = fn(self.handle, M, N, K, float(alpha), _ptr(packed), _ptr(B), ldb, _ptr(C), ldc, _ptr(bias), int(gelu))
        if rc == -2:
            return None
        _check(rc, fn.__name__)
        return C

    def gemm_skinny_partials(self, M, N, K, A, lda, B, ldb, packed=False, partial_floats=1 << 20):
        """A B left as K slices: (partials[slices, N rounded up to 32, pitch] fp32, slices, pitch); None when the
        problem does not fit."""
        partials = torch.empty(partial_floats, dtype=torch.float32, device=B.device)
        slices, pitch = ctypes.c_int(0), ctypes.c_int(0)
        fn = getattr(lib(), "cubert_gemm_skinny_partials_" + _suffix(B))
        rc = fn(self.handle, M, N, K, _ptr(A), lda, int(packed), _ptr(B), ldb, _ptr(partials), partial_floats,
                ctypes.byref(slices), ctypes.byref(pitch))
        if rc == -2:
            return None
        _check(rc, fn.__name__)
        rows = (N + 31) // 32 * 32
        return (partials[:slices.value * rows * pitch.value].view(slices.value, rows, pitch.value), slices.value,
                pitch.value)

    def gemm_strided_batch(self, transA, transB, M, N, K, alpha, A, lda, sA, B, ldb, sB, beta, C, ldc, sC, batch):
        _call("cubert_gemm_strided_batch", C, self.handle, int(transA), int(transB), M, N, K, float(alpha), _ptr(A),
              lda, sA, _ptr(B), ldb, sB, float(beta), _ptr(C), ldc, sC, batch)
        return C

    def gemm_batch(self, transA, transB, M, N, K, alpha, As, lda, Bs, ldb, beta, Cs, ldc):
        """One problem per entry of As / Bs / Cs (lists of tensors, which may be views into larger buffers): the
        entry point takes device arrays of device pointers, built here (reference: blas_gemm_batch)."""
        def pointers(ts):
            return torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64).cuda()
        pa, pb, pc = pointers(As), pointers(Bs), pointers(Cs)
        _call("cubert_gemm_batch", Cs[0], self.handle, int(transA), int(transB), M, N, K, float(alpha), _ptr(pa), lda,
              _ptr(pb), ldb, float(beta), _ptr(pc), ldc, len(Cs))
        self._keep = (pa, pb, pc)  # the launch is asynchronous: the pointer arrays must outlive it
        return Cs
