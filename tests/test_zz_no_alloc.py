"""cubert_gemm_skinny_noalloc_f32, the few-token Dense kernel for callers that cannot allocate: its scratch (split-K
partial tiles and arrival counters) is a fixed array in the library's device image instead of a BLAS context's
allocation.  Through the C ABI it must give exactly what cubert_gemm_skinny_f32 gives (same kernel, same K slices,
sums in the same order: bit for bit), on two calls in a row, the second on a smaller problem, and keep doing so
when the two are interleaved; it must refuse problems beyond its stated capacity."""
import ctypes

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

NOALLOC_MAX_M, NOALLOC_MAX_K = 32768, 65536   # include/cubert_kernels.h
TOO_LARGE, BAD_ARGUMENT, UNSUPPORTED = -3, -1, -2


@pytest.fixture(scope="module")
def L():
    from cubert_amd._lib import lib
    import cubert_amd
    if cubert_amd.get_gpu_count() < 1:
        pytest.fail("no GPU visible: the -m gpu tests must run on the MI355X box")
    return lib()


class Device(object):
    """Device buffers for one problem, made with the library's own runtime calls (the test may allocate; the entry
    point under test may not)."""

    def __init__(self, L, *arrays):
        self.L = L
        self.ptrs = []
        for a in arrays:
            p = L.cubert_malloc(max(a.nbytes, 16))
            assert p
            assert L.cubert_memcpy(p, a.ctypes.data, a.nbytes, 1) == 0
            self.ptrs.append(p)

    def fetch(self, index, like):
        out = np.empty_like(like)
        assert self.L.cubert_memcpy(out.ctypes.data, self.ptrs[index], out.nbytes, 2) == 0
        return out

    def free(self):
        for p in self.ptrs:
            self.L.cubert_free(p)


def run_pair(L, handle, stream, M, N, K, activation, seed, with_bias=True):
    """The same problem through the handle-based entry point and through the one that allocates nothing."""
    rng = np.random.default_rng(seed)
    A = rng.normal(0, 0.05, (K, M)).astype(np.float32)     # weights [in, out]: column-major M x K, lda = M
    B = rng.normal(0, 1.0, (N, K)).astype(np.float32)      # N tokens of K values: column-major K x N, ldb = K
    bias = rng.normal(0, 0.1, M).astype(np.float32)
    poison = np.full((N, M), np.nan, np.float32)
    d = Device(L, A, B, bias, poison, poison)
    bias_ptr = d.ptrs[2] if with_bias else None
    rc = L.cubert_gemm_skinny_f32(handle, M, N, K, 1.0, d.ptrs[0], M, d.ptrs[1], K, d.ptrs[3], M, bias_ptr, activation)
    assert rc == 0, rc
    rc = L.cubert_gemm_skinny_noalloc_f32(stream, M, N, K, 1.0, d.ptrs[0], M, d.ptrs[1], K, d.ptrs[4], M, bias_ptr,
                                          activation)
    assert rc == 0, rc
    assert L.cubert_stream_synchronize(stream) == 0
    with_handle, without = d.fetch(3, poison), d.fetch(4, poison)
    d.free()
    assert np.isfinite(without).all()
    assert np.array_equal(with_handle.view(np.uint32), without.view(np.uint32)), \
        "M=%d N=%d K=%d: %g" % (M, N, K, np.abs(with_handle - without).max())
    # and both are the Dense layer the oracle computes (fp32 tolerance of the model tests)
    want = oracle.dense(B, A, bias if with_bias else np.zeros(M, np.float32))
    if activation == 1:
        want = oracle.gelu(want)
    err = np.abs(without - want).max() / max(np.abs(want).max(), 1e-30)
    assert err <= 1e-5, err
    return without


@pytest.fixture()
def context(L):
    stream = L.cubert_stream_create()
    handle = L.cubert_blas_create()
    assert stream and handle
    assert L.cubert_blas_set_stream(handle, stream) == 0
    yield handle, stream
    L.cubert_stream_synchronize(stream)
    L.cubert_blas_destroy(handle)
    L.cubert_stream_destroy(stream)


def test_two_calls_in_a_row_the_second_smaller(L, context):
    handle, stream = context
    # BERT-base feed-forward shapes at 32 tokens (K cut into slices: partial tiles and counters in use), then a
    # smaller problem that reuses the front of the same scratch
    run_pair(L, handle, stream, 3072, 32, 768, 1, seed=1)
    run_pair(L, handle, stream, 768, 64, 3072, 0, seed=6)      # two blocks of 32 tokens per wavefront
    run_pair(L, handle, stream, 768, 32, 3072, 0, seed=2)
    run_pair(L, handle, stream, 96, 5, 256, 0, seed=3)
    run_pair(L, handle, stream, 768, 32, 768, 0, seed=4, with_bias=False)
    run_pair(L, handle, stream, 40, 1, 16, 0, seed=5)          # one slice: no scratch at all, ragged feature block


def free_device_bytes(L):
    free = ctypes.c_size_t()
    assert L.cubert_mem_info(ctypes.byref(free), None) == 0
    return free.value


def test_calls_leave_free_device_memory_unchanged(L, context):
    """The headline property: after the first call on the device (which looks up the array's address) no call
    changes the amount of free device memory, whether it launches, is refused for its shape or for its size."""
    _, stream = context
    rng = np.random.default_rng(11)
    M, N, K = 768, 32, 3072
    A = rng.normal(0, 0.05, (K, M)).astype(np.float32)
    B = rng.normal(0, 1.0, (N, K)).astype(np.float32)
    d = Device(L, A, B, np.zeros((N, M), np.float32))

    def call(m, n, k):
        return L.cubert_gemm_skinny_noalloc_f32(stream, m, n, k, 1.0, d.ptrs[0], m, d.ptrs[1], k, d.ptrs[2], m, None, 0)

    # every kind of call once first: the first call on the device looks up the array's address, and a kernel variant's
    # first launch is the runtime's business, not this entry point's
    assert call(M, N, K) == 0
    assert call(96, 5, 256) == 0
    assert call(32, 65, 16) == UNSUPPORTED
    assert L.cubert_stream_synchronize(stream) == 0
    before = free_device_bytes(L)
    for _ in range(20):
        assert call(M, N, K) == 0
        assert call(96, 5, 256) == 0
        assert call(32, 65, 16) == UNSUPPORTED
    assert call(NOALLOC_MAX_M + 1, 1, 16) == TOO_LARGE
    assert L.cubert_stream_synchronize(stream) == 0
    assert free_device_bytes(L) == before
    d.free()


def test_back_to_back_launches_without_a_wait_between(L, context):
    """Ten launches of alternating shapes queued on one stream before anything is waited for: each finds the counters
    cleared and its partial tiles its own."""
    handle, stream = context
    rng = np.random.default_rng(7)
    shapes = [(768, 32, 3072), (2304, 32, 768), (768, 7, 768), (3072, 32, 768), (64, 32, 512)] * 2
    problems = []
    for M, N, K in shapes:
        A = rng.normal(0, 0.05, (K, M)).astype(np.float32)
        B = rng.normal(0, 1.0, (N, K)).astype(np.float32)
        out = np.zeros((N, M), np.float32)
        problems.append((M, N, K, A, B, Device(L, A, B, out)))
    for M, N, K, A, B, d in problems:
        assert L.cubert_gemm_skinny_noalloc_f32(stream, M, N, K, 0.5, d.ptrs[0], M, d.ptrs[1], K, d.ptrs[2], M, None, 0) == 0
    assert L.cubert_stream_synchronize(stream) == 0
    for M, N, K, A, B, d in problems:
        got = d.fetch(2, np.zeros((N, M), np.float32))
        want = 0.5 * (B.astype(np.float64) @ A.astype(np.float64))
        assert np.abs(got - want).max() / np.abs(want).max() <= 1e-5
        d.free()


def test_sizes_beyond_the_fixed_scratch_are_refused(L, context, capfd):
    _, stream = context
    d = Device(L, np.zeros(64, np.float32))
    p = d.ptrs[0]
    # refused on the host before anything is looked at or launched: the pointers are never dereferenced
    assert L.cubert_gemm_skinny_noalloc_f32(stream, NOALLOC_MAX_M + 1, 1, 16, 1.0, p, NOALLOC_MAX_M + 1, p, 16, p,
                                            NOALLOC_MAX_M + 1, None, 0) == TOO_LARGE
    assert "beyond what its fixed scratch array is sized for" in capfd.readouterr().err
    assert L.cubert_gemm_skinny_noalloc_f32(stream, 32, 1, NOALLOC_MAX_K + 16, 1.0, p, 32, p, NOALLOC_MAX_K + 16, p, 32,
                                            None, 0) == TOO_LARGE
    assert L.cubert_gemm_skinny_noalloc_f32(stream, 32, 1, 16, 1.0, None, 32, p, 16, p, 32, None, 0) == BAD_ARGUMENT
    assert L.cubert_gemm_skinny_noalloc_f32(stream, 32, 65, 16, 1.0, p, 32, p, 16, p, 32, None, 0) == UNSUPPORTED
    assert L.cubert_gemm_skinny_noalloc_f32(stream, 32, 1, 24, 1.0, p, 32, p, 24, p, 32, None, 0) == UNSUPPORTED
    assert L.cubert_stream_synchronize(stream) == 0
    d.free()
