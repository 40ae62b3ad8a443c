"""The allocation-free variant of gemm(A,B): grl_gemm_nn_noalloc keeps the transposed copy of B in a static
device array instead of a pool buffer.  Called through the C ABI and checked against grl_gemm_nn (equal to the last
bits, not bit for bit: for small products grl_gemm_nn shares the K loop out over several workgroups through a pool
buffer, which the allocation-free call must not touch, so the two add their partial sums in another grouping) and the
float64 oracle, on two calls in a row, the second with a smaller input (the
array still holds the first call's image), for both storage types; the size limit is an error, and the
caching pool sees no request during the calls."""
import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16
from oracle import oracle_np as O
from grilly_amd import _lib as L

pytestmark = pytest.mark.gpu


def _run(c, entry, code, A, B):
    M, K = A.shape
    N = B.shape[1]
    es = 2 if code == L.GRL_BF16 else 4
    da, db = c.upload(A, code), c.upload(B, code)
    dc = c.alloc(M * N * es)
    try:
        before = c.pool_stats()
        if entry == "noalloc":
            L.check(c.lib.grl_gemm_nn_noalloc(c.ctx, code, code, M, N, K, da.ptr, db.ptr, dc.ptr), "gemm_nn_noalloc")
            after = c.pool_stats()
            assert after["hits"] == before["hits"] and after["misses"] == before["misses"] and \
                after["allocations"] == before["allocations"], "the allocation-free entry point asked the pool"
        else:
            L.check(c.lib.grl_gemm_nn(c.ctx, code, code, M, N, K, da.ptr, db.ptr, dc.ptr, None), "gemm_nn")
        return c.download(dc, (M, N), code)
    finally:
        da.free(); db.free(); dc.free()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_gemm_nn_noalloc_matches_gemm_nn(backend, dtype):
    c = backend.core
    code = L.GRL_BF16 if dtype == "bf16" else L.GRL_F32
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    rng = np.random.default_rng(77)
    # first a B that fills a good part of the array (3072 x 1000), then a smaller, ragged one
    for (M, K, N) in [(640, 3072, 1000), (130, 264, 250), (33, 40, 17)]:
        A = rng.standard_normal((M, K)).astype(np.float32)
        B = (rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32)
        if dtype == "bf16":
            A, B = O.bf16_round(A), O.bf16_round(B)
        got = _run(c, "noalloc", code, A, B)
        want = _run(c, "pool", code, A, B)
        assert O.max_rel(got, want) < (1e-5 if dtype == "fp32" else 8e-3)
        assert O.max_rel(got, O.truth_gemm(A, B)) < tol


def test_gemm_nn_noalloc_limit_and_arguments(backend):
    c = backend.core
    lim = c.lib.grl_gemm_nn_noalloc_max_bytes()
    assert lim == 32 << 20
    K, N = 4096, lim // (4 * 4096) + 1            # one row of fp32 too many
    with c.alloc(16) as t:
        rc = c.lib.grl_gemm_nn_noalloc(c.ctx, L.GRL_F32, L.GRL_F32, 1, N, K, t.ptr, t.ptr, t.ptr)
        assert rc == L.ERR_SHAPE and "exceeds" in L.last_error()
        with pytest.raises(ValueError):
            L.check(rc)
        assert c.lib.grl_gemm_nn_noalloc(c.ctx, 9, L.GRL_F32, 1, 1, 1, t.ptr, t.ptr, t.ptr) == L.ERR_ARG
        assert c.lib.grl_gemm_nn_noalloc(c.ctx, L.GRL_F32, L.GRL_F32, 2, 2, 2, None, t.ptr, t.ptr) == L.ERR_ARG
        assert c.lib.grl_gemm_nn_noalloc(c.ctx, L.GRL_F32, L.GRL_F32, 0, 5, 5, None, None, None) == 0
    assert c.lib.grl_gemm_nn_noalloc(None, 0, 0, 1, 1, 1, None, None, None) == L.ERR_ARG


def test_concurrent_noalloc_gemm_on_one_context(backend):
    """Two threads call the allocation-free gemm(A,B) on one context with different B matrices: its two launches
    (transpose into the shared static array, GEMM out of it) must stay adjacent on the stream, so each thread gets
    the product with its own B."""
    import threading
    c = backend.core
    errors = []

    def worker(tid):
        try:
            rng = np.random.default_rng(900 + tid)
            M, K, N = 200 + 8 * tid, 512, 384
            A = rng.standard_normal((M, K)).astype(np.float32)
            B = (rng.standard_normal((K, N)) * (1.0 + tid)).astype(np.float32)
            want = O.truth_gemm(A, B)
            da, db = c.upload(A), c.upload(B)
            dc = c.alloc(M * N * 4)
            try:
                for r in range(40):
                    L.check(c.lib.grl_gemm_nn_noalloc(c.ctx, L.GRL_F32, L.GRL_F32, M, N, K, da.ptr, db.ptr, dc.ptr), "noalloc")
                    got = c.download(dc, (M, N))
                    assert O.max_rel(got, want) < TOL_F32, (tid, r)
            finally:
                da.free(); db.free(); dc.free()
        except Exception as e:
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(3)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors
