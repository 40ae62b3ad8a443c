"""One Compute() used from several Python threads at once.  The reference serialises every dispatch on one
queue and guards its buffer pool with a lock (backend/core.py:417-418, backend/buffer_pool.py:521-540); here
the calls interleave on the one context stream and share the caching pool, and each must still return its own
result (ctypes releases the GIL during the calls, so the library really is entered concurrently)."""
import threading

import numpy as np
import pytest

from conftest import TOL_F32
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu


def test_concurrent_calls_share_one_context(backend):
    errors, n_threads, rounds = [], 6, 8

    def worker(tid):
        try:
            rng = np.random.default_rng(100 + tid)
            for r in range(rounds):
                M, K, N = 64 + 8 * tid, 96 + 16 * r, 40 + 8 * tid
                x = rng.standard_normal((M, K)).astype(np.float32)
                W = rng.standard_normal((N, K)).astype(np.float32)
                b = rng.standard_normal(N).astype(np.float32)
                y = backend.fnn.fused_linear_gelu(x, W, b)
                assert O.max_rel(y, O.truth_linear(x, W, b, "gelu")) < TOL_F32, ("gelu", tid, r)
                g = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32)
                z = backend.fnn.layernorm(y, g, b)
                assert O.max_rel(z, O.truth_layernorm(y, g, b)) < TOL_F32, ("layernorm", tid, r)
                B, S, H, D = 2, 17 + tid, 2, 32
                q, k, v = (rng.standard_normal((B, S, H, D)).astype(np.float32) for _ in range(3))
                o = backend.attention.flash_attention2(q, k, v, H, D)
                assert O.max_rel(o, O.truth_attention(q, k, v)) < TOL_F32, ("attention", tid, r)
        except Exception as e:          # reported by the main thread
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=120)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors
    # every temporary went back to the pool: nothing of these calls is still counted as in use
    import gc
    gc.collect()
    before = backend.core.pool_stats()["bytes_in_use"]
    backend.fnn.linear(np.ones((4, 8), np.float32), np.ones((3, 8), np.float32))
    assert backend.core.pool_stats()["bytes_in_use"] == before


def test_shader_clock_probe(backend):
    """The probe kernel runs on its own stream beside the context's work and reports shader cycles over 100 MHz reference
    ticks: a plausible clock for this GPU, idle and beside a GEMM; bad durations are refused."""
    from grilly_amd import _lib as L
    c = backend.core
    c.sync()
    c.clock_probe_begin(2.0)
    idle = c.clock_probe_end()
    assert 0.05 < idle < 3.5, idle
    rng = np.random.default_rng(0)
    x = O.bf16_round(rng.standard_normal((8192, 1024)).astype(np.float32))
    w = O.bf16_round((rng.standard_normal((4096, 1024)) * 0.03).astype(np.float32))
    dx, dw = c.upload(x, L.GRL_BF16), c.upload(w, L.GRL_BF16)
    dy = c.alloc(8192 * 4096 * 2)
    try:
        run = lambda: L.check(c.lib.grl_gemm_nt(c.ctx, L.GRL_BF16, L.GRL_BF16, 8192, 4096, 1024, dx.ptr, dw.ptr, None, dy.ptr, L.EPI_NONE))
        run()
        c.sync()
        c.clock_probe_begin(3.0)
        for _ in range(60):
            run()
        busy = c.clock_probe_end()
        c.sync()
        assert 0.3 < busy < 3.5, busy
        # the GEMM beside the probe still computes what it should
        y = c.download(dy, (8192, 4096), L.GRL_BF16)
        rows = [0, 4097, 8191]
        assert O.max_rel(y[rows], O.truth_linear(x[rows], w, None)) < 2e-2
    finally:
        for t in (dx, dw, dy):
            t.free()
    with pytest.raises(ValueError):
        c.clock_probe_begin(0.0)
    with pytest.raises(ValueError):
        c.clock_probe_begin(1e6)
