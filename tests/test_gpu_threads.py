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
    # the C entry point refuses durations outside (0, 500] ms (the Python wrapper holds its argument inside that range),
    # and a reading without a probe started since the last one
    import ctypes
    assert c.lib.grl_clock_probe_begin(c.ctx, 0.0) == L.ERR_ARG
    assert c.lib.grl_clock_probe_begin(c.ctx, 1e6) == L.ERR_ARG
    ghz = ctypes.c_float()
    assert c.lib.grl_clock_probe_end(c.ctx, ctypes.byref(ghz)) == L.ERR_ARG
    c.clock_probe_begin(1e6)              # clamped to 500 ms by the wrapper... keep it short: read it at once
    assert 0.05 < c.clock_probe_end() < 3.5
    assert c.lib.grl_clock_probe_end(c.ctx, ctypes.byref(ghz)) == L.ERR_ARG


def test_concurrent_rope_attention_with_growing_lengths(backend):
    """Several threads call the fused-RoPE attention on one context while the sequence length keeps growing, so the
    cached cos / sin table is replaced by longer ones while other threads hold a pointer to the previous one between
    their lookup and their launch: a replaced table stays valid until the context goes away, and every call must
    return its own result."""
    errors = []
    lengths = [33, 150, 700, 1100, 1500, 2300]

    def worker(tid):
        try:
            rng = np.random.default_rng(500 + tid)
            order = lengths if tid % 2 == 0 else lengths[::-1]
            for S in order:
                B, H, D = 1, 2, 64
                q, k, v = (O.bf16_round(rng.standard_normal((B, S, H, D)).astype(np.float32)) for _ in range(3))
                style = "interleaved" if tid % 3 else "half"
                o = backend.attention.flash_attention2_rope(q, k, v, H, D, causal=bool(tid & 1), rope_style=style, dtype="bf16")
                ref = O.truth_attention(q, k, v, causal=bool(tid & 1), rope=style)
                assert O.max_rel(o, ref) < 2e-2, (tid, S)
        except Exception as e:
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=180)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert not errors, errors



def test_lap_events_and_matrix_core_probe(backend):
    """The two other measurement aids: lap events give the time between any two recorded points of the stream (in order,
    additive), and the register-resident MFMA loop reports its FLOP count and a plausible rate for every operand order
    and both instruction shapes, on zero and on caller-supplied operand bits."""
    import ctypes
    from grilly_amd import _lib as L
    c = backend.core
    x = c.upload(np.ones((512, 512), np.float32))
    y = c.alloc(512 * 512 * 4)
    ms = ctypes.c_float()
    try:
        for i in range(4):
            L.check(c.lib.grl_timer_lap(c.ctx, i))
            L.check(c.lib.grl_gemm_nt(c.ctx, L.GRL_F32, L.GRL_F32, 512, 512, 512, x.ptr, x.ptr, None, y.ptr, L.EPI_NONE))
        L.check(c.lib.grl_timer_lap(c.ctx, 4))
        parts = []
        for i in range(4):
            L.check(c.lib.grl_timer_lap_ms(c.ctx, i, i + 1, ctypes.byref(ms)))
            assert 0.0 < ms.value < 50.0
            parts.append(ms.value)
        L.check(c.lib.grl_timer_lap_ms(c.ctx, 0, 4, ctypes.byref(ms)))
        assert abs(sum(parts) - ms.value) < 0.02 + 0.05 * ms.value
        assert c.lib.grl_timer_lap(c.ctx, 256) == L.ERR_ARG and c.lib.grl_timer_lap(c.ctx, -1) == L.ERR_ARG
        assert c.lib.grl_timer_lap_ms(c.ctx, 0, 256, ctypes.byref(ms)) == L.ERR_ARG
        np.testing.assert_allclose(c.download(y, (512, 512)), 512.0)
    finally:
        x.free(); y.free()
    rng = np.random.default_rng(0)
    ops = c.upload(rng.standard_normal(32768).astype(np.float32), L.GRL_BF16)       # 64 KiB of bf16
    fl = ctypes.c_double()
    try:
        for kind in range(5):
            for ptr in (None, ops.ptr):
                L.check(c.lib.grl_mfma_probe(c.ctx, kind, ptr, 200, ctypes.byref(ms), ctypes.byref(fl)), "mfma_probe")
                cus = c.device_info()["compute_units"]
                assert fl.value == 200 * 2 * 128 * 64 * 2 * (32 if kind == 1 else 16) * 8 * cus
                rate = fl.value / (ms.value * 1e-3)
                assert 0.05e15 < rate < 2.7e15, (kind, ptr is None, rate)          # below the 2.5 PFLOP/s peak (+ timer slack)
        assert c.lib.grl_mfma_probe(c.ctx, 5, None, 10, ctypes.byref(ms), ctypes.byref(fl)) == L.ERR_ARG
        assert c.lib.grl_mfma_probe(c.ctx, 0, None, 0, ctypes.byref(ms), ctypes.byref(fl)) == L.ERR_ARG
        assert c.lib.grl_mfma_probe(c.ctx, 0, ops.ptr + 4, 10, ctypes.byref(ms), ctypes.byref(fl)) == L.ERR_ARG
        assert c.lib.grl_mfma_probe(c.ctx, 0, None, 10, None, ctypes.byref(fl)) == L.ERR_ARG
    finally:
        ops.free()
