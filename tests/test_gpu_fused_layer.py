"""The LayerNorm-free form of the post-LN layer (reference recipe utils/vulkan_sentence_transformer.py:972-1035):
`grl_ln_gemm_nt_stats` (a GEMM that reads LayerNorm(x) without x ever being normalised in memory, statistics given),
`grl_gemm_nt_resln` (a GEMM that adds LayerNorm(R) re-formed from raw rows and writes the row statistics of its own
output) and `grl_bert_layer_fwd_fused` built from them, each through the C ABI against the float64 oracle of the
unfused formulas, plus the fused encoder against the seven-launch one.
Tolerances: max|y-ref|/max|ref| <= 1e-4 (fp32), <= 2e-2 (bf16)."""
import ctypes

import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16, sweep_rounds
from oracle import oracle_np as O
from grilly_amd import _lib as L
from grilly_amd import BertEncoder, EncoderConfig, random_bert_weights

pytestmark = pytest.mark.gpu


def _code(dtype):
    return L.GRL_BF16 if dtype == "bf16" else L.GRL_F32


def _q(dtype, a):
    return O.bf16_round(a) if dtype == "bf16" else a


def _stats(x, eps):
    x = x.astype(np.float64)
    mu = x.mean(-1)
    sd = np.sqrt(x.var(-1) + eps)
    return np.stack([1 / sd, mu / sd], -1)


# (M, K, N): 256x256 tiles with ragged edges / 128x128 tiles / a single small tile
SHAPES = [(4096 + 37, 768, 3072 + 8), (8192, 3072, 768), (300, 128, 200), (64, 64, 8)]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("epi", ["none", "gelu"])
@pytest.mark.parametrize("M,K,N", SHAPES)
def test_ln_gemm_with_given_statistics(backend, dtype, epi, M, K, N):
    c, code = backend.core, _code(dtype)
    if dtype == "fp32" and K % 32 or dtype == "bf16" and K % 64:
        pytest.skip("K is not a whole number of 128-byte slabs for this type")
    rng = np.random.default_rng(M + K + N)
    x = _q(dtype, (rng.standard_normal((M, K)) * 1.5 + 0.7 * rng.standard_normal((M, 1))).astype(np.float32))
    W = _q(dtype, (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))
    g = (1 + 0.2 * rng.standard_normal(K)).astype(np.float32)
    bt = (0.3 * rng.standard_normal(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    eps = 1e-5
    es = 2 if dtype == "bf16" else 4
    dx, dw, dg, dbt, db = c.upload(x, code), c.upload(W, code), c.upload(g), c.upload(bt), c.upload(b)
    ws, cs, bf, st, out = c.alloc(N * K * es), c.alloc(N * 4), c.alloc(N * 4), c.alloc(M * 8), c.alloc(M * N * es)
    try:
        L.check(c.lib.grl_ln_fold(c.ctx, code, N, K, dw.ptr, dg.ptr, dbt.ptr, db.ptr, ws.ptr, cs.ptr, bf.ptr), "fold")
        L.check(c.lib.grl_ln_stats(c.ctx, code, M, K, dx.ptr, eps, st.ptr), "stats")
        L.check(c.lib.grl_ln_gemm_nt_stats(c.ctx, code, code, M, N, K, dx.ptr, ws.ptr, cs.ptr, bf.ptr, st.ptr, out.ptr,
                                           L.EPI_GELU if epi == "gelu" else L.EPI_NONE), "ln_gemm_nt_stats")
        y = c.download(out, (M, N), code)
        rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 40)]))
        # the weight the kernel multiplies by is gamma*W rounded to the storage type
        wsq = _q(dtype, (W.astype(np.float64) * g[None, :]).astype(np.float32)).astype(np.float64)
        xs = x[rows].astype(np.float64)
        mu, sd = xs.mean(-1, keepdims=True), np.sqrt(xs.var(-1, keepdims=True) + eps)
        pre = ((xs - mu) / sd) @ wsq.T + (b + W.astype(np.float64) @ bt)
        ref = O.truth_gelu(pre) if epi == "gelu" else pre
        assert np.isfinite(y).all()
        assert O.max_rel(y[rows], ref) < (TOL_BF16 if dtype == "bf16" else TOL_F32)
        # and it is the LayerNorm + linear of the unfused chain (weights unrounded) within the bf16 tolerance
        ref2 = O.truth_linear(O.truth_layernorm(x[rows], g, bt, eps), W, b, epi)
        assert O.max_rel(y[rows], ref2) < (TOL_BF16 if dtype == "bf16" else TOL_F32)
    finally:
        for t in (dx, dw, dg, dbt, db, ws, cs, bf, st, out):
            t.free()
    with c.alloc(64) as t:
        assert c.lib.grl_ln_gemm_nt_stats(c.ctx, code, code, 1, 8, 64, t.ptr, t.ptr, t.ptr, t.ptr, t.ptr, t.ptr, L.EPI_SILU) == L.ERR_ARG


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("inplace", [False, True])
@pytest.mark.parametrize("M,K,N", SHAPES)
def test_gemm_with_layernormed_residual_and_row_statistics(backend, dtype, inplace, M, K, N):
    c, code = backend.core, _code(dtype)
    if dtype == "fp32" and K % 32 or dtype == "bf16" and K % 64:
        pytest.skip("K is not a whole number of 128-byte slabs for this type")
    rng = np.random.default_rng(7 * M + K + N)
    A = _q(dtype, rng.standard_normal((M, K)).astype(np.float32))
    W = _q(dtype, (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))
    b = rng.standard_normal(N).astype(np.float32)
    R = _q(dtype, (2.0 * rng.standard_normal((M, N)) + rng.standard_normal((M, 1))).astype(np.float32))
    g = (1 + 0.2 * rng.standard_normal(N)).astype(np.float32)
    bt = (0.3 * rng.standard_normal(N)).astype(np.float32)
    eps_r, eps = 1e-5, 1e-6
    rst = _stats(R, eps_r).astype(np.float32)
    es = 2 if dtype == "bf16" else 4
    dA, dW, db, dR, dst, dg, dbt = c.upload(A, code), c.upload(W, code), c.upload(b), c.upload(R, code), c.upload(rst), c.upload(g), c.upload(bt)
    dC = dR if inplace else c.alloc(M * N * es)
    so = c.alloc(M * 8)
    wk = c.alloc(c.lib.grl_gemm_nt_resln_workspace(M, N))
    try:
        L.check(c.lib.grl_gemm_nt_resln(c.ctx, code, M, N, K, dA.ptr, dW.ptr, db.ptr, dR.ptr, dst.ptr, dg.ptr, dbt.ptr, dC.ptr,
                                        eps, so.ptr, wk.ptr), "gemm_nt_resln")
        y = c.download(dC, (M, N), code)
        stats = c.download(so, (M, 2))
        rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 40)]))
        ref = O.truth_linear(A[rows], W, b) + O.truth_layernorm(R[rows], g, bt, eps_r)
        tol = TOL_BF16 if dtype == "bf16" else TOL_F32
        assert np.isfinite(y).all() and np.isfinite(stats).all()
        assert O.max_rel(y[rows], ref) < tol
        # statistics of the rows as written (every row): they feed the next LayerNorm-folded GEMM
        want = _stats(y, eps)
        assert O.max_rel(stats[:, 0], want[:, 0]) < (5e-3 if dtype == "bf16" else 1e-4)
        assert np.abs(stats[:, 1] - want[:, 1]).max() < (5e-3 if dtype == "bf16" else 1e-4) * max(1.0, np.abs(want[:, 1]).max())
        # a second run is bit-identical (partials are merged in a fixed order)
        if not inplace:
            L.check(c.lib.grl_gemm_nt_resln(c.ctx, code, M, N, K, dA.ptr, dW.ptr, db.ptr, dR.ptr, dst.ptr, dg.ptr, dbt.ptr, dC.ptr,
                                            eps, so.ptr, wk.ptr), "gemm_nt_resln")
            np.testing.assert_array_equal(c.download(dC, (M, N), code), y)
            np.testing.assert_array_equal(c.download(so, (M, 2)), stats)
    finally:
        for t in (dA, dW, db, dR, dst, dg, dbt, so, wk):
            t.free()
        if not inplace:
            dC.free()


def test_resln_rejects_what_the_staged_kernels_do_not_take(backend):
    c = backend.core
    with c.alloc(4096) as t:
        args = (t.ptr, t.ptr, None, t.ptr, t.ptr, t.ptr, t.ptr, t.ptr, 1e-5, t.ptr, t.ptr)
        assert c.lib.grl_gemm_nt_resln(c.ctx, L.GRL_F32, 4, 8, 24, *args) == L.ERR_SHAPE            # K not a whole slab
        assert c.lib.grl_gemm_nt_resln(c.ctx, L.GRL_BF16, 4, 12, 64, *args) == L.ERR_SHAPE          # rows of 24 bytes
        assert c.lib.grl_gemm_nt_resln(c.ctx, L.GRL_F32, 4, 8, 32, t.ptr, None, None, *args[3:]) == L.ERR_ARG
        assert c.lib.grl_gemm_nt_resln(c.ctx, L.GRL_F32, 0, 8, 32, *args) == 0
        f = L.BertLayerFused()
        assert c.lib.grl_bert_layer_fwd_fused(c.ctx, L.GRL_F32, 1, 4, 2, 8, 64, ctypes.byref(f), None, 1e-5, t.ptr, t.ptr, t.ptr) == L.ERR_ARG
    assert c.lib.grl_bert_layer_fused_workspace(L.GRL_F32, 2, 16, 2, 32, 128) > 0
    cfg = EncoderConfig(layers=1, d_model=48, heads=3, d_ff=96, vocab=50, max_pos=16)
    with pytest.raises(ValueError):
        BertEncoder(backend, cfg, random_bert_weights(cfg, seed=0), dtype="bf16", fused=True)
    assert BertEncoder(backend, cfg, random_bert_weights(cfg, seed=0), dtype="bf16").fused is False


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("d,heads,ff,S", [(128, 4, 512, 40), (768, 12, 3072, 512), (384, 12, 1536, 100)])
def test_fused_encoder_equals_the_unfused_one(backend, dtype, d, heads, ff, S):
    """Both layer forms against the float64 oracle, with non-trivial biases and LayerNorm parameters (the fused form
    folds gamma into weights and beta into biases) and a padding mask; and against each other."""
    cfg = EncoderConfig(layers=2, d_model=d, heads=heads, d_ff=ff, vocab=300, max_pos=512)
    w = random_bert_weights(cfg, seed=d + S)
    rng = np.random.default_rng(d + S)
    w["emb_ln_g"] = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    w["emb_ln_b"] = (0.1 * rng.standard_normal(d)).astype(np.float32)
    for lw in w["layers"]:
        for k in ("b_qkv", "b_o", "b_ff1", "b_ff2", "ln1_b", "ln2_b"):
            lw[k] = (rng.standard_normal(lw[k].shape) * 0.05).astype(np.float32)
        for k in ("ln1_g", "ln2_g"):
            lw[k] = (1 + rng.standard_normal(lw[k].shape) * 0.1).astype(np.float32)
    B = 3
    ids = rng.integers(0, cfg.vocab, (B, S))
    lens = np.array([S, max(1, S // 3), S - 1])
    mask = (np.arange(S)[None] < lens[:, None]).astype(np.float32)
    fused = BertEncoder(backend, cfg, w, dtype=dtype, fused=True)
    plain = BertEncoder(backend, cfg, w, dtype=dtype, fused=False)
    assert fused.fused and not plain.fused
    hf, hp = fused.forward(ids, mask, pool=False), plain.forward(ids, mask, pool=False)
    quant = O.bf16_round if dtype == "bf16" else None
    qf = (lambda a: a) if quant is None else (lambda a: quant(np.asarray(a, np.float32)).astype(np.float64))
    x = qf(O.truth_layernorm(qf(O.truth_embed(ids, w["tok_emb"], w["pos_emb"], w["type_emb"])), w["emb_ln_g"], w["emb_ln_b"], cfg.eps))
    for lw in w["layers"]:
        lq = {k: (quant(v) if (quant and k.startswith("w_")) else v) for k, v in lw.items()}
        x = O.truth_bert_layer(x, lq, mask, heads, cfg.eps, quant)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    assert np.isfinite(hf).all()
    assert O.max_rel(hp, x) < tol
    assert O.max_rel(hf, x) < tol
    assert O.max_rel(hf, hp) < tol
    pf, pp = fused.forward(ids, mask, pool=True), plain.forward(ids, mask, pool=True)
    assert O.max_rel(pf, pp) < (1e-4 if dtype == "fp32" else 1e-2)
    fused.release_activations(); plain.release_activations()


@pytest.mark.parametrize("fused", [True, False])
def test_lap_trace_marks_every_launch_of_the_layers(backend, fused):
    """With a lap trace on, each layer call records a lap at entry and after each of its kernels (five with the folded
    LayerNorms, seven without); the intervals are non-negative and add up to the time between the first and the last
    lap; with the trace off the layers record nothing; the hidden states do not depend on the trace."""
    c = backend.core
    cfg = EncoderConfig(layers=3, d_model=128, heads=2, d_ff=256, vocab=100, max_pos=64)
    w = random_bert_weights(cfg, seed=5)
    enc = BertEncoder(backend, cfg, w, dtype="bf16", fused=fused)
    rng = np.random.default_rng(5)
    ids = rng.integers(0, cfg.vocab, (4, 40))
    want = enc.forward(ids, None, pool=False)
    per_layer = (5 if fused else 7) + 1
    nxt, ms = ctypes.c_int(123), ctypes.c_float()
    L.check(c.lib.grl_timer_lap_trace(c.ctx, -1, ctypes.byref(nxt)))
    assert nxt.value == -1                                  # no trace was on
    L.check(c.lib.grl_timer_lap_trace(c.ctx, 10, None))
    got = enc.forward(ids, None, pool=False)
    L.check(c.lib.grl_timer_lap_trace(c.ctx, -1, ctypes.byref(nxt)))
    assert nxt.value == 11 + per_layer * cfg.layers
    np.testing.assert_array_equal(got, want)
    parts = []
    for i in range(10, nxt.value - 1):
        L.check(c.lib.grl_timer_lap_ms(c.ctx, i, i + 1, ctypes.byref(ms)))
        assert ms.value >= 0.0
        parts.append(ms.value)
    L.check(c.lib.grl_timer_lap_ms(c.ctx, 10, nxt.value - 1, ctypes.byref(ms)))
    assert abs(sum(parts) - ms.value) < 0.05 + 0.05 * ms.value
    # off again: a forward leaves the next index alone
    enc.forward(ids, None, pool=False)
    L.check(c.lib.grl_timer_lap_trace(c.ctx, -1, ctypes.byref(nxt)))
    assert nxt.value == -1
    # marks past the last event index are dropped, the forward still runs
    L.check(c.lib.grl_timer_lap_trace(c.ctx, 250, None))
    np.testing.assert_array_equal(enc.forward(ids, None, pool=False), want)
    L.check(c.lib.grl_timer_lap_trace(c.ctx, -1, ctypes.byref(nxt)))
    assert nxt.value == 256
    assert c.lib.grl_timer_lap_trace(c.ctx, 256, None) == L.ERR_ARG
    assert c.lib.grl_timer_lap_trace(c.ctx, -2, None) == L.ERR_ARG
    assert c.lib.grl_timer_lap_trace(None, 0, None) == L.ERR_ARG
    enc.release_activations()


def test_resln_and_given_statistics_gemms_randomized(backend):
    """Seeded sweep over the two GEMM entry points of the LayerNorm-free layer through the C ABI: both storage types,
    ragged M, widths in 16-byte steps, one to six K slabs, big-tile and small-tile launches, with and without a bias,
    in place and out of place; outputs against float64 on every row, row statistics against the moments of the stored
    rows.  GRILLY_SWEEP_ROUNDS continues the stream."""
    c = backend.core
    rng = np.random.default_rng(4242)
    worst = {"fp32": 0.0, "bf16": 0.0}
    for case in range(36 * sweep_rounds()):
        if case and case % 50 == 0:
            print("sweep case", case, flush=True)
        dtype = "bf16" if case % 2 else "fp32"
        code, es = _code(dtype), (2 if dtype == "bf16" else 4)
        slab, chunk = (64, 8) if dtype == "bf16" else (32, 4)
        K = slab * int(rng.integers(1, 7))
        if case % 6 == 0:                                   # enough 256 x 256 tiles for the persistent big-tile kernels
            M, N = int(rng.integers(3100, 4300)), chunk * int(rng.integers(3100 // chunk, 4300 // chunk))
            while ((M + 255) // 256) * ((N + 255) // 256) < 192:
                N += 256
        else:
            M, N = int(rng.integers(1, 700)), chunk * int(rng.integers(1, 700 // chunk))
        tol = TOL_BF16 if dtype == "bf16" else TOL_F32
        eps_r, eps = 1e-5, 1e-6
        has_bias, inplace = rng.random() < 0.7, rng.random() < 0.5
        A = _q(dtype, rng.standard_normal((M, K)).astype(np.float32))
        W = _q(dtype, (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))
        b = rng.standard_normal(N).astype(np.float32) if has_bias else None
        R = _q(dtype, (rng.uniform(0.3, 3.0) * rng.standard_normal((M, N)) + rng.standard_normal((M, 1))).astype(np.float32))
        g = (1 + 0.2 * rng.standard_normal(N)).astype(np.float32)
        bt = (0.3 * rng.standard_normal(N)).astype(np.float32)
        rst = _stats(R, eps_r).astype(np.float32)
        tag = (case, dtype, M, K, N, has_bias, inplace)
        dA, dW, dR, dst, dg, dbt = c.upload(A, code), c.upload(W, code), c.upload(R, code), c.upload(rst), c.upload(g), c.upload(bt)
        db = c.upload(b) if has_bias else None
        dC = dR if inplace else c.alloc(M * N * es)
        so, wk = c.alloc(M * 8), c.alloc(c.lib.grl_gemm_nt_resln_workspace(M, N))
        # second entry point: y2 = LN(y; g2, bt2) . W2^T + b2 from the statistics the first one wrote
        N2 = chunk * int(rng.integers(1, 40))
        K2ok = N % slab == 0                                # its K is the first one's N: whole slabs only
        try:
            L.check(c.lib.grl_gemm_nt_resln(c.ctx, code, M, N, K, dA.ptr, dW.ptr, db.ptr if db else None, dR.ptr, dst.ptr, dg.ptr, dbt.ptr,
                                            dC.ptr, eps, so.ptr, wk.ptr), f"gemm_nt_resln {tag}")
            y = c.download(dC, (M, N), code)
            stats = c.download(so, (M, 2))
            ref = O.truth_linear(A, W, b) + O.truth_layernorm(R, g, bt, eps_r)
            assert np.isfinite(y).all() and np.isfinite(stats).all(), tag
            err = O.max_rel(y, ref)
            worst[dtype] = max(worst[dtype], err)
            assert err < tol, (tag, err)
            want = _stats(y, eps)
            stol = 5e-3 if dtype == "bf16" else 2e-4
            assert O.max_rel(stats[:, 0], want[:, 0]) < stol, tag
            assert np.abs(stats[:, 1] - want[:, 1]).max() < stol * max(1.0, np.abs(want[:, 1]).max()), tag
            if K2ok:
                W2 = _q(dtype, (rng.standard_normal((N2, N)) / np.sqrt(N)).astype(np.float32))
                g2 = (1 + 0.2 * rng.standard_normal(N)).astype(np.float32)
                bt2 = (0.3 * rng.standard_normal(N)).astype(np.float32)
                b2 = rng.standard_normal(N2).astype(np.float32)
                epi = "gelu" if rng.random() < 0.5 else "none"
                dW2, dg2, dbt2, db2 = c.upload(W2, code), c.upload(g2), c.upload(bt2), c.upload(b2)
                ws, cs, bf, out = c.alloc(N2 * N * es), c.alloc(N2 * 4), c.alloc(N2 * 4), c.alloc(M * N2 * es)
                try:
                    L.check(c.lib.grl_ln_fold(c.ctx, code, N2, N, dW2.ptr, dg2.ptr, dbt2.ptr, db2.ptr, ws.ptr, cs.ptr, bf.ptr), "fold")
                    L.check(c.lib.grl_ln_gemm_nt_stats(c.ctx, code, code, M, N2, N, dC.ptr, ws.ptr, cs.ptr, bf.ptr, so.ptr, out.ptr,
                                                       L.EPI_GELU if epi == "gelu" else L.EPI_NONE), f"ln_gemm_nt_stats {tag}")
                    y2 = c.download(out, (M, N2), code)
                    ref2 = O.truth_linear(O.truth_layernorm(y, g2, bt2, eps), W2, b2, epi)
                    assert np.isfinite(y2).all(), tag
                    err2 = O.max_rel(y2, ref2)
                    assert err2 < tol * (1.5 if dtype == "bf16" else 2.0), (tag, N2, epi, err2)
                finally:
                    for t in (dW2, dg2, dbt2, db2, ws, cs, bf, out):
                        t.free()
        finally:
            for t in (dA, dW, dR, dst, dg, dbt, so, wk):
                t.free()
            if db:
                db.free()
            if not inplace:
                dC.free()
    print("worst", worst)
