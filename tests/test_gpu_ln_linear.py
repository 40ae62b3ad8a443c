"""GPU parity of Linear(LayerNorm(x)) with the normalisation folded into the GEMM (reference shader
shaders/fused-layernorm-linear.glsl:67-128: per-row mean / variance, then the product with the normalised row) and of its
gated form on the pre-norm MLP (gate * act(up) of LN(x), the ModernBERT branch of
utils/vulkan_sentence_transformer.py:799-970).  Truth: float64 LayerNorm followed by the float64 linear / gated
linear of the oracle on the same (bf16-rounded, for the bf16 path) x and W.  Shapes select every kernel that carries
the folded epilogue: the persistent 256x256 and 128x128 tile kernels (staged and direct stores), the register-staged
kernels (K rows that are not whole 128-byte slabs) and the scalar kernel (rows not 16-byte aligned).
Tolerances: max|y-ref|/max|ref| <= 1e-4 (fp32), <= 2e-2 (bf16)."""
import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16
from oracle import oracle_np as O
from grilly_amd import _lib as L

pytestmark = pytest.mark.gpu


def tol(dtype):
    return TOL_F32 if dtype == "fp32" else TOL_BF16


def q(dtype, a):
    return O.bf16_round(a) if dtype == "bf16" else a


def ln_linear(backend, dtype, x, g, bt, W, b, eps):
    """grl_ln_fold + grl_ln_gemm_nt through the C ABI; returns (y, stats, W_scaled, colsum, bias_folded)"""
    c = backend.core
    code = L.GRL_BF16 if dtype == "bf16" else L.GRL_F32
    es = 2 if dtype == "bf16" else 4
    M, K = x.shape
    N = W.shape[0]
    dx, dw, dg, dbt = c.upload(x, code), c.upload(W, code), c.upload(g), c.upload(bt)
    db = c.upload(b) if b is not None else None
    dws, dcs, dbf, dst, dy = c.alloc(N * K * es), c.alloc(N * 4), c.alloc(N * 4), c.alloc(M * 8), c.alloc(M * N * es)
    try:
        L.check(c.lib.grl_ln_fold(c.ctx, code, N, K, dw.ptr, dg.ptr, dbt.ptr, db.ptr if db else None, dws.ptr, dcs.ptr, dbf.ptr), "fold")
        L.check(c.lib.grl_ln_gemm_nt(c.ctx, code, code, M, N, K, dx.ptr, dws.ptr, dcs.ptr, dbf.ptr, float(eps), dst.ptr, dy.ptr), "gemm")
        return (c.download(dy, (M, N), code), c.download(dst, (M, 2)), c.download(dws, (N, K), code), c.download(dcs, (N,)),
                c.download(dbf, (N,)))
    finally:
        for t in (dx, dw, dg, dbt, db, dws, dcs, dbf, dst, dy):
            if t is not None:
                t.free()


def ln_glu(backend, dtype, x, g, bt, Wg, Wu, bg, bu, eps, act):
    c = backend.core
    code = L.GRL_BF16 if dtype == "bf16" else L.GRL_F32
    es = 2 if dtype == "bf16" else 4
    M, K = x.shape
    N = Wg.shape[0]
    bufs = [c.upload(x, code), c.upload(Wg, code), c.upload(Wu, code), c.upload(g), c.upload(bt), c.upload(bg), c.upload(bu)]
    dx, dwg, dwu, dg, dbt, dbg, dbu = bufs
    outs = [c.alloc(N * K * es), c.alloc(N * K * es), c.alloc(N * 4), c.alloc(N * 4), c.alloc(N * 4), c.alloc(N * 4), c.alloc(M * 8),
            c.alloc(M * N * es)]
    wgs, wus, cg, cu, dgf, duf, dst, dy = outs
    try:
        L.check(c.lib.grl_ln_fold(c.ctx, code, N, K, dwg.ptr, dg.ptr, dbt.ptr, dbg.ptr, wgs.ptr, cg.ptr, dgf.ptr), "fold gate")
        L.check(c.lib.grl_ln_fold(c.ctx, code, N, K, dwu.ptr, dg.ptr, dbt.ptr, dbu.ptr, wus.ptr, cu.ptr, duf.ptr), "fold up")
        L.check(c.lib.grl_ln_glu_nt(c.ctx, code, code, M, N, K, dx.ptr, wgs.ptr, wus.ptr, cg.ptr, cu.ptr, dgf.ptr, duf.ptr, float(eps),
                                    dst.ptr, dy.ptr, {"silu": L.EPI_SILU, "relu": L.EPI_RELU, "gelu": L.EPI_GELU}[act]), "ln_glu")
        return c.download(dy, (M, N), code)
    finally:
        for t in bufs + outs:
            t.free()


def make(rng, M, K, N, mean=0.0, scale=1.0):
    x = (rng.standard_normal((M, K)) * scale + mean).astype(np.float32)
    # rows with their own offset and spread, so that the statistics matter
    x = x * (0.5 + rng.random((M, 1))).astype(np.float32) + rng.standard_normal((M, 1)).astype(np.float32)
    W = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    g = (1.0 + 0.3 * rng.standard_normal(K)).astype(np.float32)
    bt = (0.3 * rng.standard_normal(K)).astype(np.float32)
    return x, W, b, g, bt


# (M, K, N, what it selects)
SHAPES = [
    (16384, 768, 768, "256x256 persistent tiles (192 of them), staged stores"),
    (16384 + 37, 768, 776, "256x256 tiles with a ragged row band and an 8-column edge tile"),
    (1000, 768, 2304, "128x128 persistent tiles"),
    (515, 768, 300, "128x128 tiles, rows of 600 / 1200 bytes: direct stores"),
    (300, 776, 200, "K rows that are not whole 128-byte slabs: register-staged kernel"),
    (16384, 776, 3072, "register-staged 256x256 kernel"),
    (70, 13, 9, "rows not 16-byte aligned: scalar kernel"),
    (5, 64, 1, "single output column"),
]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("M,K,N,what", SHAPES)
def test_ln_linear_parity(backend, dtype, M, K, N, what):
    rng = np.random.default_rng(M * 7 + K * 3 + N)
    x, W, b, g, bt = make(rng, M, K, N)
    x, W = q(dtype, x), q(dtype, W)
    eps = 1e-5
    y, stats, Ws, cs, bf = ln_linear(backend, dtype, x, g, bt, W, b, eps)
    rows = np.unique(np.concatenate([np.arange(0, M, max(1, M // 64)), [M - 1], rng.integers(0, M, 32)]))
    ref = O.truth_linear(O.truth_layernorm(x[rows], g, bt, eps), W, b)
    assert O.max_rel(y[rows], ref) < tol(dtype), what
    assert np.isfinite(y).all()
    # the pieces: statistics, scaled weight, column sums, folded bias
    x64 = x.astype(np.float64)
    mean = x64.mean(1)
    rstd = 1.0 / np.sqrt(x64.var(1) + eps)
    np.testing.assert_allclose(stats[:, 0], rstd, rtol=2e-5)
    np.testing.assert_allclose(stats[:, 1], rstd * mean, rtol=2e-5, atol=1e-5)
    Ws_ref = q(dtype, (g[None, :] * W).astype(np.float32))
    np.testing.assert_allclose(Ws, Ws_ref, rtol=1e-6 if dtype == "fp32" else 8e-3, atol=1e-7)
    np.testing.assert_allclose(cs, Ws.astype(np.float64).sum(1), rtol=1e-4, atol=2e-5)       # of the values as stored
    np.testing.assert_allclose(bf, b + W.astype(np.float64) @ bt.astype(np.float64), rtol=1e-4, atol=2e-5)
    # without bias
    y0 = ln_linear(backend, dtype, x, g, bt, W, None, eps)[0]
    ref0 = O.truth_linear(O.truth_layernorm(x[rows], g, bt, eps), W, None)
    assert O.max_rel(y0[rows], ref0) < tol(dtype)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_ln_linear_rows_far_from_zero(backend, dtype):
    """Row mean several spreads away from zero: the epilogue subtracts mean * column sum from the raw product, which
    must not cost the result its accuracy (fp32 accumulation; bf16 inputs already carry the offset's rounding)."""
    rng = np.random.default_rng(5)
    M, K, N = 777, 1024, 512
    x, W, b, g, bt = make(rng, M, K, N, mean=6.0, scale=1.0)
    x, W = q(dtype, x), q(dtype, W)
    y = ln_linear(backend, dtype, x, g, bt, W, b, 1e-5)[0]
    ref = O.truth_linear(O.truth_layernorm(x, g, bt, 1e-5), W, b)
    assert O.max_rel(y, ref) < (5e-4 if dtype == "fp32" else TOL_BF16)


def test_ln_linear_closed_forms(backend):
    # constant rows: variance 0, normalised row 0 -> out = bias + W.beta whatever gamma is.  The epilogue forms
    # rstd * (x.Ws - mean * c) with rstd = 1/sqrt(eps) = 316 here, so the fp32 rounding of the two products
    # (about 2^-23 * |mean| * sum|Ws| = 2e-5) comes back multiplied by 316: the bound below.
    K, N = 64, 8
    x = np.full((4, K), 3.25, np.float32)
    rng = np.random.default_rng(1)
    W = rng.standard_normal((N, K)).astype(np.float32)
    g, bt, b = rng.standard_normal(K).astype(np.float32), rng.standard_normal(K).astype(np.float32), rng.standard_normal(N).astype(np.float32)
    y = ln_linear(backend, "fp32", x, g, bt, W, b, 1e-5)[0]
    np.testing.assert_allclose(y, np.tile(b + W.astype(np.float64) @ bt, (4, 1)), rtol=1e-4, atol=1e-2)
    # gamma = 1, beta = 0, W = identity rows: out = the normalised row itself
    x = rng.standard_normal((6, K)).astype(np.float32)
    y = ln_linear(backend, "fp32", x, np.ones(K, np.float32), np.zeros(K, np.float32), np.eye(K, dtype=np.float32), None, 1e-5)[0]
    np.testing.assert_allclose(y, O.truth_layernorm(x, None, None, 1e-5), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(y.mean(1), 0, atol=1e-5)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("act", ["gelu", "silu", "relu"])
@pytest.mark.parametrize("M,K,N", [(16384, 768, 1152), (700, 768, 1152), (130, 776, 72), (33, 10, 5)])
def test_ln_glu_parity(backend, dtype, act, M, K, N):
    if M == 16384 and act != "gelu":
        pytest.skip("the large shape runs with the activation the pre-norm encoder uses")
    rng = np.random.default_rng(M + K + N + len(act))
    x, Wg, bg, g, bt = make(rng, M, K, N)
    Wu = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
    bu = rng.standard_normal(N).astype(np.float32)
    x, Wg, Wu = q(dtype, x), q(dtype, Wg), q(dtype, Wu)
    y = ln_glu(backend, dtype, x, g, bt, Wg, Wu, bg, bu, 1e-5, act)
    rows = np.unique(np.concatenate([np.arange(0, M, max(1, M // 48)), [M - 1]]))
    xn = O.truth_layernorm(x[rows], g, bt, 1e-5)
    ref = O.truth_fused_glu(xn, Wg, Wu, bg, bu, act)[0]
    assert O.max_rel(y[rows], ref) < tol(dtype)


def test_ln_linear_argument_errors(backend):
    c = backend.core
    with pytest.raises(ValueError):
        L.check(c.lib.grl_ln_gemm_nt(c.ctx, 0, 0, 4, 4, 8, None, None, None, None, 1e-5, None, None))
    with pytest.raises(ValueError):
        L.check(c.lib.grl_ln_stats(c.ctx, 7, 4, 8, None, 1e-5, None))
    with pytest.raises(ValueError):
        L.check(c.lib.grl_ln_fold(c.ctx, 0, 4, 0, None, None, None, None, None, None, None))
    # empty problems are no-ops
    L.check(c.lib.grl_ln_gemm_nt(c.ctx, 0, 0, 0, 4, 8, None, None, None, None, 1e-5, None, None))
    L.check(c.lib.grl_ln_fold(c.ctx, 0, 0, 8, None, None, None, None, None, None, None))


def test_gated_and_ln_folded_gemms_c_abi_randomized(backend):
    """Seeded sweep through ctypes of grl_glu_nt (gate and up caches on and off), grl_gemm_nt_res, grl_ln_gemm_nt and
    grl_ln_glu_nt: the four storage-type pairs where the entry point has them, the three gate activations, biases on and
    off, ragged shapes on both sides of the 256x256-tile threshold, K a whole number of 128-byte slabs or not; outputs and
    caches sit inside larger buffers whose surroundings must keep a sentinel."""
    from conftest import sweep_rounds
    c = backend.core
    rng = np.random.default_rng(55007)
    acts = [(L.EPI_SILU, "silu"), (L.EPI_RELU, "relu"), (L.EPI_GELU, "gelu")]
    PAD = 48

    def padded(n, code):
        return c.upload(np.full(n + 2 * PAD, 7.0, np.float32), code)

    def take(buf, n, code, info):
        es = 2 if code == L.GRL_BF16 else 4
        got = c.download(buf, (n + 2 * PAD,), code)
        assert (got[:PAD] == 7.0).all() and (got[PAD + n:] == 7.0).all(), info
        return got[PAD:PAD + n]

    for case in range(24 * sweep_rounds()):
        cin, cout = [(L.GRL_F32, L.GRL_F32), (L.GRL_BF16, L.GRL_BF16), (L.GRL_BF16, L.GRL_F32), (L.GRL_F32, L.GRL_BF16)][case % 4]
        es_out = 2 if cout == L.GRL_BF16 else 4
        q = (lambda a: O.bf16_round(a)) if cin == L.GRL_BF16 else (lambda a: a)
        t = TOL_F32 if (cin == L.GRL_F32 and cout == L.GRL_F32) else TOL_BF16
        K = int(rng.choice([16, 64, 96, 128, 264, 512]))
        if case % 7 == 6:                                      # >= 192 tiles of 256x256 (256x128 output tiles for the dual forms)
            M, N = int(rng.integers(3300, 3600)), int(rng.integers(1900, 2100))
        else:
            M, N = int(rng.integers(1, 500)), int(rng.integers(1, 400))
        x = q((rng.standard_normal((M, K)) * 1.5 + 0.3).astype(np.float32))
        W1 = q((rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))
        W2 = q((rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))
        bias = rng.random() < 0.6
        b1 = rng.standard_normal(N).astype(np.float32) if bias else None
        b2 = rng.standard_normal(N).astype(np.float32) if bias else None
        code, name = acts[int(rng.integers(0, 3))]
        what = case % 3
        info = (case, what, cin, cout, M, N, K, name, bias)
        dx, dw1, dw2 = c.upload(x, cin), c.upload(W1, cin), c.upload(W2, cin)
        db1, db2 = (c.upload(b1), c.upload(b2)) if bias else (None, None)
        dout = padded(M * N, cout)
        held = [dx, dw1, dw2, dout] + ([db1, db2] if bias else [])
        optr = dout.ptr + PAD * es_out
        try:
            if what == 0:                                      # gated GEMM, with or without the pre-activation caches
                caches = rng.random() < 0.5
                dg, du = (padded(M * N, L.GRL_F32), padded(M * N, L.GRL_F32)) if caches else (None, None)
                held += [dg, du] if caches else []
                L.check(c.lib.grl_glu_nt(c.ctx, cin, cout, M, N, K, dx.ptr, dw1.ptr, dw2.ptr, db1.ptr if bias else None, db2.ptr if bias else None,
                                         optr, dg.ptr + PAD * 4 if caches else None, du.ptr + PAD * 4 if caches else None, code), "glu_nt")
                ref, g, u = O.truth_fused_glu(x, W1, W2, b1, b2, name)
                y = take(dout, M * N, cout, info).reshape(M, N)
                assert O.max_rel(y, ref) < t, info + (O.max_rel(y, ref),)
                if caches:
                    tc = TOL_F32 if cin == L.GRL_F32 else TOL_BF16
                    assert O.max_rel(take(dg, M * N, L.GRL_F32, info).reshape(M, N), g) < tc, info
                    assert O.max_rel(take(du, M * N, L.GRL_F32, info).reshape(M, N), u) < tc, info
            elif what == 1:                                    # GEMM + residual of the output type
                r = (2.0 * rng.standard_normal((M, N))).astype(np.float32)
                if cout == L.GRL_BF16:
                    r = O.bf16_round(r)
                dr = c.upload(r, cout); held.append(dr)
                L.check(c.lib.grl_gemm_nt_res(c.ctx, cin, cout, M, N, K, dx.ptr, dw1.ptr, db1.ptr if bias else None, dr.ptr, optr), "gemm_nt_res")
                y = take(dout, M * N, cout, info).reshape(M, N)
                ref = O.truth_linear(x, W1, b1) + r.astype(np.float64)
                assert O.max_rel(y, ref) < t, info + (O.max_rel(y, ref),)
            else:                                              # LayerNorm folded into the GEMM / the gated GEMM
                gamma = (1 + 0.2 * rng.standard_normal(K)).astype(np.float32); beta = (0.2 * rng.standard_normal(K)).astype(np.float32)
                dgm, dbt = c.upload(gamma), c.upload(beta)
                es_in = 2 if cin == L.GRL_BF16 else 4
                ws1, ws2 = c.alloc(N * K * es_in), c.alloc(N * K * es_in)
                c1, c2, f1, f2 = (c.alloc(N * 4) for _ in range(4))
                stats = c.alloc(2 * M * 4 + 16)
                held += [dgm, dbt, ws1, ws2, c1, c2, f1, f2, stats]
                L.check(c.lib.grl_ln_fold(c.ctx, cin, N, K, dw1.ptr, dgm.ptr, dbt.ptr, db1.ptr if bias else None, ws1.ptr, c1.ptr, f1.ptr), "ln_fold")
                L.check(c.lib.grl_ln_fold(c.ctx, cin, N, K, dw2.ptr, dgm.ptr, dbt.ptr, db2.ptr if bias else None, ws2.ptr, c2.ptr, f2.ptr), "ln_fold")
                eps = 1e-5
                ln = O.truth_layernorm(x, gamma, beta, eps)
                gated = case % 2 == 0
                if gated:
                    L.check(c.lib.grl_ln_glu_nt(c.ctx, cin, cout, M, N, K, dx.ptr, ws1.ptr, ws2.ptr, c1.ptr, c2.ptr, f1.ptr, f2.ptr, eps, stats.ptr, optr, code), "ln_glu_nt")
                    ref = O.truth_fused_glu(ln, W1, W2, b1 if bias else np.zeros(N), b2 if bias else np.zeros(N), name)[0]
                else:
                    L.check(c.lib.grl_ln_gemm_nt(c.ctx, cin, cout, M, N, K, dx.ptr, ws1.ptr, c1.ptr, f1.ptr, eps, stats.ptr, optr), "ln_gemm_nt")
                    ref = O.truth_linear(ln, W1, b1)
                y = take(dout, M * N, cout, info).reshape(M, N)
                # the folded weight gamma*W is rounded to the storage type once more than the composed form rounds
                tl = t if cin == L.GRL_F32 else 1.5 * TOL_BF16
                assert O.max_rel(y, ref) < tl, info + (gated, O.max_rel(y, ref))
        finally:
            for b in held:
                if b is not None:
                    b.free()
        if case and case % 50 == 0:
            print("sweep case", case, flush=True)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_residual_gemm_statistics_feed_the_gated_gemm(backend, dtype):
    """The pre-norm layer's chain without a pass over the rows: grl_gemm_nt_resln with the identity in place of the
    LayerNorm on its residual (statistics {1, 0}, scale 1, shift 0) is the plain residual GEMM x + att.Wo^T + b,
    and the row statistics it writes drive grl_ln_glu_nt_stats to what grl_ln_glu_nt computes from its own pass."""
    import ctypes
    from grilly_amd import _lib as L
    c = backend.core
    code, es = (L.GRL_BF16, 2) if dtype == "bf16" else (L.GRL_F32, 4)
    rng = np.random.default_rng(31)
    M, d, ff, eps = 1000, 256, 320, 1e-5
    qd = (lambda a: O.bf16_round(a)) if dtype == "bf16" else (lambda a: a)
    att = qd(rng.standard_normal((M, d)).astype(np.float32))
    Wo = qd((rng.standard_normal((d, d)) / np.sqrt(d)).astype(np.float32))
    bo = rng.standard_normal(d).astype(np.float32)
    x = qd((1.5 * rng.standard_normal((M, d)) + rng.standard_normal((M, 1))).astype(np.float32))
    Wg, Wu = (qd((rng.standard_normal((ff, d)) / np.sqrt(d)).astype(np.float32)) for _ in range(2))
    bg, bu = (rng.standard_normal(ff).astype(np.float32) for _ in range(2))
    g, bt = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32), (0.1 * rng.standard_normal(d)).astype(np.float32)
    ident = np.zeros((M, 2), np.float32); ident[:, 0] = 1.0
    up = lambda a, cd=L.GRL_F32: c.upload(a, cd)
    datt, dWo, dbo, dx1, dx2 = up(att, code), up(Wo, code), up(bo), up(x, code), up(x, code)
    did, dones, dzeros = up(ident), up(np.ones(d, np.float32)), up(np.zeros(d, np.float32))
    dWg, dWu, dbg, dbu, dg, dbt = up(Wg, code), up(Wu, code), up(bg), up(bu), up(g), up(bt)
    st1, st2 = c.alloc(M * 8), c.alloc(M * 8)
    part = c.alloc(int(c.lib.grl_gemm_nt_resln_workspace(M, d)))
    wsg, wsu = c.alloc(ff * d * es), c.alloc(ff * d * es)
    csg, csu, bfg, bfu = (c.alloc(ff * 4) for _ in range(4))
    h1, h2 = c.alloc(M * ff * es), c.alloc(M * ff * es)
    bufs = [datt, dWo, dbo, dx1, dx2, did, dones, dzeros, dWg, dWu, dbg, dbu, dg, dbt, st1, st2, part, wsg, wsu, csg, csu, bfg, bfu, h1, h2]
    try:
        L.check(c.lib.grl_ln_fold(c.ctx, code, ff, d, dWg.ptr, dg.ptr, dbt.ptr, dbg.ptr, wsg.ptr, csg.ptr, bfg.ptr))
        L.check(c.lib.grl_ln_fold(c.ctx, code, ff, d, dWu.ptr, dg.ptr, dbt.ptr, dbu.ptr, wsu.ptr, csu.ptr, bfu.ptr))
        # route 1: residual GEMM, then the gated GEMM with its own statistics pass
        L.check(c.lib.grl_gemm_nt_res(c.ctx, code, code, M, d, d, datt.ptr, dWo.ptr, dbo.ptr, dx1.ptr, dx1.ptr))
        L.check(c.lib.grl_ln_glu_nt(c.ctx, code, code, M, ff, d, dx1.ptr, wsg.ptr, wsu.ptr, csg.ptr, csu.ptr, bfg.ptr, bfu.ptr, eps,
                                    st1.ptr, h1.ptr, L.EPI_GELU))
        # route 2: the statistics out of the residual GEMM's epilogue
        L.check(c.lib.grl_gemm_nt_resln(c.ctx, code, M, d, d, datt.ptr, dWo.ptr, dbo.ptr, dx2.ptr, did.ptr, dones.ptr, dzeros.ptr,
                                        dx2.ptr, eps, st2.ptr, part.ptr))
        L.check(c.lib.grl_ln_glu_nt_stats(c.ctx, code, code, M, ff, d, dx2.ptr, wsg.ptr, wsu.ptr, csg.ptr, csu.ptr, bfg.ptr, bfu.ptr,
                                          st2.ptr, h2.ptr, L.EPI_GELU))
        x1, x2 = c.download(dx1, (M, d), code), c.download(dx2, (M, d), code)
        # (the two entry points may pick different tile sizes, and the staged epilogue starts its sums from the bias where the
        # direct one adds it last: equal up to the last bit, not bit for bit)
        assert O.max_rel(x1, x2) < (2e-6 if dtype == "fp32" else 8e-3)
        # the statistics describe the rows as each route stored them (in bf16 the two differ by single roundings)
        for xs, st in ((x1, st1), (x2, st2)):
            got = c.download(st, (M, 2))
            mu, sd = xs.astype(np.float64).mean(-1), np.sqrt(xs.astype(np.float64).var(-1) + eps)
            assert O.max_rel(got[:, 0], 1 / sd) < 1e-4 and np.abs(got[:, 1] - mu / sd).max() < 1e-4 * max(1.0, np.abs(mu / sd).max())
        y1, y2 = c.download(h1, (M, ff), code), c.download(h2, (M, ff), code)
        tol = TOL_BF16 if dtype == "bf16" else TOL_F32
        assert O.max_rel(y2, y1) < tol * 0.5
        ref_x = O.truth_linear(att, Wo, bo) + x.astype(np.float64)
        xn = O.truth_layernorm(x2, g, bt, eps)
        ref = O.truth_linear(xn, Wg, bg) * O.truth_gelu(O.truth_linear(xn, Wu, bu))
        assert O.max_rel(x2, ref_x) < tol and O.max_rel(y2, ref) < tol * (1.5 if dtype == "bf16" else 1.0)
        assert c.lib.grl_ln_glu_nt_stats(c.ctx, code, code, M, ff, d, dx2.ptr, wsg.ptr, wsu.ptr, csg.ptr, csu.ptr, bfg.ptr, bfu.ptr,
                                         None, h2.ptr, L.EPI_GELU) == L.ERR_ARG
    finally:
        for b in bufs:
            b.free()
