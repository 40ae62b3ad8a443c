"""GPU parity of the HBM-bound kernels: LayerNorm(+residual), residual add, GELU, SiLU,
SwiGLU activation, casts, embedding gather, masked mean pooling."""
import ctypes

import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16
from oracle import oracle_np as O
from grilly_amd import _lib as L

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("shape", [(100,), (7, 384), (4, 16, 768), (3, 5, 1024), (2, 2048), (5, 2052), (9, 333), (2, 4100)])
def test_layernorm_parity(backend, corc, dtype, shape):
    rng = np.random.default_rng(sum(shape))
    x = (rng.standard_normal(shape) * 3 + 1).astype(np.float32)
    if dtype == "bf16":
        x = O.bf16_round(x)
    F = shape[-1]
    g = rng.standard_normal(F).astype(np.float32); b = rng.standard_normal(F).astype(np.float32)
    y = backend.fnn.layernorm(x, g, b, dtype=dtype)
    assert y.shape == x.shape
    assert O.max_rel(y, O.truth_layernorm(x, g, b)) < (TOL_F32 if dtype == "fp32" else TOL_BF16)
    if dtype == "fp32":
        assert O.max_rel(y, corc.layernorm(x, g, b)) < 1e-5
        y0 = backend.fnn.layernorm(x)          # gamma/beta default to ones/zeros; reference test: mean~0, std~1
        assert np.abs(y0.mean(-1)).max() < 1e-4 and np.abs(y0.std(-1) - 1).max() < 1e-2
        assert O.max_rel(backend.fnn.layernorm(x, g, b, eps=0.5), O.truth_layernorm(x, g, b, eps=0.5)) < TOL_F32


def test_layernorm_constant_row_and_rank_check(backend):
    beta = np.arange(16, dtype=np.float32)
    y = backend.fnn.layernorm(np.full((3, 16), 2.5, np.float32), np.ones(16), beta)
    np.testing.assert_allclose(y, np.tile(beta, (3, 1)), atol=1e-6)
    with pytest.raises(ValueError):
        backend.fnn.layernorm(np.zeros((2, 2, 2, 8), np.float32))
    with pytest.raises(ValueError):
        backend.fnn.layernorm(np.zeros((2, 8), np.float32), np.ones(7))


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_layernorm_with_residual_device_api(backend, dtype):
    # the fused residual+LayerNorm entry point the encoder layer uses, called on device pointers
    rng = np.random.default_rng(5)
    rows, F = 1000, 768
    x = rng.standard_normal((rows, F)).astype(np.float32); r = rng.standard_normal((rows, F)).astype(np.float32)
    if dtype == "bf16":
        x, r = O.bf16_round(x), O.bf16_round(r)
    g = rng.standard_normal(F).astype(np.float32); b = rng.standard_normal(F).astype(np.float32)
    c = backend.core
    code = L.GRL_BF16 if dtype == "bf16" else L.GRL_F32
    dx, dr, dg, db = c.upload(x, code), c.upload(r, code), c.upload(g), c.upload(b)
    L.check(c.lib.grl_layernorm(c.ctx, code, rows, F, dx.ptr, dr.ptr, dg.ptr, db.ptr, 1e-5, dx.ptr))    # in place
    y = c.download(dx, (rows, F), code)
    assert O.max_rel(y, O.truth_layernorm(x, g, b, residual=r)) < (TOL_F32 if dtype == "fp32" else TOL_BF16)
    for t in (dx, dr, dg, db):
        t.free()


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("n", [1, 5, 1023, 4096, 100003])
def test_elementwise_parity(backend, dtype, n):
    rng = np.random.default_rng(n)
    a = (rng.standard_normal(n) * 4).astype(np.float32); b = rng.standard_normal(n).astype(np.float32)
    if dtype == "bf16":
        a, b = O.bf16_round(a), O.bf16_round(b)
    t = TOL_F32 if dtype == "fp32" else TOL_BF16
    r = backend.fnn.residual(a, b, dtype=dtype)
    if dtype == "fp32":
        np.testing.assert_array_equal(r, a + b)                       # exact
    else:
        np.testing.assert_array_equal(r, O.bf16_round(a + b))         # one RNE rounding of the exact fp32 sum
    assert O.max_rel(backend.fnn.activation_gelu(a, dtype=dtype), O.truth_gelu(a)) < t
    assert O.max_rel(backend.fnn.activation_silu(a, dtype=dtype), O.truth_silu(a)) < t


def test_activation_edges(backend):
    x = np.array([0.0, 1.0, -1.0, 49.9, 50.1, -50.1, 88.5, -88.5, -200.0, 200.0], np.float32)
    g = backend.fnn.activation_gelu(x)
    assert g[0] == 0.0 and g[1] > 0                                  # reference tests/test_gpu_operations.py:109-118
    np.testing.assert_allclose(g, O.truth_gelu(x), rtol=1e-5, atol=1e-6)
    s = backend.fnn.activation_silu(x)
    np.testing.assert_allclose(s, O.truth_silu(x), rtol=1e-5, atol=1e-30)
    assert np.isfinite(s).all()


@pytest.mark.parametrize("shape", [(32,), (8, 64), (2, 3, 128), (5, 4098)])
def test_activation_swiglu(backend, shape):
    rng = np.random.default_rng(shape[-1])
    x = rng.standard_normal(shape).astype(np.float32)
    y = backend.fnn.activation_swiglu(x)
    h = shape[-1] // 2
    assert y.shape == shape[:-1] + (h,)
    x1, x2 = x[..., :h], x[..., h:]
    np.testing.assert_allclose(y, x1 * x2 / (1.0 + np.exp(-x2)), rtol=1e-5, atol=1e-6)      # reference test formula
    with pytest.raises(ValueError):
        backend.fnn.activation_swiglu(np.zeros((2, 5), np.float32))


def test_casts_are_rne(backend):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(5000).astype(np.float32) * 100,
                        np.array([1.00390625, 1.005859375, 0.0, -0.0, 3.3895314e38, 1e-39], np.float32)])
    c = backend.core
    d = c.upload(x, L.GRL_BF16)
    np.testing.assert_array_equal(c.download(d, x.shape, L.GRL_BF16), O.bf16_round(x))
    d.free()


def test_embed_and_mean_pool(backend):
    rng = np.random.default_rng(2)
    B, S, F, V = 3, 50, 384, 1000
    tok = rng.standard_normal((V, F)).astype(np.float32); pos = rng.standard_normal((64, F)).astype(np.float32)
    typ = rng.standard_normal((2, F)).astype(np.float32)
    ids = rng.integers(0, V, (B, S)).astype(np.int32)
    c = backend.core
    dt, dp, dty, di = c.upload(tok), c.upload(pos), c.upload(typ), c.upload_raw(ids)
    dx = c.alloc(B * S * F * 4)
    L.check(c.lib.grl_embed(c.ctx, L.GRL_F32, B, S, F, V, di.ptr, dt.ptr, dp.ptr, dty.ptr, dx.ptr))
    x = c.download(dx, (B, S, F))
    np.testing.assert_allclose(x, O.truth_embed(ids, tok, pos, typ), atol=1e-6)
    m = (np.arange(S)[None] < np.array([50, 1, 17])[:, None]).astype(np.float32)
    dm = c.upload(m); do = c.alloc(B * F * 4)
    L.check(c.lib.grl_mean_pool(c.ctx, L.GRL_F32, B, S, F, dx.ptr, dm.ptr, do.ptr, 1))
    assert O.max_rel(c.download(do, (B, F)), O.truth_mean_pool(x, m)) < 1e-5
    L.check(c.lib.grl_mean_pool(c.ctx, L.GRL_F32, B, S, F, dx.ptr, None, do.ptr, 0))
    assert O.max_rel(c.download(do, (B, F)), O.truth_mean_pool(x, None, l2=False)) < 1e-5
    for t in (dt, dp, dty, di, dx, dm, do):
        t.free()


@pytest.mark.parametrize("dtype,F", [("f32", 390), ("f32", 301), ("bf16", 768), ("bf16", 250), ("bf16", 37)])
def test_mean_pool_shapes(backend, dtype, F):
    """vector path (F % 4 == 0, also with a ragged last 256-feature block) and the any-F path"""
    rng = np.random.default_rng(F)
    B, S = 5, 77
    code = L.GRL_BF16 if dtype == "bf16" else L.GRL_F32
    x = rng.standard_normal((B, S, F)).astype(np.float32)
    if dtype == "bf16":
        x = O.bf16_round(x)
    m = (np.arange(S)[None] < np.array([77, 1, 40, 76, 3])[:, None]).astype(np.float32)
    c = backend.core
    dx, dm, do = c.upload(x, code), c.upload(m), c.alloc(B * F * 4)
    for l2 in (0, 1):
        L.check(c.lib.grl_mean_pool(c.ctx, code, B, S, F, dx.ptr, dm.ptr, do.ptr, l2))
        assert O.max_rel(c.download(do, (B, F)), O.truth_mean_pool(x, m, l2=bool(l2))) < 1e-5
    for t in (dx, dm, do):
        t.free()


def test_c_abi_argument_errors(backend):
    c = backend.core
    lib = c.lib
    buf = c.alloc(1024)
    assert lib.grl_gemm_nt(c.ctx, 5, 0, 4, 4, 4, buf.ptr, buf.ptr, None, buf.ptr, 0) == L.ERR_ARG
    assert lib.grl_gemm_nt(c.ctx, 0, 0, 4, 4, 4, buf.ptr, buf.ptr, None, buf.ptr, 9) == L.ERR_ARG
    assert lib.grl_gemm_nt(c.ctx, 0, 0, -1, 4, 4, buf.ptr, buf.ptr, None, buf.ptr, 0) == L.ERR_SHAPE
    assert lib.grl_gemm_nt(c.ctx, 0, 0, 4, 4, 4, None, buf.ptr, None, buf.ptr, 0) == L.ERR_ARG
    assert lib.grl_fa2_fwd(c.ctx, 0, 1, 8, 1, 2048, buf.ptr, buf.ptr, buf.ptr, None, buf.ptr, 1.0, 0, 0, 1e4, 1.0, None) == L.ERR_SHAPE
    assert "head_dim" in L.last_error()
    assert lib.grl_layernorm(c.ctx, 0, 4, 0, buf.ptr, None, buf.ptr, buf.ptr, 1e-5, buf.ptr) == L.ERR_SHAPE
    assert lib.grl_free(c.ctx, ctypes.c_void_p(12345)) == L.ERR_ARG          # foreign pointer
    # an impossible allocation reports out-of-memory instead of crashing
    assert lib.grl_malloc(c.ctx, 1 << 50) is None and "hipMalloc" in L.last_error()
    buf.free()
    info = backend.device_info()
    assert info["arch"].startswith("gfx950") and info["wavefront"] == 64 and info["compute_units"] > 0


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_gcu_roswish_softmax_activations(backend, dtype):
    """activation_gcu / activation_roswish / activation_softmax (reference backend/fnn.py:393-497, :574-700) and
    the reference's keyword name `input_data` on every activation."""
    rng = np.random.default_rng(31)
    x = (3 * rng.standard_normal((5, 7, 33))).astype(np.float32)
    if dtype == "bf16":
        x = O.bf16_round(x)
    t = TOL_F32 if dtype == "fp32" else TOL_BF16
    x64 = x.astype(np.float64)
    assert O.max_rel(backend.fnn.activation_gcu(input_data=x, dtype=dtype), x64 * np.cos(x64)) < t
    assert O.max_rel(backend.activation_roswish(x, alpha=0.7, beta=1.3, dtype=dtype), O.truth_roswish(x64, 0.7, 1.3)) < t
    for axis in (-1, 1, 0):
        e = np.exp(x64 - x64.max(axis=axis, keepdims=True))
        sm = backend.fnn.activation_softmax(x, axis=axis, dtype=dtype)
        assert sm.shape == x.shape and O.max_rel(sm, e / e.sum(axis=axis, keepdims=True)) < t
    np.testing.assert_allclose(backend.activation_softmax(np.array([1.0, 1.0, 1.0, 1.0], np.float32)), 0.25, rtol=1e-6)
    # keyword compatibility
    np.testing.assert_array_equal(backend.fnn.activation_gelu(input_data=x, dtype=dtype), backend.fnn.activation_gelu(x, dtype=dtype))
    np.testing.assert_array_equal(backend.fnn.activation_silu(input_data=x, dtype=dtype), backend.fnn.activation_silu(x, dtype=dtype))
    np.testing.assert_array_equal(backend.fnn.activation_relu(input_data=x, dtype=dtype), np.maximum(x, 0))
    x2 = x.reshape(5, 7 * 33)[:, :230]
    np.testing.assert_array_equal(backend.fnn.activation_swiglu(input_data=x2, dtype=dtype), backend.fnn.activation_swiglu(x2, dtype=dtype))


def test_gelu_epilogue_at_infinity_and_geglu_beyond_the_clip(backend):
    """fused GELU at +-inf follows the shader's |x| > 50 rule (x, 0); the gated GELU keeps the unclipped
    activation (the reference clips it at +-50, utils/vulkan_sentence_transformer.py:924-930: a documented deviation)."""
    s = np.array([np.inf, -np.inf, 1e30, -1e30, 60.0, -60.0], np.float32)
    x = np.zeros((len(s), 8), np.float32); x[:, 0] = s
    W = np.zeros((4, 8), np.float32); W[:, 0] = 1
    g = backend.fnn.fused_linear_gelu(np.nan_to_num(x, posinf=3e38, neginf=-3e38), W)[:, 0]
    np.testing.assert_array_equal(g, np.array([3e38, 0, 1e30, 0, 60, 0], np.float32))
    xg = np.zeros((2, 8), np.float32); xg[:, 0] = [60.0, 2.0]
    out = backend.fnn.fused_geglu(xg, W, W)[:, 0]            # gate * gelu(up), both 60 / 2
    np.testing.assert_allclose(out, [60.0 * 60.0, 2.0 * O.truth_gelu(np.array([2.0]))[0]], rtol=1e-5)


def test_rowwise_randomized_shapes(backend):
    """Seeded sweep over the row-wise kernels at random shapes (row widths from 1 to a few thousand, multiples of the
    16-byte vector and not, single rows and thousands): LayerNorm with random gamma / beta / eps and rows far from zero,
    softmax along the last axis with large spreads, rotate-half and interleaved RoPE with random position ids, GELU /
    SiLU / SwiGLU activations, and the three gated dual GEMMs; both dtypes, each against the float64 closed form."""
    from conftest import sweep_rounds
    rng = np.random.default_rng(55003)
    for case in range(40 * sweep_rounds()):
        dtype = "bf16" if case % 2 else "fp32"
        t = TOL_F32 if dtype == "fp32" else TOL_BF16
        q = (lambda a: O.bf16_round(a)) if dtype == "bf16" else (lambda a: a)
        what = case % 5
        rows = int(rng.choice([1, 2, 7, 65, 300, 3001]))
        F = int(rng.choice([1, 3, 8, 31, 64, 200, 384, 768, 1000, 1024, 2050, 4104]))
        if what == 0:
            # rows up to 20 standard deviations away from zero; narrow rows stay near it (among thousands of 3-element
            # rows some have a spread a hundred times below the scale, and offset / spread times the float ulp is the
            # conditioning of the fp32 normalisation itself, shader and kernel alike)
            off = rng.uniform(-20, 20) if F >= 8 else rng.uniform(-1, 1)
            x = q(((rng.standard_normal((rows, F)) + off) * rng.uniform(0.1, 5)).astype(np.float32))
            g = rng.standard_normal(F).astype(np.float32); b = rng.standard_normal(F).astype(np.float32)
            eps = float(rng.choice([1e-12, 1e-5, 1e-2]))
            if F == 1:
                continue                                   # a one-element row normalises to beta whatever the kernel does
            # (bf16 rows far from zero keep few bits of their deviations: the oracle sees the same rounded inputs)
            err = O.max_rel(backend.fnn.layernorm(x, g, b, eps=eps, dtype=dtype), O.truth_layernorm(x, g, b, eps))
        elif what == 1:
            x = q((rng.standard_normal((rows, F)) * rng.uniform(0.5, 30)).astype(np.float32))
            x64 = x.astype(np.float64)
            e = np.exp(x64 - x64.max(-1, keepdims=True))
            err = O.max_rel(backend.fnn.activation_softmax(x, dtype=dtype), e / e.sum(-1, keepdims=True))
        elif what == 2:
            B, S, H = int(rng.integers(1, 3)), int(rng.choice([1, 5, 130])), int(rng.integers(1, 4))
            D = int(rng.choice([2, 8, 32, 64, 96, 128]))
            style = "half" if case % 10 < 5 else "interleaved"
            x = q(rng.standard_normal((B, S, H, D)).astype(np.float32))
            pid = rng.integers(0, 4000, (B, S)) if rng.random() < 0.5 else None
            base, scaling = float(rng.choice([10000.0, 500.0])), float(rng.choice([1.0, 0.25, 8.0]))
            y = backend.attention.apply_rope(x, position_ids=pid, rope_base=base, rope_scaling=scaling, rope_style=style, dtype=dtype)
            err = O.max_rel(y, O.truth_rope(x, base, scaling, style, pid))
        elif what == 3:
            x = q((rng.standard_normal((rows, F)) * 3).astype(np.float32))
            err = max(O.max_rel(backend.fnn.activation_gelu(x, dtype=dtype), O.truth_gelu(x)),
                      O.max_rel(backend.fnn.activation_silu(x, dtype=dtype), O.truth_silu(x)))
            if F % 2 == 0:
                err = max(err, O.max_rel(backend.fnn.activation_swiglu(x, dtype=dtype), O.truth_swiglu_act(x)))
        else:
            M, K, N = min(rows, 400), 8 * int(rng.integers(1, 40)), int(rng.integers(1, 300))
            x = q(rng.standard_normal((M, K)).astype(np.float32))
            Wg = q((rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))
            Wu = q((rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))
            bias = rng.random() < 0.5
            bg = rng.standard_normal(N).astype(np.float32) if bias else None
            bu = rng.standard_normal(N).astype(np.float32) if bias else None
            act = ["silu", "relu", "gelu"][int(rng.integers(0, 3))]
            fn = {"silu": backend.fnn.fused_swiglu, "relu": backend.fnn.fused_reglu, "gelu": backend.fnn.fused_geglu}[act]
            err = O.max_rel(fn(x, Wg, Wu, bg, bu, dtype=dtype), O.truth_fused_glu(x, Wg, Wu, bg, bu, act)[0])
        assert err < t, (case, dtype, what, rows, F, err)
        if case and case % 50 == 0:
            print("sweep case", case, flush=True)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("F,tables", [(768, "all"), (384, "all"), (2048, "tok"), (36, "tok+pos"), (250, "all"), (2052, "all")])
def test_embed_layernorm_one_pass(backend, dtype, F, tables):
    """grl_embed_layernorm against grl_embed followed by grl_layernorm (same rows within an ulp of the storage type:
    the two LayerNorm kernels reduce in different lane orders) and against the float64 oracle; feature counts the
    one-pass kernel takes (multiples of 4 up to 2048) and those that run the two kernels, with and without the
    position / type tables."""
    c = backend.core
    code = L.GRL_BF16 if dtype == "bf16" else L.GRL_F32
    es = 2 if dtype == "bf16" else 4
    rng = np.random.default_rng(F)
    B, S, V = 3, 37, 101
    tok = rng.standard_normal((V, F)).astype(np.float32)
    pos = rng.standard_normal((S, F)).astype(np.float32) if tables != "tok" else None
    typ = rng.standard_normal((2, F)).astype(np.float32) if tables == "all" else None
    g = (1 + 0.2 * rng.standard_normal(F)).astype(np.float32); b = (0.2 * rng.standard_normal(F)).astype(np.float32)
    ids = rng.integers(0, V, (B, S)).astype(np.int32)
    dtok, dg, db, dids = c.upload(tok), c.upload(g), c.upload(b), c.upload_raw(ids)
    dpos = c.upload(pos) if pos is not None else None
    dtyp = c.upload(typ) if typ is not None else None
    x1, x2 = c.alloc(B * S * F * es), c.alloc(B * S * F * es)
    pp, tp = (dpos.ptr if dpos else None), (dtyp.ptr if dtyp else None)
    try:
        L.check(c.lib.grl_embed_layernorm(c.ctx, code, B, S, F, V, dids.ptr, dtok.ptr, pp, tp, dg.ptr, db.ptr, 1e-5, x1.ptr), "embed_layernorm")
        L.check(c.lib.grl_embed(c.ctx, code, B, S, F, V, dids.ptr, dtok.ptr, pp, tp, x2.ptr), "embed")
        L.check(c.lib.grl_layernorm(c.ctx, code, B * S, F, x2.ptr, None, dg.ptr, db.ptr, 1e-5, x2.ptr), "layernorm")
        y1, y2 = c.download(x1, (B, S, F), code), c.download(x2, (B, S, F), code)
    finally:
        for t in (dtok, dg, db, dids, dpos, dtyp, x1, x2):
            if t is not None:
                t.free()
    e = tok[ids].astype(np.float64) + (typ[0] if typ is not None else 0.0) + (pos[None] if pos is not None else 0.0)
    if dtype == "bf16":
        e = O.bf16_round(e.astype(np.float32)).astype(np.float64)
    ref = O.truth_layernorm(e, g, b, 1e-5)
    t = TOL_F32 if dtype == "fp32" else TOL_BF16
    assert O.max_rel(y1, ref) < t and O.max_rel(y2, ref) < t
    np.testing.assert_allclose(y1, y2, rtol=2.0 ** -7 if dtype == "bf16" else 1e-5, atol=2.0 ** -9 if dtype == "bf16" else 1e-6)


def test_embedding_lookup_and_mean_pool_facade(backend):
    """numpy-in / numpy-out `learning.embedding_lookup` (reference backend/learning.py:811-877, shaders/embedding-lookup.glsl:
    out-of-range ids give zero rows, 1-D ids are one batch entry) and `pooling.mean_pool` (backend/pooling.py:22-143,
    shaders/embedding-pool.glsl: the mask is a 0.5 threshold, a sequence without kept positions pools to zeros)."""
    rng = np.random.default_rng(31)
    for (B, S, V, F) in [(3, 17, 50, 384), (2, 5, 9, 7), (1, 1, 1, 1), (4, 64, 300, 768)]:
        table = rng.standard_normal((V, F)).astype(np.float32)
        ids = rng.integers(0, V, (B, S))
        out = backend.learning.embedding_lookup(ids, table)
        assert out.dtype == np.float32 and out.shape == (B, S, F)
        np.testing.assert_array_equal(out, table[ids])
        np.testing.assert_array_equal(backend.embedding_lookup(ids[0], table), table[ids[0]][None])      # 1-D ids, Compute delegate
        bad = ids.copy(); bad[0, 0] = V; bad[-1, -1] = -1
        got = backend.learning.embedding_lookup(bad, table)
        want = table[np.clip(bad, 0, V - 1)]; want[0, 0] = 0; want[-1, -1] = 0
        np.testing.assert_array_equal(got, want)
        x = rng.standard_normal((B, S, F)).astype(np.float32)
        np.testing.assert_allclose(backend.pooling.mean_pool(x), x.astype(np.float64).mean(1), rtol=1e-5, atol=1e-6)
        mask = (rng.random((B, S)) < 0.6).astype(np.float32)
        mask[0] = 0                                     # nothing kept: zeros
        if B > 1:
            mask[1] = np.where(np.arange(S) % 2, 0.51, 0.49)    # threshold, not weight
        keep = (mask > 0.5)
        cnt = keep.sum(1, keepdims=True)
        want = np.where(cnt > 0, (x.astype(np.float64) * keep[..., None]).sum(1) / np.maximum(cnt, 1), 0.0)
        got = backend.pooling.mean_pool(x, mask)
        assert got.dtype == np.float32 and got.shape == (B, F)
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        backend.pooling.mean_pool(np.zeros((2, 3), np.float32))
    with pytest.raises(ValueError):
        backend.pooling.mean_pool(np.zeros((2, 3, 4), np.float32), np.zeros((2, 4), np.float32))
    with pytest.raises(ValueError):
        backend.learning.embedding_lookup(np.zeros((2, 3), np.int64), np.zeros(5, np.float32))
