"""GPU parity of the GEMM family against the oracle (float64 closed form of the reference
shaders), called through the numpy facade which goes through the C ABI.
Tolerances: max|y-ref|/max|ref| <= 1e-4 on the fp32 path, <= 2e-2 on the bf16 path."""
import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16, rng_for
from oracle import oracle_np as O
from grilly_amd import _lib as L

pytestmark = pytest.mark.gpu


def tol(dtype):
    return TOL_F32 if dtype == "fp32" else TOL_BF16


def prep(dtype, *arrs):
    """the bf16 path's oracle consumes the bf16-rounded inputs"""
    return [O.bf16_round(a) if dtype == "bf16" else a for a in arrs]


SHAPES = [
    (32, 384, 128),      # BASELINE config 1
    (1, 8, 4), (3, 16, 5), (33, 40, 17), (64, 128, 256),      # reference test_gemm_backward shape + ragged edges
    (130, 264, 250), (257, 72, 513), (300, 2056, 129),
    (1024, 384, 1536),   # MiniLM FFN1 slice
    (2048, 768, 768), (4096, 768, 2304),                      # BERT-base out-proj / QKV (big-tile kernel)
]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("M,K,N", SHAPES)
def test_linear_parity(backend, dtype, M, K, N):
    rng = np.random.default_rng(M * 7 + K * 3 + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = rng.standard_normal((N, K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    x, W = prep(dtype, x, W)
    y = backend.fnn.linear(x, W, b, dtype=dtype)
    assert y.shape == (M, N) and y.dtype == np.float32 and y.flags.c_contiguous
    assert O.max_rel(y, O.truth_linear(x, W, b)) < tol(dtype)
    y0 = backend.fnn.linear(x, W, dtype=dtype)
    assert O.max_rel(y0, O.truth_linear(x, W)) < tol(dtype)


def test_config1_linear_then_swiglu(backend, corc):
    # BASELINE config 1: x[32,384].W[384,128]+b (W given as (in,out) -> passed transposed), then swiglu
    rng = rng_for(1)
    x = rng.standard_normal((32, 384)).astype(np.float32)
    W = rng.standard_normal((384, 128)).astype(np.float32)
    b = np.zeros(128, np.float32)
    y = backend.fnn.linear(x, W.T.copy(), b)
    assert O.max_rel(y, x.astype(np.float64) @ W.astype(np.float64)) < TOL_F32
    assert O.max_rel(y, corc.linear(x, W.T.copy(), b)) < TOL_F32          # shader-order fp32 restatement
    z = backend.fnn.activation_swiglu(y)
    assert z.shape == (32, 64)
    assert O.max_rel(z, O.truth_swiglu_act(y)) < TOL_F32


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("epi", ["gelu", "silu"])
@pytest.mark.parametrize("M,K,N", [(5, 24, 7), (129, 136, 260), (2048, 768, 3072)])
def test_fused_linear_parity(backend, dtype, epi, M, K, N):
    rng = np.random.default_rng(11 + M + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((N, K)) * 0.2).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    x, W = prep(dtype, x, W)
    fn = backend.fnn.fused_linear_gelu if epi == "gelu" else backend.fnn.fused_linear_silu
    y = fn(x, W, b, dtype=dtype)
    assert O.max_rel(y, O.truth_linear(x, W, b, epi)) < tol(dtype)


def test_fused_epilogue_clamp_edges(backend):
    # drive the pre-activation to the +-50 (gelu) and +-88 (silu) edges through a 1-wide GEMM
    s = np.array([0.0, 1.0, -1.0, 49.5, 50.5, -49.5, -50.5, 87.0, 89.0, -87.0, -89.0, -120.0, 300.0], np.float32)
    x = np.zeros((len(s), 8), np.float32); x[:, 0] = s
    W = np.zeros((4, 8), np.float32); W[:, 0] = 1
    g = backend.fnn.fused_linear_gelu(x, W)
    np.testing.assert_allclose(g[:, 0], O.truth_gelu(s), rtol=1e-5, atol=1e-6)
    assert g[0, 0] == 0.0 and g[4, 0] == 50.5 and g[6, 0] == 0.0
    si = backend.fnn.fused_linear_silu(x, W)
    np.testing.assert_allclose(si[:, 0], O.truth_silu_clamped(s), rtol=1e-5, atol=1e-30)
    ga = backend.fnn.activation_gelu(s)
    np.testing.assert_allclose(ga, O.truth_gelu(s), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("M,K,N,bias", [(6, 20, 10, True), (70, 72, 33, False), (513, 264, 130, True), (2048, 512, 1408, False)])
def test_fused_swiglu_parity(backend, dtype, M, K, N, bias):
    rng = np.random.default_rng(M + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    Wg = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    Wu = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    bg = rng.standard_normal(N).astype(np.float32) if bias else None
    bu = rng.standard_normal(N).astype(np.float32) if bias else None
    x, Wg, Wu = prep(dtype, x, Wg, Wu)
    t_out, t_g, t_u = O.truth_fused_swiglu(x, Wg, Wu, bg, bu)
    out, g, u = backend.fnn.fused_swiglu(x, Wg, Wu, bg, bu, return_cache=True, dtype=dtype)
    assert out.shape == (M, N)
    assert O.max_rel(out, t_out) < tol(dtype)
    assert O.max_rel(g, t_g) < tol(dtype) and O.max_rel(u, t_u) < tol(dtype)
    out2 = backend.fnn.fused_swiglu(x, Wg, Wu, bg, bu, dtype=dtype)
    np.testing.assert_array_equal(out2, out)          # deterministic, cache stores do not disturb the result
    # a single bias is ignored, as in the reference
    np.testing.assert_array_equal(backend.fnn.fused_swiglu(x, Wg, Wu, bg, None, dtype=dtype),
                                  backend.fnn.fused_swiglu(x, Wg, Wu, dtype=dtype))


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("epi", ["relu", "gcu", "roswish"])
@pytest.mark.parametrize("M,K,N", [(5, 24, 7), (129, 136, 260), (1024, 768, 1536)])
def test_further_fused_linear_parity(backend, dtype, epi, M, K, N):
    rng = np.random.default_rng(17 + M + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    x, W = prep(dtype, x, W)
    if epi == "relu":
        y = backend.fnn.fused_linear_relu(x, W, b, dtype=dtype)
    elif epi == "gcu":
        y = backend.fnn.fused_linear_gcu(x, W, b, dtype=dtype)
    else:
        y = backend.fnn.fused_linear_roswish(x, W, b, alpha=0.7, beta=1.3, dtype=dtype)
    assert y.shape == (M, N)
    assert O.max_rel(y, O.truth_linear(x, W, b, epi, 0.7, 1.3)) < tol(dtype)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("act", ["relu", "gelu"])
@pytest.mark.parametrize("M,K,N,bias", [(6, 20, 10, True), (513, 264, 130, False), (1024, 512, 1408, True)])
def test_reglu_geglu_parity(backend, dtype, act, M, K, N, bias):
    rng = np.random.default_rng(M + N + 3)
    x = rng.standard_normal((M, K)).astype(np.float32)
    Wg = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    Wu = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    bg = rng.standard_normal(N).astype(np.float32) if bias else None
    bu = rng.standard_normal(N).astype(np.float32) if bias else None
    x, Wg, Wu = prep(dtype, x, Wg, Wu)
    t_out, t_g, t_u = O.truth_fused_glu(x, Wg, Wu, bg, bu, act)
    fn = backend.fnn.fused_reglu if act == "relu" else backend.fnn.fused_geglu
    out, g, u = fn(x, Wg, Wu, bg, bu, return_cache=True, dtype=dtype)
    assert out.shape == (M, N)
    assert O.max_rel(out, t_out) < tol(dtype)
    assert O.max_rel(g, t_g) < 1e-4 and O.max_rel(u, t_u) < 1e-4
    assert O.max_rel(fn(x, Wg, Wu, bg, bu, dtype=dtype), t_out) < tol(dtype)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_fused_layernorm_linear(backend, dtype):
    rng = np.random.default_rng(23)
    x = rng.standard_normal((3, 50, 768)).astype(np.float32)
    W = (rng.standard_normal((300, 768)) * 0.05).astype(np.float32)
    b = rng.standard_normal(300).astype(np.float32)
    g, bt = rng.standard_normal(768).astype(np.float32), rng.standard_normal(768).astype(np.float32)
    x, W = prep(dtype, x, W)
    y = backend.fnn.fused_layernorm_linear(x, g, bt, W, b, eps=1e-5, dtype=dtype)
    assert y.shape == (3, 50, 300)
    ref = O.truth_linear(O.truth_layernorm(x, g, bt, 1e-5), W, b)
    assert O.max_rel(y, ref) < tol(dtype)


def test_further_epilogue_edges(backend):
    s = np.array([0.0, np.pi, -np.pi, 2.0, -3.0, 60.0, -60.0, 200.0, -200.0], np.float32)
    x = np.zeros((len(s), 8), np.float32); x[:, 0] = s
    W = np.zeros((4, 8), np.float32); W[:, 0] = 1
    np.testing.assert_array_equal(backend.fnn.fused_linear_relu(x, W)[:, 0], np.maximum(s, 0))
    np.testing.assert_allclose(backend.fnn.fused_linear_gcu(x, W)[:, 0], O.truth_linear(x, W, None, "gcu")[:, 0], rtol=1e-5, atol=1e-5)
    ro = backend.fnn.fused_linear_roswish(x, W, alpha=0.8, beta=1.5)[:, 0]
    np.testing.assert_allclose(ro, O.truth_roswish(s, 0.8, 1.5), rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        L.check(backend.core.lib.grl_gemm_nt(backend.core.ctx, 0, 0, 1, 1, 1, None, None, None, None, 6))
    with pytest.raises(ValueError):
        L.check(backend.core.lib.grl_glu_nt(backend.core.ctx, 0, 0, 1, 1, 1, None, None, None, None, None, None, None, None, 4))


def test_fused_swiglu_always_2d_and_config4_convention(backend):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 5, 16)).astype(np.float32)
    Wg = rng.standard_normal((12, 16)).astype(np.float32); Wu = rng.standard_normal((12, 16)).astype(np.float32)
    out = backend.fnn.fused_swiglu(x, Wg, Wu)
    assert out.shape == (10, 12)
    # BASELINE config 4 wants silu(x.Wg)*(x.Wu): pass W_gate:=Wu, W_up:=Wg
    want = O.truth_silu(x.reshape(10, 16).astype(np.float64) @ Wg.T) * (x.reshape(10, 16).astype(np.float64) @ Wu.T)
    assert O.max_rel(backend.fnn.fused_swiglu(x, Wu, Wg), want) < TOL_F32


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_gemm_nn_and_transposed_view(backend, dtype):
    rng = np.random.default_rng(8)
    A = rng.standard_normal((65, 40)).astype(np.float32)
    B = rng.standard_normal((40, 77)).astype(np.float32)
    A, B = prep(dtype, A, B)
    assert O.max_rel(backend.fnn.gemm(A, B, dtype=dtype), O.truth_gemm(A, B)) < tol(dtype)
    W = np.ascontiguousarray(B.T)                 # nn.Linear calls gemm(x, W.T) with a transposed view
    assert O.max_rel(backend.fnn.gemm(A, W.T, dtype=dtype), O.truth_gemm(A, B)) < tol(dtype)
    if dtype == "fp32":
        np.testing.assert_array_equal(backend.fnn.gemm(np.array([[1, 2], [3, 4]], np.float32), np.array([[5, 6], [7, 8]], np.float32)),
                                      np.array([[19, 22], [43, 50]], np.float32))     # reference tests/test_pytorch_ops.py:42-48


def test_qkv_projection_equals_three_linears(backend):
    rng = np.random.default_rng(9)
    H, D, K = 4, 32, 96
    x = rng.standard_normal((3, 7, K)).astype(np.float32)
    Ws = [rng.standard_normal((H * D, K)).astype(np.float32) * 0.1 for _ in range(3)]
    bs = [rng.standard_normal(H * D).astype(np.float32) for _ in range(3)]
    qkv = backend.fnn.fused_qkv_projection(x, np.concatenate(Ws), np.concatenate(bs), num_heads=H, head_dim=D)
    assert qkv.shape == (3, 7, 3 * H * D)
    for i in range(3):
        assert O.max_rel(qkv[..., i * H * D:(i + 1) * H * D], O.truth_linear(x, Ws[i], bs[i])) < TOL_F32
    with pytest.raises(ValueError):
        backend.fnn.fused_qkv_projection(x, np.concatenate(Ws), None, num_heads=5, head_dim=D)


def test_shapes_dtypes_and_errors(backend):
    rng = np.random.default_rng(10)
    W = rng.standard_normal((6, 8)).astype(np.float32)
    x3 = rng.standard_normal((2, 3, 8))                       # float64 in -> float32 out, leading dims kept
    y = backend.fnn.linear(x3, W)
    assert y.shape == (2, 3, 6) and y.dtype == np.float32
    assert O.max_rel(y, O.truth_linear(x3, W)) < TOL_F32
    assert backend.fnn.fused_linear_gelu(x3[0, 0], W).shape == (1, 6)     # rank-1 -> (1,N) (reference fnn.py:2055-2060)
    assert backend.fnn.fused_linear_silu(x3, W).shape == (2, 3, 6)
    xs = np.asfortranarray(rng.standard_normal((5, 8)).astype(np.float32))   # non-contiguous input is copied
    assert O.max_rel(backend.fnn.linear(xs, W), O.truth_linear(xs, W)) < TOL_F32
    before = x3.copy(); backend.fnn.linear(x3, W); np.testing.assert_array_equal(x3, before)   # inputs untouched
    with pytest.raises(ValueError):
        backend.fnn.linear(rng.standard_normal((4, 7)), W)
    with pytest.raises(ValueError):
        backend.fnn.linear(x3, W, np.zeros(5))
    with pytest.raises(AssertionError):
        backend.fnn.gemm(np.zeros((2, 3)), np.zeros((4, 5)))
    with pytest.raises(ValueError):
        backend.fnn.linear(x3, W, dtype="fp16")
    assert backend.fnn.linear(np.zeros((0, 8), np.float32), W).shape == (0, 6)      # empty batch


def test_full_size_properties_bert_ffn1(backend):
    # BASELINE config 3 shape (one GEMM at full size, bf16): linearity + a row-sample against the oracle
    rng = rng_for(3)
    M, K, N = 65536, 768, 3072
    x = O.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    W = O.bf16_round((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
    y = backend.fnn.linear(x, W, dtype="bf16")
    rows = rng.integers(0, M, 64)
    assert O.max_rel(y[rows], O.truth_linear(x[rows], W)) < TOL_BF16
    # scaling the input by 2 (exact in bf16) scales the output by exactly 2
    y2 = backend.fnn.linear(2 * x[:4096], W, dtype="bf16")
    np.testing.assert_array_equal(y2, 2 * y[:4096])
    # every tile was written: no row is left at its allocation value
    assert np.isfinite(y).all() and (np.abs(y).max(axis=1) > 0).all()


def test_buffer_pool_stats(backend):
    s0 = backend.fnn.buffer_pool.get_stats()
    x = np.ones((16, 16), np.float32)
    for _ in range(20):
        backend.fnn.linear(x, x)
    s1 = backend.fnn.get_buffer_pool_stats()
    assert s1["hits"] - s0["hits"] >= 60 and s1["allocations"] - s0["allocations"] < 10    # reference claims <10 allocs / 100 ops
    assert 0.0 <= s1["hit_rate"] <= 1.0 and s1["bytes_in_use"] == s0["bytes_in_use"]


RES_SHAPES = [(1, 8, 4), (3, 16, 5), (33, 40, 17), (130, 264, 250), (257, 72, 513), (300, 2056, 136),
              (1024, 384, 1536), (2048, 768, 768), (16384, 768, 768), (4096, 3072, 768)]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("M,K,N", RES_SHAPES)
def test_linear_residual_parity(backend, dtype, M, K, N):
    """residual + x.W^T + b in one kernel against linear followed by residual
    (backend/fnn.py:1394-1496, :1950-2014): every kernel variant (ragged, 128- and 256-wide tiles)."""
    rng = np.random.default_rng(M * 5 + K * 11 + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    r = (3.0 * rng.standard_normal((M, N))).astype(np.float32)
    x, W, r = prep(dtype, x, W, r)
    ref = O.truth_linear(x, W, b) + r.astype(np.float64)
    y = backend.fnn.fused_linear_residual(x, W, b, r, dtype=dtype)
    assert y.shape == (M, N) and y.dtype == np.float32
    assert O.max_rel(y, ref) < tol(dtype)
    y0 = backend.fnn.fused_linear_residual(x, W, None, r, dtype=dtype)
    assert O.max_rel(y0, O.truth_linear(x, W) + r.astype(np.float64)) < tol(dtype)


def test_linear_residual_shapes_and_errors(backend):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 5, 16)).astype(np.float32)
    W = rng.standard_normal((24, 16)).astype(np.float32)
    r = rng.standard_normal((2, 5, 24)).astype(np.float32)
    y = backend.fnn.fused_linear_residual(x, W, None, r)
    assert y.shape == (2, 5, 24)
    assert O.max_rel(y, O.truth_linear(x.reshape(10, 16), W).reshape(2, 5, 24) + r) < TOL_F32
    with pytest.raises(ValueError):
        backend.fnn.fused_linear_residual(x, W, None, r[:, :4])
    with pytest.raises(ValueError):
        backend.fnn.fused_linear_residual(x, W, np.zeros(23, np.float32), r)
    # the C entry point: empty K gives bias + residual; a missing residual is an argument error
    c = backend.core
    M, N = 7, 12
    b = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    db, dr = c.upload(b), c.upload(res)
    L.check(c.lib.grl_gemm_nt_res(c.ctx, L.GRL_F32, L.GRL_F32, M, N, 0, None, None, db.ptr, dr.ptr, dr.ptr))
    np.testing.assert_allclose(c.download(dr, (M, N)), res + b, rtol=1e-6, atol=1e-6)
    assert c.lib.grl_gemm_nt_res(c.ctx, L.GRL_F32, L.GRL_F32, M, N, 0, None, None, db.ptr, None, dr.ptr) != 0
    db.free(); dr.free()


def test_gemm_nt_c_abi_randomized(backend):
    """Seeded sweep of grl_gemm_nt / grl_gemm_nt_act through ctypes: all four (input, output) storage-type pairs, every
    epilogue code, bias or NULL, ragged shapes on both sides of the kernel-selection thresholds, and an output that sits
    inside a larger buffer at an aligned or an odd element offset (odd: the one-thread-per-output kernel) whose
    surroundings must keep a sentinel: a tile-edge store that leaves the matrix shows up there."""
    from conftest import sweep_rounds
    c = backend.core
    rng = np.random.default_rng(55005)
    epis = [(L.EPI_NONE, "none"), (L.EPI_GELU, "gelu"), (L.EPI_SILU, "silu"), (L.EPI_RELU, "relu"), (L.EPI_GCU, "gcu"), (L.EPI_ROSWISH, "roswish")]
    for case in range(32 * sweep_rounds()):
        cin, cout = [(L.GRL_F32, L.GRL_F32), (L.GRL_BF16, L.GRL_BF16), (L.GRL_BF16, L.GRL_F32), (L.GRL_F32, L.GRL_BF16)][case % 4]
        es_out = 2 if cout == L.GRL_BF16 else 4
        K = int(rng.choice([8, 24, 64, 72, 128, 200, 512]))
        if case % 8 == 7:                                      # >= 192 tiles of 256x256
            M, N = int(rng.integers(3300, 3700)), int(rng.integers(3600, 4000))
        else:
            M, N = int(rng.integers(1, 700)), int(rng.integers(1, 700))
        code, name = epis[int(rng.integers(0, len(epis)))]
        x = rng.standard_normal((M, K)).astype(np.float32)
        W = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
        b = rng.standard_normal(N).astype(np.float32) if rng.random() < 0.6 else None
        if cin == L.GRL_BF16:
            x, W = O.bf16_round(x), O.bf16_round(W)
        lead = int(rng.choice([0, 32, 1, 3]))                  # elements in front of the output inside its buffer
        tail = 64
        host_out = np.full(lead + M * N + tail, 7.0, np.float32)
        dx, dw, dout = c.upload(x, cin), c.upload(W, cin), c.upload(host_out, cout)
        db = c.upload(b) if b is not None else None
        try:
            cptr = dout.ptr + lead * es_out
            bptr = db.ptr if db else None
            if code <= L.EPI_SILU:
                rc = c.lib.grl_gemm_nt(c.ctx, cin, cout, M, N, K, dx.ptr, dw.ptr, bptr, cptr, code)
            else:
                rc = c.lib.grl_gemm_nt_act(c.ctx, cin, cout, M, N, K, dx.ptr, dw.ptr, bptr, cptr, code, 0.7, 1.3)
            L.check(rc, "gemm_nt")
            got = c.download(dout, (lead + M * N + tail,), cout)
        finally:
            for t in (dx, dw, dout, db):
                if t is not None:
                    t.free()
        ref = O.truth_linear(x, W, b, name, 0.7, 1.3)
        info = (case, cin, cout, M, N, K, name, b is not None, lead)
        y = got[lead:lead + M * N].reshape(M, N)
        t = TOL_F32 if (cin == L.GRL_F32 and cout == L.GRL_F32) else TOL_BF16
        assert np.isfinite(y).all(), info
        assert O.max_rel(y, ref) < t, info + (O.max_rel(y, ref),)
        assert (got[:lead] == 7.0).all() and (got[lead + M * N:] == 7.0).all(), info
        if case and case % 50 == 0:
            print("sweep case", case, flush=True)


# (M, K, N): few 64 x 64 tiles and at least sixteen K slabs: the launcher shares the slabs of a tile out over several
# workgroups and a second kernel adds the shares and runs the epilogue.  One sentence through the feed-forward block's
# second GEMM; a single row; ragged M and N (N a multiple of 4); a K tail in the last share; fp32 K = 512 is exactly 16 slabs
# (bf16: 8, not split).
SPLIT_K = [(32, 3072, 768), (128, 3072, 768), (1, 4096, 64), (100, 1024, 200), (70, 1000, 36), (50, 512, 40)]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("epi", ["none", "gelu", "silu", "relu", "roswish", "res"])
@pytest.mark.parametrize("M,K,N", SPLIT_K)
def test_split_k_products(backend, dtype, epi, M, K, N):
    rng = np.random.default_rng(M + 3 * K + 7 * N + len(epi))
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    if dtype == "bf16":
        x, W = O.bf16_round(x), O.bf16_round(W)
    tol = TOL_BF16 if dtype == "bf16" else TOL_F32
    f = backend.fnn
    for bias in (b, None):
        if epi == "res":
            r = (2.0 * rng.standard_normal((M, N))).astype(np.float32)
            r = O.bf16_round(r) if dtype == "bf16" else r
            y = f.fused_linear_residual(x, W, bias, r, dtype=dtype)
            ref = O.truth_linear(x, W, bias) + r.astype(np.float64)
        else:
            y = {"none": lambda: f.linear(x, W, bias, dtype=dtype),
                 "gelu": lambda: f.fused_linear_gelu(x, W, bias, dtype=dtype),
                 "silu": lambda: f.fused_linear_silu(x, W, bias, dtype=dtype),
                 "relu": lambda: f.fused_linear_relu(x, W, bias, dtype=dtype),
                 "roswish": lambda: f.fused_linear_roswish(x, W, bias, alpha=0.7, beta=1.3, dtype=dtype)}[epi]()
            ref = O.truth_linear(x, W, bias, epi, 0.7, 1.3)
        assert y.shape == (M, N) and np.isfinite(y).all()
        assert O.max_rel(y, ref) < tol, (epi, bias is None)
    # the same call twice gives the same bits (the shares are added in a fixed order)
    y1, y2 = f.linear(x, W, b, dtype=dtype), f.linear(x, W, b, dtype=dtype)
    np.testing.assert_array_equal(y1, y2)
