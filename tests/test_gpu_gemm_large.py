"""GPU parity of the GEMM family at shapes that select the kernels the benchmark times: the persistent
256x256-tile kernel (chosen from 192 such tiles on), with every epilogue, both storage types, ragged edges,
the register-staged variant for K rows that are not whole 128-byte slabs, and BASELINE configs[3]'s
N = 11008 / K = 4096 / K = 11008 shapes (narrow-band tile walk).  The oracle (float64 closed forms of the
reference shaders, shaders/fused-linear-gelu.glsl:42-93, fused-linear-silu.glsl:42-78,
fused-swiglu.glsl:43-79, fnn-linear.glsl:33-58) is evaluated on sampled output rows that cover every
256-row tile band (first row, last row and two random rows of each band).
Tolerances: max|y-ref|/max|ref| <= 1e-4 (fp32), <= 2e-2 (bf16)."""
import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16, rng_for, sweep_rounds
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu


def tol(dtype):
    return TOL_F32 if dtype == "fp32" else TOL_BF16


def prep(dtype, *arrs):
    return [O.bf16_round(a) if dtype == "bf16" else a for a in arrs]


def band_rows(M, rng, band=256, per=2):
    """first and last row of every `band`-row tile band plus `per` random rows inside it"""
    rows = []
    for r0 in range(0, M, band):
        r1 = min(M, r0 + band)
        rows += [r0, r1 - 1] + list(rng.integers(r0, r1, per))
    return np.unique(np.asarray(rows, dtype=np.int64))


def big_tiles(M, N, dual=False):
    return -(-M // 256) * -(-N // (128 if dual else 256))


def gen(rng, M, K, N, wstd):
    x = rng.standard_normal((M, K), dtype=np.float32)
    W = rng.standard_normal((N, K), dtype=np.float32) * np.float32(wstd)
    b = rng.standard_normal(N, dtype=np.float32)
    return x, W, b


# (M, K, N): all >= 192 tiles of 256x256.  N = 3080 leaves an 8-column edge tile, M = 16384+37 a 37-row edge band.
BIG = [(16384, 768, 3072), (16384 + 37, 768, 3072 + 8), (16384, 768, 768)]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("epi", ["none", "gelu", "silu", "relu", "roswish", "gcu"])
@pytest.mark.parametrize("M,K,N", BIG)
def test_big_tile_fused_linear(backend, dtype, epi, M, K, N):
    if (M, K, N) == BIG[2] and epi in ("roswish", "gcu"):
        pytest.skip("run-time epilogue is covered at the two wider shapes")
    assert big_tiles(M, N) >= 192
    rng = np.random.default_rng(M + 3 * N + len(epi))
    x, W, b = gen(rng, M, K, N, 1.0 / np.sqrt(K))
    x, W = prep(dtype, x, W)
    f = backend.fnn
    call = {"none": lambda bb: f.linear(x, W, bb, dtype=dtype),
            "gelu": lambda bb: f.fused_linear_gelu(x, W, bb, dtype=dtype),
            "silu": lambda bb: f.fused_linear_silu(x, W, bb, dtype=dtype),
            "relu": lambda bb: f.fused_linear_relu(x, W, bb, dtype=dtype),
            "gcu": lambda bb: f.fused_linear_gcu(x, W, bb, dtype=dtype),
            "roswish": lambda bb: f.fused_linear_roswish(x, W, bb, alpha=0.7, beta=1.3, dtype=dtype)}[epi]
    rows = band_rows(M, rng)
    y = call(b)
    assert y.shape == (M, N) and np.isfinite(y).all()
    ref = O.truth_linear(x[rows], W, b, epi, 0.7, 1.3)
    assert O.max_rel(y[rows], ref) < tol(dtype)
    # without bias (the bias slice is not fetched at all then)
    y0 = call(None)
    ref0 = O.truth_linear(x[rows], W, None, epi, 0.7, 1.3)
    assert O.max_rel(y0[rows], ref0) < tol(dtype)
    # every element was written by exactly the row it belongs to: a second run is bit-identical
    np.testing.assert_array_equal(call(b), y)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("act", ["silu", "gelu", "relu"])
@pytest.mark.parametrize("M,K,N,bias", [(16384, 512, 3072, True), (16384 + 37, 512, 1152 + 8, False)])
def test_big_tile_glu(backend, dtype, act, M, K, N, bias):
    assert big_tiles(M, N, dual=True) >= 192
    rng = np.random.default_rng(M + N + len(act))
    x = rng.standard_normal((M, K), dtype=np.float32)
    Wg = rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.06)
    Wu = rng.standard_normal((N, K), dtype=np.float32) * np.float32(0.06)
    bg = rng.standard_normal(N, dtype=np.float32) if bias else None
    bu = rng.standard_normal(N, dtype=np.float32) if bias else None
    x, Wg, Wu = prep(dtype, x, Wg, Wu)
    fn = {"silu": backend.fnn.fused_swiglu, "gelu": backend.fnn.fused_geglu, "relu": backend.fnn.fused_reglu}[act]
    rows = band_rows(M, rng)
    t_out, t_g, t_u = (O.truth_fused_swiglu(x[rows], Wg, Wu, bg, bu) if act == "silu"
                       else O.truth_fused_glu(x[rows], Wg, Wu, bg, bu, act))
    out = fn(x, Wg, Wu, bg, bu, dtype=dtype)                      # LDS-staged epilogue
    assert out.shape == (M, N) and np.isfinite(out).all()
    assert O.max_rel(out[rows], t_out) < tol(dtype)
    if act == "silu":
        out2, g, u = fn(x, Wg, Wu, bg, bu, return_cache=True, dtype=dtype)     # direct epilogue with the fp32 pre-activations
        assert O.max_rel(out2[rows], t_out) < tol(dtype)
        assert O.max_rel(g[rows], t_g) < tol(dtype) and O.max_rel(u[rows], t_u) < tol(dtype)
        # the staged epilogue starts its accumulators from the bias, the direct one adds the bias after the sum: the two
        # agree to the last bits of the float sums
        assert O.max_rel(out2, out) < (2e-6 if dtype == "fp32" else 8e-3)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_big_tile_register_staged_variant(backend, dtype):
    """K = 776: rows are 16-byte aligned but not whole 128-byte slabs, so the 256x256 register-staged kernel
    with its zero-filled K tail runs (plain and with the residual epilogue)."""
    M, K, N = 16384, 776, 3072
    rng = np.random.default_rng(776)
    x, W, b = gen(rng, M, K, N, 1.0 / np.sqrt(K))
    r = 3.0 * rng.standard_normal((M, N), dtype=np.float32)
    x, W, r = prep(dtype, x, W, r)
    rows = band_rows(M, rng)
    ref = O.truth_linear(x[rows], W, b)
    y = backend.fnn.linear(x, W, b, dtype=dtype)
    assert O.max_rel(y[rows], ref) < tol(dtype)
    yr = backend.fnn.fused_linear_residual(x, W, b, r, dtype=dtype)
    assert O.max_rel(yr[rows], ref + r[rows].astype(np.float64)) < tol(dtype)


def test_config4_swiglu_mlp_shapes(backend):
    """BASELINE configs[3] (reference backend/_glu_append.py:8-129 then backend/fnn.py:1394-1496):
    X . (W_g, W_u)[11008,4096]^T -> silu(X.W_g) * (X.W_u) -> . W_d[4096,11008]^T in bf16 with fp32 accumulation,
    at the full feature sizes (N = 11008, K = 4096, then K = 11008: the narrow-band tile walk) and M = 4096 of
    the 16384 rows (16 x 86 and 16 x 16 tiles still select the persistent kernel).  Row-sampled against the
    float64 oracle on the bf16-rounded inputs, plus exact homogeneity of the down projection under x2."""
    rng = rng_for(4)
    M, Kd, F = 4096, 4096, 11008
    X = O.bf16_round(rng.standard_normal((M, Kd), dtype=np.float32))
    Wg = O.bf16_round(rng.standard_normal((F, Kd), dtype=np.float32) * np.float32(0.02))
    Wu = O.bf16_round(rng.standard_normal((F, Kd), dtype=np.float32) * np.float32(0.02))
    Wd = O.bf16_round(rng.standard_normal((Kd, F), dtype=np.float32) * np.float32(0.02))
    assert big_tiles(M, F, dual=True) >= 192 and big_tiles(M, Kd) >= 192
    rows = band_rows(M, rng)
    # config 4 wants SiLU on the gate product: the reference's fused_swiglu puts it on its W_up argument
    Hh = backend.fnn.fused_swiglu(X, Wu, Wg, dtype="bf16")
    assert Hh.shape == (M, F) and np.isfinite(Hh).all()
    xs = X[rows].astype(np.float64)
    want_h = O.truth_silu(xs @ Wg.T.astype(np.float64)) * (xs @ Wu.T.astype(np.float64))
    assert O.max_rel(Hh[rows], want_h) < TOL_BF16
    Hq = O.bf16_round(Hh)                        # the device buffer held exactly these values
    np.testing.assert_array_equal(Hq, Hh)
    Y = backend.fnn.linear(Hq, Wd, dtype="bf16")
    assert Y.shape == (M, Kd) and np.isfinite(Y).all()
    assert O.max_rel(Y[rows], O.truth_linear(Hq[rows], Wd)) < TOL_BF16
    Y2 = backend.fnn.linear(2 * Hq[:1024], Wd, dtype="bf16")
    np.testing.assert_array_equal(Y2, 2 * Y[:1024])


def test_randomized_shapes_over_every_kernel_variant(backend):
    """Seeded sweep over what selects a GEMM kernel and what its edges see: K a multiple of the 128-byte slab (the
    direct-to-LDS kernels), of 16 bytes only (register-staged loads with a zero-filled K tail) or of neither (one thread
    per output); few tiles (128x128) or at least 192 tiles of 256x256 (the persistent kernel, with tile counts that do not
    divide by the 256 workgroups or the 8 XCD runs); ragged M and N; every epilogue, with and without bias; both
    dtypes.  Each case against the float64 closed form."""
    rng = np.random.default_rng(977)
    epis = ["none", "gelu", "silu", "relu", "res", "gcu", "roswish"]
    worst = {"fp32": 0.0, "bf16": 0.0}
    for case in range(42 * sweep_rounds()):
        if case and case % 50 == 0:
            print("sweep case", case, flush=True)      # long runs (pytest -s) show that they are alive
        dtype = "bf16" if case % 2 else "fp32"
        slab = 64 if dtype == "bf16" else 32
        chunk = 8 if dtype == "bf16" else 4
        kkind = case % 3                       # 0: whole slabs, 1: 16-byte rows with a K tail, 2: unaligned rows
        if kkind == 0:
            # every fifth of these with a long K: small products then share their K loop out over several workgroups
            K = slab * (int(rng.integers(16, 70)) if case % 5 == 0 else int(rng.integers(1, 9)))
        elif kkind == 1:
            K = chunk * int(rng.integers(1, 60))
            K += chunk if K % slab == 0 else 0
        else:
            K = int(rng.integers(1, 300)) | 1
        if case % 7 in (0, 3):                # the persistent big-tile kernels: >= 192 tiles
            M = int(rng.integers(3100, 4600)); N = int(rng.integers(3100, 4600))
            while ((M + 255) // 256) * ((N + 255) // 256) < 192:
                N += 256
            if kkind == 2:
                M //= 8                        # the one-thread-per-output kernel is slow: keep it small
        elif case % 7 in (1, 4) and kkind != 2:   # too many 64 x 64 tiles for one pass, too few 256 x 256 ones: the 128 x 128 kernels
            M = int(rng.integers(1100, 2600)); N = int(rng.integers(1100, 2600))
        else:
            M = int(rng.integers(1, 900)); N = int(rng.integers(1, 900))
        epi = epis[int(rng.integers(0, len(epis)))]
        x = rng.standard_normal((M, K)).astype(np.float32)
        W = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
        b = rng.standard_normal(N).astype(np.float32) if rng.random() < 0.7 else None
        x, W = prep(dtype, x, W)
        if epi == "res":
            r = prep(dtype, (2.0 * rng.standard_normal((M, N))).astype(np.float32))[0]
            y = backend.fnn.fused_linear_residual(x, W, b, r, dtype=dtype)
            ref = O.truth_linear(x, W, b) + r.astype(np.float64)
        elif epi == "none":
            y = backend.fnn.linear(x, W, b, dtype=dtype)
            ref = O.truth_linear(x, W, b)
        else:
            y = getattr(backend.fnn, "fused_linear_" + epi)(x, W, b, dtype=dtype)
            ref = O.truth_linear(x, W, b, epi)
        assert y.shape == (M, N) and np.isfinite(y).all(), (case, dtype, M, K, N, epi)
        err = O.max_rel(y, ref)
        worst[dtype] = max(worst[dtype], err)
        assert err < tol(dtype), (case, dtype, M, K, N, epi, b is not None, err)
    assert worst["fp32"] < TOL_F32 and worst["bf16"] < TOL_BF16


# (M, K, N) either side of the tile choice: few enough 64 x 64 tiles for one pass over the CUs (also with a K tail and with
# ragged edges), 320 and 192 big tiles whose last pass would stay mostly empty (128 x 128 tiles instead), 256 and 512 big
# tiles that fill their passes (256 x 256 tiles)
TILE_CHOICE = [(32, 384, 128), (100, 72, 200), (500, 256, 460), (16384, 384, 1152), (4096, 768, 3072), (8192, 768, 2048), (8192, 512, 4096)]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("M,K,N", TILE_CHOICE)
def test_linear_across_the_tile_choice(backend, dtype, M, K, N):
    """Every tile size the launcher picks by problem shape gives the same product: fused GELU, the gated dual GEMM and
    the LayerNorm-folded GEMM against float64 on band-edge and random rows."""
    rng = np.random.default_rng(M + 5 * N + K)
    x, W, b = gen(rng, M, K, N, 1.0 / np.sqrt(K))
    x, W = prep(dtype, x, W)
    rows = band_rows(M, rng, band=64, per=1) if M <= 1024 else band_rows(M, rng)
    f = backend.fnn
    y = f.fused_linear_gelu(x, W, b, dtype=dtype)
    assert y.shape == (M, N) and np.isfinite(y).all()
    assert O.max_rel(y[rows], O.truth_linear(x[rows], W, b, "gelu")) < tol(dtype)
    Nh = N // 2
    g = f.fused_swiglu(x, W[:Nh], W[Nh:2 * Nh], b[:Nh], b[Nh:2 * Nh], dtype=dtype)
    up = O.truth_linear(x[rows], W[Nh:2 * Nh], b[Nh:2 * Nh])
    gate = O.truth_linear(x[rows], W[:Nh], b[:Nh])
    assert O.max_rel(g[rows], gate * (up / (1 + np.exp(-up)))) < tol(dtype)
    gamma = (1 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(K)).astype(np.float32)
    z = f.fused_layernorm_linear(x, gamma, beta, W, b, dtype=dtype)
    ref = O.truth_linear(O.truth_layernorm(x[rows], gamma, beta), W, b)
    assert O.max_rel(z[rows], ref) < tol(dtype) * (1.5 if dtype == "bf16" else 1.0)
