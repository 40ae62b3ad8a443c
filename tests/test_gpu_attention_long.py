"""GPU parity of flash_attention2 at the launch configurations the short tests do not reach: sequences
longer than 1024 (eight-wave workgroups, 128-key tiles, both workgroup orders) for every head dim, dense /
causal / key-padding mask / ragged length; head dim 128 with at most 128 keys (deep ring of 64-key tiles);
and score distributions that force the running-maximum rescale inside tiles whose scores are formed
relative to the running reference.  Contract: reference backend/attention.py:374-395
(softmax(scale.QK^T + (mask-1).1e9).V, layout (B,S,H,D)); oracle = float64 closed form.
Tolerances: max|y-ref|/max|ref| <= 1e-4 (fp32), <= 2e-2 (bf16)."""
import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16, sweep_rounds
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu


def tol(dtype):
    return TOL_F32 if dtype == "fp32" else TOL_BF16


def qkv(rng, B, S, H, D, dtype):
    t = [rng.standard_normal((B, S, H, D)).astype(np.float32) for _ in range(3)]
    return [O.bf16_round(a) for a in t] if dtype == "bf16" else t


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("mode", ["dense", "causal", "mask"])
@pytest.mark.parametrize("S,D", [(1100, 32), (1100, 64), (2048 + 17, 32), (2048 + 17, 64), (1500, 128), (2048, 128)])
def test_fa2_long_sequences(backend, dtype, mode, S, D):
    B, H = 2, 2
    rng = np.random.default_rng(S * 7 + D + len(mode))
    q, k, v = qkv(rng, B, S, H, D, dtype)
    mask = None
    if mode == "mask":
        lens = np.array([S - 3, S // 2 + 5])
        mask = (np.arange(S)[None] < lens[:, None]).astype(np.float32)
    o = backend.attention.flash_attention2(q, k, v, H, D, mask=mask, causal=(mode == "causal"), dtype=dtype)
    assert o.shape == (B, S, H, D) and np.isfinite(o).all()
    ref = O.truth_attention(q, k, v, mask=mask, causal=(mode == "causal"))
    assert O.max_rel(o, ref) < tol(dtype)
    if mode == "causal":
        np.testing.assert_allclose(o[:, 0], v[:, 0], atol=1e-6 if dtype == "fp32" else 1e-2)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("S", [64, 128, 100])
@pytest.mark.parametrize("causal", [False, True])
def test_fa2_head_dim_128_short(backend, dtype, S, causal):
    B, H, D = 3, 2, 128
    rng = np.random.default_rng(S + 128 + int(causal))
    q, k, v = qkv(rng, B, S, H, D, dtype)
    o = backend.attention.flash_attention2(q, k, v, H, D, causal=causal, dtype=dtype)
    assert O.max_rel(o, O.truth_attention(q, k, v, causal=causal)) < tol(dtype)


def _growing_keys(rng, S, D, profile):
    """keys whose projection on the queries' common direction follows `profile` (natural-log score units):
    q = |N(0,1)| rows, k_j = g_j * ones / D * sqrt(D) so that <q_i, k_j>/sqrt(D) ~ g_j * mean(q_i)."""
    q = np.abs(rng.standard_normal((1, S, 1, D))).astype(np.float32)
    k = (profile[None, :, None, None] * np.ones((1, S, 1, D)) / np.sqrt(D)).astype(np.float32)
    k += 0.05 * rng.standard_normal(k.shape).astype(np.float32)
    v = rng.standard_normal((1, S, 1, D)).astype(np.float32)
    return q, k, v


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("S", [512, 2048])
@pytest.mark.parametrize("shape", ["ramp", "step", "jumps", "sawtooth"])
def test_fa2_running_maximum_rescale(backend, dtype, D, S, shape):
    """Scores that climb along the key axis: `ramp` raises the row maximum by far more than 2^6 in every
    tile, `step` once in the middle of a tile, `jumps` at random keys, `sawtooth` climbs and falls back so
    that earlier tiles keep a visible share of the output.  mean(|N(0,1)|) ~ 0.8, so a profile value g gives
    scores ~0.8 g sqrt(D)/sqrt(D)... in natural units about 0.8*g."""
    rng = np.random.default_rng(S + D + len(shape))
    j = np.arange(S, dtype=np.float64)
    if shape == "ramp":
        prof = 0.12 * j                                   # ~ +6 natural units (8.9 binades) per 64 keys
    elif shape == "step":
        prof = np.where(j < S // 2 + 21, 0.0, 40.0)
    elif shape == "jumps":
        prof = np.cumsum(np.where(rng.random(S) < 0.01, 12.0, 0.0))
    else:
        prof = 10.0 * ((j % 192) / 192.0)
    q, k, v = _growing_keys(rng, S, D, prof)
    if dtype == "bf16":
        q, k, v = (O.bf16_round(t) for t in (q, k, v))
    for causal in (False, True):
        o = backend.attention.flash_attention2(q, k, v, 1, D, causal=causal, dtype=dtype)
        ref = O.truth_attention(q, k, v, causal=causal)
        assert np.isfinite(o).all()
        assert O.max_rel(o, ref) < tol(dtype), (shape, causal)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("S,D", [(200, 64), (512, 64), (512, 32), (300, 128), (1300, 64), (1300, 128)])
def test_fa2_mask_layouts(backend, dtype, S, D):
    """Key masks other than right padding: whole leading tiles masked out (left padding of 70 and of 130 keys: the
    softmax reference of those rows starts at the -1e9 of masked scores and has to come up to the first real
    key's), holes inside the sequence, and a single visible key (the output is that key's value row)."""
    B, H = 4, 2
    rng = np.random.default_rng(S * 3 + D)
    q, k, v = qkv(rng, B, S, H, D, dtype)
    mask = np.ones((B, S), np.float32)
    mask[0, :70] = 0
    mask[1, :130] = 0; mask[1, S - 9:] = 0
    mask[2, 40:110] = 0; mask[2, 150:170] = 0
    mask[3, :] = 0; mask[3, 137] = 1
    o = backend.attention.flash_attention2(q, k, v, H, D, mask=mask, dtype=dtype)
    assert np.isfinite(o).all()
    ref = O.truth_attention(q, k, v, mask=mask)
    assert O.max_rel(o, ref) < tol(dtype)
    np.testing.assert_allclose(o[3], np.broadcast_to(v[3, 137], o[3].shape), atol=1e-6 if dtype == "fp32" else 1e-2)


@pytest.mark.parametrize("D", [32, 64, 128])
def test_fa2_left_padding_under_large_scores(backend, D):
    """Several tiles of left padding whose (masked) scores run into the hundreds: a row that has seen padding only
    holds a reference near -1.4e9, against which scores have a granularity of 128, and the reference-raising path must
    keep every weight finite there (an infinity would survive the rescale by zero that the first real key brings).
    All rows have real keys, so the float64 oracle applies to every one."""
    rng = np.random.default_rng(31 + D)
    B, S, H = 2, 1024, 2
    q = np.abs(rng.standard_normal((B, S, H, D))).astype(np.float32) * 0.5 + 1.0
    ramp = np.cumsum(np.where(rng.random(S) < 0.03, rng.uniform(20.0, 90.0, S), 0.0))
    k = (0.05 * rng.standard_normal((B, S, H, D)) + ramp[None, :, None, None] / np.sqrt(D) / 1.4).astype(np.float32)
    v = rng.standard_normal((B, S, H, D)).astype(np.float32)
    q, k, v = (O.bf16_round(t) for t in (q, k, v))
    mask = np.ones((B, S), np.float32)
    mask[0, :415] = 0
    mask[1, :200] = 0; mask[1, 900:] = 0
    o = backend.attention.flash_attention2(q, k, v, H, D, mask=mask, dtype="bf16")
    assert np.isfinite(o).all()
    assert O.max_rel(o, O.truth_attention(q, k, v, mask=mask)) < TOL_BF16


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("S,D", [(512, 64), (512, 32), (700, 128), (1536, 64), (1536, 128), (330, 48), (330, 80)])
def test_fa2_padded_batches(backend, S, D, causal, dtype):
    """Right-padded batches: most tiles carry no mask bias at all and whole tiles of padding follow the real keys
    (the bf16 kernel runs the former like unmasked tiles and passes over the latter once every row of a wave has a
    real key behind it).  Lengths on and around tile edges; padding written as 0, as 0.5 (still an exact zero weight)
    and as 0.75 (a bias the kernel adds rather than skips); a row whose only real keys come after a masked first
    tile, under the causal rule, keeps rows that have seen masked keys only; one key weighted up by a mask above 1; a
    sequence with every key masked (the mean over all keys, or over the causal ones: keys masked alike weigh alike in
    every tile, which a mask bias rounded differently from tile to tile would break)."""
    lens = [S, 1, 63, 64, 65, 200, S - 1, S // 2, 0]
    B, H = len(lens) + 2, 2
    rng = np.random.default_rng(S + 7 * D + causal)
    q, k, v = qkv(rng, B, S, H, D, dtype)
    mask = np.ones((B, S), np.float32)
    for i, n in enumerate(lens):
        mask[i, n:] = (0.0, 0.5, 0.75)[i % 3]
    mask[B - 2, :96] = 0; mask[B - 2, 300:] = 0
    mask[B - 1, 400:] = 0; mask[B - 1, 77] = np.float32(1.0) + np.float32(2.0 ** -23)
    o = backend.attention.flash_attention2(q, k, v, H, D, mask=mask, causal=causal, dtype=dtype)
    assert np.isfinite(o).all()
    ref = O.truth_attention(q, k, v, mask=mask, causal=causal)
    for i in range(B):
        assert O.max_rel(o[i], ref[i]) < tol(dtype), (i, S, D, causal)
    if not causal:
        atol = 1e-2 if dtype == "bf16" else 1e-5
        np.testing.assert_allclose(o[1], np.broadcast_to(v[1, 0], o[1].shape), atol=atol)
        np.testing.assert_allclose(o[8], np.broadcast_to(v[8].mean(0), o[8].shape), atol=atol)


def test_fa2_randomized_configurations(backend):
    """Seeded sweep over what steers the bf16 kernel's paths: sequence length (whole and ragged tiles, below and above
    the 1024-key switch to eight-wave workgroups), head dim, causal, key masks with random holes and padding on either
    side, and score profiles that raise the row maximum at random keys (the rare path of the tile loop, possibly several
    times per row and next to masked or diagonal tiles).  Every case against the float64 closed form."""
    rng = np.random.default_rng(20240611)
    worst = 0.0
    for case in range(36 * sweep_rounds()):
        if case and case % 50 == 0:
            print("sweep case", case, flush=True)      # long runs (pytest -s) show that they are alive
        D = int(rng.choice([32, 64, 128]))
        S = int(rng.choice([65, 128, 191, 256, 448, 512, 777, 1024, 1100, 1536]))
        B, H = 2, int(rng.choice([1, 3]))
        causal = bool(rng.integers(0, 2))
        q = rng.standard_normal((B, S, H, D)).astype(np.float32)
        k = rng.standard_normal((B, S, H, D)).astype(np.float32)
        v = rng.standard_normal((B, S, H, D)).astype(np.float32)
        kind = case % 3
        if kind == 1:          # a few keys line up with every query: jumps of the running maximum at random places
            qdir = np.abs(rng.standard_normal((1, 1, H, D))).astype(np.float32)
            q = np.abs(q) * 0.5 + qdir
            jumps = np.cumsum(np.where(rng.random(S) < 0.02, rng.uniform(4.0, 30.0, S), 0.0))
            k = 0.05 * k + (jumps[None, :, None, None] / np.sqrt(D) / max(float(qdir.mean()), 0.5)).astype(np.float32)
        mask = None
        if kind == 2 or case % 4 == 0:
            mask = (rng.random((B, S)) > 0.15).astype(np.float32)
            left, right = int(rng.integers(0, S // 2)), int(rng.integers(0, S // 3))
            mask[0, :left] = 0
            if right:
                mask[1, S - right:] = 0
            mask[:, S // 2] = 1            # at least one visible key per row (not causal-safe for early rows: see below)
            if causal:
                mask[:, 0] = 1             # every causal row sees key 0
        q, k, v = (O.bf16_round(t) for t in (q, k, v))
        o = backend.attention.flash_attention2(q, k, v, H, D, mask=mask, causal=causal, dtype="bf16")
        assert np.isfinite(o).all(), (case, S, D, causal, kind)
        ref = O.truth_attention(q, k, v, mask=mask, causal=causal)
        err = O.max_rel(o, ref)
        worst = max(worst, err)
        assert err < TOL_BF16, (case, S, D, causal, kind, err)
    assert worst < TOL_BF16


def test_fa2_randomized_api_surface(backend):
    """Seeded sweep over the whole flash_attention2 / flash_attention2_rope surface: both dtypes; head dims the MFMA
    kernels take directly (32, 64, 128), head dims that run on zero-padded copies (8 ... 120) and head dims above 128
    (one wave per query); both RoPE pairings with bases and scalings other than the default; right and left padding
    and random holes in the key mask; causal; sequence lengths from one key to a few tiles.  Every case against the
    float64 closed form (bf16 cases on bf16-rounded inputs)."""
    rng = np.random.default_rng(424242)
    worst = {"fp32": 0.0, "bf16": 0.0}
    dims = [8, 24, 32, 40, 64, 80, 96, 120, 128, 160, 256]
    for case in range(48 * sweep_rounds()):
        if case and case % 50 == 0:
            print("sweep case", case, flush=True)      # long runs (pytest -s) show that they are alive
        dtype = "bf16" if case % 2 else "fp32"
        D = int(dims[int(rng.integers(0, len(dims)))])
        S = int(rng.choice([1, 2, 31, 64, 65, 130, 257, 400, 700]))
        if D > 128:
            S = min(S, 257)
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        causal = bool(rng.integers(0, 2))
        style = [None, "interleaved", "half"][case % 3] if D <= 128 else None      # the fused rotation stops at head dim 128
        base = float(rng.choice([10000.0, 500.0, 160000.0]))
        scaling = float(rng.choice([1.0, 0.5, 4.0]))
        q, k, v = qkv(rng, B, S, H, D, dtype)
        mask = None
        if case % 4 in (1, 2):
            mask = (rng.random((B, S)) > 0.2).astype(np.float32)
            if case % 4 == 2:
                n = int(rng.integers(0, S + 1))
                mask[0, n:] = 0                      # right padding (possibly the whole sequence)
                mask[B - 1, : S // 3] = 0            # left padding
            mask[:, 0] = 1                           # (every causal row keeps a key: masked-only rows weigh by rounding)
        if style is None:
            o = backend.attention.flash_attention2(q, k, v, H, D, mask=mask, causal=causal, dtype=dtype)
            ref = O.truth_attention(q, k, v, mask=mask, causal=causal)
        else:
            o = backend.attention.flash_attention2_rope(q, k, v, H, D, mask=mask, causal=causal, rope_base=base,
                                                        rope_scaling=scaling, rope_style=style, dtype=dtype)
            ref = O.truth_attention(q, k, v, mask=mask, causal=causal, rope=style, base=base, scaling=scaling)
        assert o.shape == (B, S, H, D) and np.isfinite(o).all(), (case, dtype, S, D, style, causal)
        err = O.max_rel(o, ref)
        worst[dtype] = max(worst[dtype], err)
        assert err < tol(dtype), (case, dtype, B, S, H, D, style, base, scaling, causal, mask is not None, err)
    assert worst["fp32"] < TOL_F32 and worst["bf16"] < TOL_BF16
