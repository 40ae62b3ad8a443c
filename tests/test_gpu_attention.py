"""GPU parity of flash_attention2 / flash_attention2_rope / apply_rope against the oracle.
The reference's FA2 shader has no defined output (racy, and its host wrapper raises before
the first dispatch), so parity is against the documented contract -- softmax(scale.QK^T +
mask bias).V in layout (B,S,H,D) -- which tests/test_oracle.py pins by closed-form answers."""
import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16, rng_for
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu


def tol(dtype):
    return TOL_F32 if dtype == "fp32" else TOL_BF16


def qkv(rng, B, S, H, D, dtype):
    t = [rng.standard_normal((B, S, H, D)).astype(np.float32) for _ in range(3)]
    return [O.bf16_round(a) for a in t] if dtype == "bf16" else t


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("B,S,H,D", [(2, 64, 3, 64), (1, 1, 1, 32), (2, 37, 2, 32), (1, 129, 2, 128), (2, 200, 4, 64),
                                     (1, 300, 1, 128), (3, 256, 12, 32)])
def test_fa2_parity(backend, dtype, B, S, H, D):
    rng = np.random.default_rng(S * 13 + D)
    q, k, v = qkv(rng, B, S, H, D, dtype)
    o = backend.attention.flash_attention2(q, k, v, H, D, dtype=dtype)
    assert o.shape == (B, S, H, D) and o.dtype == np.float32
    assert O.max_rel(o, O.truth_attention(q, k, v)) < tol(dtype)


def test_config1_attention(backend, corc):
    # BASELINE config 1: Q/K/V (32,8,64,64) given as (batch, heads, seq, dim), no mask, scale 1/8
    rng = rng_for(1)
    q, k, v = [rng.standard_normal((32, 8, 64, 64)).astype(np.float32) for _ in range(3)]
    o = backend.attention.flash_attention2(q, k, v, 8, 64, scale=0.125, layout="bhsd")
    qs, ks, vs = [np.ascontiguousarray(t.transpose(0, 2, 1, 3)) for t in (q, k, v)]
    assert o.shape == (32, 64, 8, 64)
    assert O.max_rel(o, O.truth_attention(qs, ks, vs, scale=0.125)) < TOL_F32
    assert O.max_rel(o, corc.attention(qs, ks, vs, scale=0.125)) < TOL_F32
    np.testing.assert_array_equal(o, backend.attention.flash_attention2(qs, ks, vs, 8, 64, scale=0.125))


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_fa2_key_padding_mask(backend, dtype):
    # BASELINE config 2 shape (reduced batch): 12 heads x 32, S=256, lengths in [32,256]
    rng = rng_for(2)
    B, S, H, D = 8, 256, 12, 32
    q, k, v = qkv(rng, B, S, H, D, dtype)
    lens = rng.integers(32, 257, B)
    m = (np.arange(S)[None] < lens[:, None]).astype(np.float32)
    o = backend.attention.flash_attention2(q, k, v, H, D, mask=m, dtype=dtype)
    ref = O.truth_attention(q, k, v, mask=m)
    assert O.max_rel(o, ref) < tol(dtype)
    # masked keys carry no weight: changing their K/V changes nothing
    k2, v2 = k.copy(), v.copy()
    for b in range(B):
        k2[b, lens[b]:] = 7.0; v2[b, lens[b]:] = -3.0
    np.testing.assert_array_equal(backend.attention.flash_attention2(q, k2, v2, H, D, mask=m, dtype=dtype), o)


def test_fa2_known_answers(backend):
    rng = np.random.default_rng(6)
    q, k, v = qkv(rng, 1, 70, 2, 64, "fp32")
    mean = np.broadcast_to(v.astype(np.float64).mean(1, keepdims=True), v.shape)
    assert O.max_rel(backend.attention.flash_attention2(np.zeros_like(q), k, v, 2, 64), mean) < 1e-5     # equal scores -> mean of V
    k2 = np.repeat(k[:, :1], 70, 1)                                                                   # all keys equal -> mean of V
    assert O.max_rel(backend.attention.flash_attention2(q, k2, v, 2, 64), mean) < 1e-5
    m = np.zeros((1, 70), np.float32); m[0, 41] = 1                                                   # one key kept -> that V
    assert O.max_rel(backend.attention.flash_attention2(q, k, v, 2, 64, mask=m), np.broadcast_to(v[:, 41:42], v.shape)) < 1e-6
    z = np.zeros((1, 70), np.float32)                                                                 # fully masked row -> uniform mean
    assert O.max_rel(backend.attention.flash_attention2(q, k, v, 2, 64, mask=z), mean) < 1e-5
    oc = backend.attention.flash_attention2(q, k, v, 2, 64, causal=True)                              # causal row 0 -> V[0]
    np.testing.assert_allclose(oc[:, 0], v[:, 0], atol=1e-6)
    # heads are independent and live in axis 2
    np.testing.assert_array_equal(backend.attention.flash_attention2(q[:, :, ::-1], k[:, :, ::-1], v[:, :, ::-1], 2, 64),
                                  backend.attention.flash_attention2(q, k, v, 2, 64)[:, :, ::-1])


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("B,S,H,D", [(2, 130, 2, 64), (1, 257, 2, 128), (1, 96, 3, 32)])
def test_fa2_causal(backend, dtype, B, S, H, D):
    rng = np.random.default_rng(S + D)
    q, k, v = qkv(rng, B, S, H, D, dtype)
    o = backend.attention.flash_attention2(q, k, v, H, D, causal=True, dtype=dtype)
    assert O.max_rel(o, O.truth_attention(q, k, v, causal=True)) < tol(dtype)
    # the future does not leak: perturbing the last third of K/V leaves earlier rows unchanged
    cut = 2 * S // 3
    k2, v2 = k.copy(), v.copy(); k2[:, cut:] += 1.0; v2[:, cut:] -= 2.0
    o2 = backend.attention.flash_attention2(q, k2, v2, H, D, causal=True, dtype=dtype)
    np.testing.assert_array_equal(o2[:, :cut], o[:, :cut])


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("style", ["interleaved", "half"])
@pytest.mark.parametrize("B,S,H,D,causal", [(1, 150, 2, 128, True), (2, 64, 2, 64, False), (1, 200, 2, 32, True)])
def test_fa2_rope(backend, dtype, style, B, S, H, D, causal):
    rng = np.random.default_rng(S + D + len(style))
    q, k, v = qkv(rng, B, S, H, D, dtype)
    o = backend.attention.flash_attention2_rope(q, k, v, H, D, causal=causal, rope_style=style, dtype=dtype)
    assert O.max_rel(o, O.truth_attention(q, k, v, causal=causal, rope=style)) < tol(dtype)
    if dtype == "fp32":
        # fused == apply_rope + plain attention
        qr = backend.attention.apply_rope(q, rope_style=style); kr = backend.attention.apply_rope(k, rope_style=style)
        o2 = backend.attention.flash_attention2(qr, kr, v, H, D, causal=causal)
        assert O.max_rel(o, o2) < 1e-5


def test_rope_scaling_and_base(backend):
    rng = np.random.default_rng(3)
    q, k, v = qkv(rng, 1, 64, 1, 64, "fp32")
    o = backend.attention.flash_attention2_rope(q, k, v, 1, 64, rope_base=500.0, rope_scaling=4.0)
    assert O.max_rel(o, O.truth_attention(q, k, v, rope="interleaved", base=500.0, scaling=4.0)) < TOL_F32
    x = rng.standard_normal((2, 33, 3, 32)).astype(np.float32)
    pid = rng.integers(0, 500, (2, 33)).astype(np.int32)
    y = backend.attention.apply_rope(x, pid, 10000.0, 2.0)
    assert O.max_rel(y, O.truth_rope(x, 10000.0, 2.0, "half", pid)) < 1e-5
    np.testing.assert_allclose(backend.attention.apply_rope(x)[:, 0], x[:, 0], atol=1e-7)       # position 0 unrotated


def test_fa2_shapes_and_errors(backend):
    rng = np.random.default_rng(12)
    q, k, v = qkv(rng, 2, 40, 2, 32, "fp32")
    flat = [t.reshape(2, 40, 64) for t in (q, k, v)]
    o = backend.attention.flash_attention2(*flat, 2, 32)                       # (B,S,H*D) input
    assert o.shape == (2, 40, 2, 32)
    np.testing.assert_array_equal(o, backend.attention.flash_attention2(q, k, v, 99, 99))    # rank-4 overrides the arguments
    np.testing.assert_array_equal(o, backend.attention.flash_attention2(q, k, v, 2, 32, tile_size_q=16, tile_size_k=32))
    with pytest.raises(ValueError):
        backend.attention.flash_attention2(q, k, v, 2, 32, mask=np.ones((2, 39)))
    with pytest.raises(ValueError):
        backend.attention.flash_attention2(np.zeros((1, 4, 1, 1100), np.float32), np.zeros((1, 4, 1, 1100), np.float32),
                                           np.zeros((1, 4, 1, 1100), np.float32), 1, 1100)      # head_dim above 1024
    with pytest.raises(ValueError):
        backend.attention.flash_attention2(q, k[:, :10], v, 2, 32)
    # deterministic across runs (the reference shader is not)
    np.testing.assert_array_equal(backend.attention.flash_attention2(q, k, v, 2, 32), backend.attention.flash_attention2(q, k, v, 2, 32))


def test_full_size_long_causal_rope_properties(backend):
    # BASELINE config 5 at full sequence length (one batch entry, 4 heads to bound the download):
    # S=8192, D=128, bf16, causal, interleaved RoPE.  Size-independent properties + sampled oracle rows.
    rng = rng_for(5)
    B, S, H, D = 1, 8192, 4, 128
    q, k, v = qkv(rng, B, S, H, D, "bf16")
    o = backend.attention.flash_attention2_rope(q, k, v, H, D, causal=True, dtype="bf16")
    assert np.isfinite(o).all()
    np.testing.assert_allclose(o[:, 0], v[:, 0], atol=1e-2)                  # row 0 sees key 0 only
    # outputs are convex combinations of V rows
    assert (o.max(axis=1) <= v.max(axis=1) + 1e-2).all() and (o.min(axis=1) >= v.min(axis=1) - 1e-2).all()
    # sampled query rows against the oracle (row i needs keys 0..i only)
    qr = O.truth_rope(q, style="interleaved"); kr = O.truth_rope(k, style="interleaved")
    for i in (1, 63, 64, 127, 128, 1000, 4095, 4096, 8191):
        s = np.einsum("hd,jhd->hj", qr[0, i], kr[0, :i + 1]) / np.sqrt(D)
        p = np.exp(s - s.max(-1, keepdims=True)); p /= p.sum(-1, keepdims=True)
        ref = np.einsum("hj,jhd->hd", p, v[0, :i + 1].astype(np.float64))
        assert O.max_rel(o[0, i], ref) < TOL_BF16, i


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("style", ["half", "interleaved"])
@pytest.mark.parametrize("B,S,H,D", [(2, 37, 3, 32), (1, 130, 2, 64), (2, 19, 4, 128), (1, 9, 2, 24), (2, 11, 3, 6)])
def test_apply_rope_parity_table_and_pairwise_paths(backend, dtype, style, B, S, H, D):
    """apply_rope (backend/attention.py:599-676, shaders/rope.glsl:74-125) with default positions takes the
    table-driven 16-byte path when the (half) row is 16-byte granular and the per-pair path otherwise
    (D = 24, 6), and the per-pair path whenever position ids are given; all must agree with the oracle,
    including base / scaling other than the defaults."""
    rng = np.random.default_rng(B * 1000 + S * 10 + D)
    x = rng.standard_normal((B, S, H, D)).astype(np.float32)
    if dtype == "bf16":
        x = O.bf16_round(x)
    t = TOL_F32 if dtype == "fp32" else TOL_BF16
    ref = O.truth_rope(x, 500.0, 1.5, style)
    y = backend.attention.apply_rope(x, None, 500.0, 1.5, rope_style=style, dtype=dtype)
    assert y.shape == x.shape and O.max_rel(y, ref) < t
    pid = np.tile(np.arange(S, dtype=np.int32), (B, 1))
    y2 = backend.attention.apply_rope(x, pid, 500.0, 1.5, rope_style=style, dtype=dtype)
    assert O.max_rel(y2, ref) < t
    assert O.max_rel(y2, y) < (1e-6 if dtype == "fp32" else 1e-2)      # same angles, same arithmetic


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("D", [8, 24, 40, 80, 96, 6, 1, 33, 130, 160, 320])
@pytest.mark.parametrize("mode", ["dense", "causal_mask"])
def test_fa2_any_head_dim(backend, dtype, D, mode):
    """The reference reshapes with whatever head_dim it is given (backend/attention.py:403-410): head dims other
    than 32 / 64 / 128 run on zero-padded copies (up to 128) or the one-wave-per-query kernel (above)."""
    B, S, H = 2, 75, 3
    rng = np.random.default_rng(D * 7 + len(mode))
    q, k, v = qkv(rng, B, S, H, D, dtype)
    causal = mode != "dense"
    mask = None
    if causal:
        mask = np.ones((B, S), np.float32); mask[0, 50:] = 0; mask[1, :3] = 0
    o = backend.attention.flash_attention2(q, k, v, H, D, mask=mask, causal=causal, dtype=dtype)
    assert o.shape == (B, S, H, D)
    assert O.max_rel(o, O.truth_attention(q, k, v, mask=mask, causal=causal)) < tol(dtype)
    # (B,S,H*D) input with the head split given by the arguments
    flat = [t.reshape(B, S, H * D) for t in (q, k, v)]
    np.testing.assert_array_equal(backend.attention.flash_attention2(*flat, H, D, mask=mask, causal=causal, dtype=dtype), o)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("style", ["interleaved", "half"])
@pytest.mark.parametrize("D", [8, 24, 96])
def test_fa2_rope_any_head_dim(backend, dtype, style, D):
    rng = np.random.default_rng(D + len(style))
    q, k, v = qkv(rng, 1, 60, 2, D, dtype)
    o = backend.attention.flash_attention2_rope(q, k, v, 2, D, causal=True, rope_style=style, dtype=dtype)
    assert O.max_rel(o, O.truth_attention(q, k, v, causal=True, rope=style)) < tol(dtype)
    with pytest.raises(ValueError):
        backend.attention.flash_attention2_rope(q[..., :7], k[..., :7], v[..., :7], 2, 7, rope_style=style, dtype=dtype)


def test_rope_table_is_reused_across_calls(backend):
    """the cos/sin table of the fused rotation is built once per (head dim, base, scaling) and serves shorter sequences"""
    rng = np.random.default_rng(77)
    for S in (96, 40, 96, 130):
        q, k, v = qkv(rng, 1, S, 2, 64, "bf16")
        o = backend.attention.flash_attention2_rope(q, k, v, 2, 64, causal=True, dtype="bf16")
        assert O.max_rel(o, O.truth_attention(q, k, v, causal=True, rope="interleaved")) < TOL_BF16
    o2 = backend.attention.flash_attention2_rope(q, k, v, 2, 64, causal=True, rope_base=500.0, dtype="bf16")
    assert O.max_rel(o2, O.truth_attention(q, k, v, causal=True, rope="interleaved", base=500.0)) < TOL_BF16


def test_fa2_strided_randomized(backend):
    """Seeded sweep of grl_fa2_fwd_strided through the C ABI: Q, K and V as column blocks of one packed buffer or in
    buffers of their own, position strides from exactly H*D upwards, block offsets and strides that are 16-byte granular
    (the kernels read the operands in place) or not (dense copies from the pool), the output written into a strided buffer
    whose other columns must stay untouched; both dtypes, key mask, causal, both RoPE pairings."""
    from conftest import sweep_rounds
    from grilly_amd import _lib as L
    c = backend.core
    rng = np.random.default_rng(55004)
    for case in range(24 * sweep_rounds()):
        dtype = "bf16" if case % 2 else "fp32"
        code, es = (L.GRL_BF16, 2) if dtype == "bf16" else (L.GRL_F32, 4)
        D = int(rng.choice([32, 64, 128, 40]))
        H = int(rng.integers(1, 4))
        S = int(rng.choice([1, 19, 64, 130, 300]))
        B = int(rng.integers(1, 3))
        hd = H * D
        gran = 16 // es                                    # elements per 16 bytes
        granular = case % 4 != 3
        pad = lambda: int(rng.integers(0, 4)) * gran + (0 if granular else int(rng.integers(1, gran)))
        packed = bool(rng.integers(0, 2))
        q, k, v = qkv(rng, B, S, H, D, dtype)
        flat = lambda a: a.reshape(B, S, hd)
        bufs = []
        if packed:
            offs = [pad(), 0, 0]
            offs[1] = offs[0] + hd + pad(); offs[2] = offs[1] + hd + pad()
            stride = offs[2] + hd + pad()
            host = rng.standard_normal((B, S, stride)).astype(np.float32)
            for a, o in zip((q, k, v), offs):
                host[:, :, o:o + hd] = flat(a)
            dev = c.upload(host, code); bufs.append(dev)
            ptrs = [dev.ptr + o * es for o in offs]; strides = [stride] * 3
        else:
            ptrs, strides = [], []
            for a in (q, k, v):
                o = pad(); stride = o + hd + pad()
                host = rng.standard_normal((B, S, stride)).astype(np.float32)
                host[:, :, o:o + hd] = flat(a)
                dev = c.upload(host, code); bufs.append(dev)
                ptrs.append(dev.ptr + o * es); strides.append(stride)
        oo = pad(); ostride = oo + hd + pad()
        sentinel = np.full((B, S, ostride), 7.0, np.float32)
        dout = c.upload(sentinel, code); bufs.append(dout)
        mask = None
        if case % 3 == 1:
            mask = (rng.random((B, S)) > 0.2).astype(np.float32); mask[:, 0] = 1
        dmask = c.upload(mask) if mask is not None else None
        causal = bool(rng.integers(0, 2))
        style = [None, "interleaved", "half"][int(rng.integers(0, 3))]
        rope = {None: L.ROPE_NONE, "interleaved": L.ROPE_INTERLEAVED, "half": L.ROPE_HALF}[style]
        base, scaling = float(rng.choice([10000.0, 500.0])), float(rng.choice([1.0, 2.0]))
        scale = 1.0 / np.sqrt(D)
        try:
            L.check(c.lib.grl_fa2_fwd_strided(c.ctx, code, B, S, H, D, ptrs[0], ptrs[1], ptrs[2], dmask.ptr if dmask else None,
                                              dout.ptr + oo * es, strides[0], strides[1], strides[2], ostride, scale, int(causal),
                                              rope, base, scaling), "fa2_fwd_strided")
            got = c.download(dout, (B, S, ostride), code)
        finally:
            for b in bufs + ([dmask] if dmask else []):
                b.free()
        ref = O.truth_attention(q, k, v, mask=mask, causal=causal, rope=style, base=base, scaling=scaling)
        info = (case, dtype, B, S, H, D, packed, granular, strides, ostride, style, causal, mask is not None)
        o = got[:, :, oo:oo + hd].reshape(B, S, H, D)
        assert np.isfinite(o).all(), info
        assert O.max_rel(o, ref) < tol(dtype), info + (O.max_rel(o, ref),)
        rest = np.delete(got, np.s_[oo:oo + hd], axis=2)
        assert (rest == 7.0).all(), info
        if case and case % 50 == 0:
            print("sweep case", case, flush=True)
