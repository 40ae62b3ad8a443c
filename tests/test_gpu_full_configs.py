"""The five benchmark configurations at their FULL sizes on the GPU (the other GPU tests run them at sizes the
float64 oracle covers whole): size-independent properties over the whole output plus oracle checks on sampled
sequences / rows, and the fp32 leg of the BERT-base-shaped encoder.
Recipes: utils/vulkan_sentence_transformer.py:972-1035 (post-LN layer), backend/_glu_append.py:8-129 then
backend/fnn.py:1394-1496 (SwiGLU MLP), shaders/flash-attention2-rope.glsl:73-148 (attention with RoPE).
Tolerances: max|y-ref|/max|ref| <= 1e-4 (fp32), <= 2e-2 (bf16)."""
import numpy as np
import pytest

from conftest import TOL_F32, TOL_BF16, rng_for
from oracle import oracle_np as O
from grilly_amd import BertEncoder, EncoderConfig, random_bert_weights

pytestmark = pytest.mark.gpu


def truth_encoder(w, cfg, ids, mask, quant=None):
    qf = (lambda a: a) if quant is None else (lambda a: quant(np.asarray(a, np.float32)).astype(np.float64))
    x = qf(O.truth_embed(ids, w["tok_emb"], w["pos_emb"], w["type_emb"]))
    x = qf(O.truth_layernorm(x, w["emb_ln_g"], w["emb_ln_b"], cfg.eps))
    for lw in w["layers"]:
        if quant is not None:
            lw = {k: (quant(v) if k.startswith("w_") else v) for k, v in lw.items()}
        x = O.truth_bert_layer(x, lw, mask, cfg.heads, cfg.eps, quant)
    return x


def band_rows(M, rng, band=256, per=2):
    rows = []
    for r0 in range(0, M, band):
        r1 = min(M, r0 + band)
        rows += [r0, r1 - 1] + list(rng.integers(r0, r1, per))
    return np.unique(np.asarray(rows, dtype=np.int64))


def test_readme_quickstart_ops_fp32(backend):
    """configs[0]: x[32,384] . W[384,128] + 0 -> swiglu, and attention on Q/K/V (32,8,64,64) given as
    (batch, heads, seq, dim), no mask, scale 1/8, fp32; whole outputs against the float64 oracle."""
    rng = rng_for(1)
    x = rng.standard_normal((32, 384)).astype(np.float32)
    W = rng.standard_normal((384, 128)).astype(np.float32)
    Wt = np.ascontiguousarray(W.T)
    y = backend.fnn.linear(x, Wt, np.zeros(128, np.float32))
    assert y.shape == (32, 128) and O.max_rel(y, x.astype(np.float64) @ W.astype(np.float64)) < TOL_F32
    g = backend.fnn.activation_swiglu(y)
    yd = y.astype(np.float64)
    assert g.shape == (32, 64) and O.max_rel(g, yd[:, :64] * (yd[:, 64:] / (1 + np.exp(-yd[:, 64:])))) < TOL_F32
    q, k, v = (rng.standard_normal((32, 8, 64, 64)).astype(np.float32) for _ in range(3))
    qs, ks, vs = (np.ascontiguousarray(t.transpose(0, 2, 1, 3)) for t in (q, k, v))
    o = backend.attention.flash_attention2(qs, ks, vs, 8, 64, scale=0.125)
    assert o.shape == (32, 64, 8, 64) and O.max_rel(o, O.truth_attention(qs, ks, vs, scale=0.125)) < TOL_F32
    o2 = backend.attention.flash_attention2(q, k, v, 8, 64, layout="bhsd")
    np.testing.assert_array_equal(o2, o)


def test_minilm_full_batch_fp32(backend, corc):
    """configs[1] at its full size: 6 post-LN layers, d=384, 12x32 heads, FFN 1536, fp32, batch 64 x seq 256,
    lengths uniform in [32,256].  Two sampled sequences (the shortest and another one) through the C oracle
    (fp32, shader summation order) and the float64 oracle; every sequence's real positions must be finite and the
    pooled rows unit vectors equal to the masked mean of the hidden states."""
    from grilly_amd.encoder import MINILM_L6 as cfg
    w = random_bert_weights(cfg, seed=20260133)
    rng = rng_for(2)
    B, S = 64, 256
    ids = rng.integers(0, cfg.vocab, (B, S))
    lens = rng.integers(32, 257, B)
    mask = (np.arange(S)[None] < lens[:, None]).astype(np.float32)
    enc = BertEncoder(backend, cfg, w, dtype="fp32")
    h = enc.forward(ids, mask, pool=False)
    assert h.shape == (B, S, cfg.d_model) and np.isfinite(h).all()
    for b in (int(np.argmin(lens)), 41):
        x = corc.layernorm(corc.embed(ids[b:b + 1], w["tok_emb"], w["pos_emb"], w["type_emb"]), w["emb_ln_g"], w["emb_ln_b"], cfg.eps)
        for lw in w["layers"]:
            x = corc.bert_layer(x, lw, mask[b:b + 1], cfg.heads, cfg.eps)
        assert O.max_rel(h[b:b + 1], x) < TOL_F32, b
        assert O.max_rel(h[b:b + 1], truth_encoder(w, cfg, ids[b:b + 1], mask[b:b + 1])) < TOL_F32, b
    pooled = enc.forward(ids, mask, pool=True)
    assert O.max_rel(pooled, O.truth_mean_pool(h, mask)) < 1e-4
    np.testing.assert_allclose(np.linalg.norm(pooled, axis=1), 1.0, atol=1e-5)
    enc.release_activations()


def test_bert_base_layer_fp32_full_width(backend):
    """configs[2], fp32 leg: one layer at full width (d=768, 12x64 heads, FFN 3072, fused QKV), batch 2 x seq 512,
    every position against the float64 oracle at 1e-4."""
    cfg = EncoderConfig(layers=1)
    w = random_bert_weights(cfg, seed=20260134)
    rng = rng_for(3)
    B, S = 2, 512
    ids = rng.integers(0, cfg.vocab, (B, S))
    enc = BertEncoder(backend, cfg, w, dtype="fp32")
    h = enc.forward(ids, None, pool=False)
    ref = truth_encoder(w, cfg, ids, None)
    assert O.max_rel(h, ref) < TOL_F32
    assert np.abs(h.mean(-1)).max() < 1e-4 and np.abs(h.var(-1) - 1).max() < 1e-3
    enc.release_activations()


def test_bert_base_forward_fp32_b128(backend, corc):
    """configs[2], fp32 leg at the benchmark size (12 layers, batch 128 x seq 512, M = 65536 rows per GEMM):
    sampled sequences equal their own batch-of-one runs (other tile walk, same arithmetic up to summation order),
    one sampled sequence through all 12 layers against the C oracle (fp32, shader order), and the first layer at
    full batch width against the float64 oracle."""
    cfg = EncoderConfig()
    w = random_bert_weights(cfg, seed=20260134)
    rng = rng_for(3)
    B, S = 128, 512
    ids = rng.integers(0, cfg.vocab, (B, S))
    enc = BertEncoder(backend, cfg, w, dtype="fp32")
    h = enc.forward(ids, None, pool=False)
    assert h.shape == (B, S, cfg.d_model) and np.isfinite(h).all()
    for b in (0, 77, 127):
        one = enc.forward(ids[b:b + 1], None, pool=False)
        assert O.max_rel(h[b:b + 1], one) < 2e-5, b
    x = corc.layernorm(corc.embed(ids[77:78], w["tok_emb"], w["pos_emb"], w["type_emb"]), w["emb_ln_g"], w["emb_ln_b"], cfg.eps)
    for lw in w["layers"]:
        x = corc.bert_layer(x, lw, None, cfg.heads, cfg.eps)
    assert O.max_rel(h[77:78], x) < TOL_F32
    enc.release_activations()
    cfg1 = EncoderConfig(layers=1)
    w1 = dict(w, layers=w["layers"][:1])
    enc1 = BertEncoder(backend, cfg1, w1, dtype="fp32")
    h1 = enc1.forward(ids, None, pool=False)
    for b in (3, 126):
        assert O.max_rel(h1[b:b + 1], truth_encoder(w1, cfg1, ids[b:b + 1], None)) < TOL_F32, b
    enc1.release_activations()


def test_swiglu_mlp_full_rows(backend):
    """configs[3] at its full size: X[16384,4096], W_g / W_u [11008,4096], W_d [4096,11008], bf16 storage with fp32
    accumulation.  H = silu(X.W_g^T) * (X.W_u^T) and Y = H.W_d^T on rows sampled from every 256-row tile band
    against the float64 oracle on the bf16-rounded inputs; the stored H is bf16-exact; the down projection is
    exactly homogeneous under a factor 2."""
    rng = rng_for(4)
    M, Kd, F = 16384, 4096, 11008
    X = O.bf16_round(rng.standard_normal((M, Kd), dtype=np.float32))
    Wg = O.bf16_round(rng.standard_normal((F, Kd), dtype=np.float32) * np.float32(0.02))
    Wu = O.bf16_round(rng.standard_normal((F, Kd), dtype=np.float32) * np.float32(0.02))
    Wd = O.bf16_round(rng.standard_normal((Kd, F), dtype=np.float32) * np.float32(0.02))
    rows = band_rows(M, rng, per=1)
    # the configuration wants SiLU on the gate product: the reference's fused_swiglu activates its W_up argument
    Hh = backend.fnn.fused_swiglu(X, Wu, Wg, dtype="bf16")
    assert Hh.shape == (M, F) and np.isfinite(Hh).all()
    xs = X[rows].astype(np.float64)
    want_h = O.truth_silu(xs @ Wg.T.astype(np.float64)) * (xs @ Wu.T.astype(np.float64))
    assert O.max_rel(Hh[rows], want_h) < TOL_BF16
    np.testing.assert_array_equal(O.bf16_round(Hh[rows]), Hh[rows])
    del X, Wg, Wu
    Y = backend.fnn.linear(Hh, Wd, dtype="bf16")
    assert Y.shape == (M, Kd) and np.isfinite(Y).all()
    assert O.max_rel(Y[rows], O.truth_linear(Hh[rows], Wd)) < TOL_BF16
    Y2 = backend.fnn.linear(2 * Hh[:2048], Wd, dtype="bf16")
    np.testing.assert_array_equal(Y2, 2 * Y[:2048])


def test_long_causal_rope_attention_full_batch(backend):
    """configs[4] at its full size: (B,S,H,D) = (4,8192,32,128), bf16, causal, interleaved RoPE base 10000.
    Row 0 of every (batch, head) is V[0]; every output is a convex combination of V rows; sampled (b, h, i) query
    rows against the float64 closed form (row i needs keys 0..i only)."""
    rng = rng_for(5)
    B, S, H, D = 4, 8192, 32, 128
    q, k, v = (O.bf16_round(rng.standard_normal((B, S, H, D), dtype=np.float32)) for _ in range(3))
    o = backend.attention.flash_attention2_rope(q, k, v, H, D, causal=True, dtype="bf16")
    assert o.shape == (B, S, H, D) and np.isfinite(o).all()
    np.testing.assert_allclose(o[:, 0], v[:, 0], atol=1e-2)
    assert (o.max(axis=1) <= v.max(axis=1) + 1e-2).all() and (o.min(axis=1) >= v.min(axis=1) - 1e-2).all()
    for (b, h, i) in [(0, 0, 1), (1, 5, 127), (2, 17, 128), (3, 31, 4097), (0, 9, 8191), (1, 30, 2049), (3, 0, 255), (2, 31, 6144)]:
        qr = O.truth_rope(q[b:b + 1, i:i + 1, h:h + 1], style="interleaved", position_ids=np.array([[i]]))[0, 0, 0]
        kr = O.truth_rope(k[b:b + 1, :i + 1, h:h + 1], style="interleaved")[0, :, 0]
        s = kr @ qr / np.sqrt(D)
        p = np.exp(s - s.max()); p /= p.sum()
        ref = p @ v[b, :i + 1, h].astype(np.float64)
        assert O.max_rel(o[b, i, h], ref) < TOL_BF16, (b, h, i)
