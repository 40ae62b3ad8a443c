"""nn adapters on the HIP backend against the float64 oracle (fp32 path, tolerance 1e-4)."""
import numpy as np
import pytest

from conftest import TOL_F32
from grilly_amd import nn
from oracle import oracle_np as O

pytestmark = pytest.mark.gpu


def test_linear_module_both_routes(backend):
    rng = np.random.default_rng(31)
    np.random.seed(31)
    lin = nn.Linear(96, 80).to_backend(backend)
    lin.bias.data[:] = rng.standard_normal(80)
    small = rng.standard_normal((7, 96)).astype(np.float32)            # 560 outputs: fused linear
    big = rng.standard_normal((3, 40, 96)).astype(np.float32)          # 9600 outputs: gemm on the transposed view
    for x in (small, big):
        y = lin(x)
        assert y.shape == x.shape[:-1] + (80,) and y.dtype == np.float32
        assert O.max_rel(y, O.truth_linear(x, lin.weight.data, lin.bias.data)) < TOL_F32


def test_layernorm_and_activation_modules(backend):
    rng = np.random.default_rng(32)
    x = rng.standard_normal((4, 9, 64)).astype(np.float32) * 3
    ln = nn.LayerNorm(64, eps=1e-6).to_backend(backend)
    ln.weight.data[:] = rng.standard_normal(64); ln.bias.data[:] = rng.standard_normal(64)
    assert O.max_rel(ln(x), O.truth_layernorm(x, ln.weight.data, ln.bias.data, 1e-6)) < TOL_F32
    assert O.max_rel(nn.GELU().to_backend(backend)(x), O.truth_gelu(x)) < TOL_F32
    assert O.max_rel(nn.SiLU().to_backend(backend)(x), O.truth_silu(x)) < TOL_F32
    np.testing.assert_array_equal(nn.ReLU().to_backend(backend)(x), np.maximum(x, 0))
    xb = O.bf16_round(x)
    np.testing.assert_array_equal(backend.fnn.activation_relu(xb, dtype="bf16"), np.maximum(xb, 0))


def test_flash_attention_module(backend):
    rng = np.random.default_rng(33)
    q, k, v = (rng.standard_normal((2, 70, 128)).astype(np.float32) for _ in range(3))
    mask = (np.arange(70)[None] < np.array([70, 33])[:, None]).astype(np.float32)
    fa = nn.FlashAttention2(128, 4).to_backend(backend)
    o = fa(q, k, v, mask)
    sh = (2, 70, 4, 32)
    assert o.shape == sh
    assert O.max_rel(o, O.truth_attention(q.reshape(sh), k.reshape(sh), v.reshape(sh), mask=mask)) < TOL_F32
    far = nn.FlashAttention2(128, 4, use_rope=True).to_backend(backend)
    assert O.max_rel(far(q, k, v), O.truth_attention(q.reshape(sh), k.reshape(sh), v.reshape(sh), rope="interleaved")) < TOL_F32


@pytest.mark.parametrize("act", ["gelu", "relu"])
def test_transformer_encoder_layer(backend, act):
    np.random.seed(34)
    rng = np.random.default_rng(34)
    d, H, ff, B, S = 128, 4, 320, 3, 50
    layer = nn.TransformerEncoderLayer(d, H, dim_feedforward=ff, activation=act).to_backend(backend).eval()
    for n, p in layer.named_parameters():
        if n.startswith("norm"):
            p.data[...] = 1.0 + 0.1 * rng.standard_normal(p.shape) if n.endswith("weight") else 0.1 * rng.standard_normal(p.shape)
        else:
            p.data[...] = rng.standard_normal(p.shape) * (0.08 if n.endswith("weight") else 0.05)
    x = rng.standard_normal((B, S, d)).astype(np.float32)
    mask = (np.arange(S)[None] < np.array([50, 20, 1])[:, None]).astype(np.float32)
    y = layer(x, mask)
    P = {n: p.data.astype(np.float64) for n, p in layer.named_parameters()}
    h = O.truth_layernorm(x, P["norm1.weight"], P["norm1.bias"])
    proj = lambda t, n: t @ P[f"self_attn.{n}.weight"].T + P[f"self_attn.{n}.bias"]
    sh = (B, S, H, d // H)
    a = O.truth_attention(proj(h, "q_proj").reshape(sh), proj(h, "k_proj").reshape(sh), proj(h, "v_proj").reshape(sh), mask=mask)
    x1 = x + proj(a.reshape(B, S, d), "out_proj")
    h2 = O.truth_layernorm(x1, P["norm2.weight"], P["norm2.bias"])
    f = h2 @ P["linear1.weight"].T + P["linear1.bias"]
    f = O.truth_gelu(f) if act == "gelu" else np.maximum(f, 0)
    ref = x1 + f @ P["linear2.weight"].T + P["linear2.bias"]
    assert y.shape == (B, S, d)
    assert O.max_rel(y, ref) < TOL_F32


@pytest.mark.parametrize("Sq,Sk", [(30, 30), (17, 45), (40, 9)])
def test_multihead_attention_weights_and_cross_length(backend, Sq, Sk):
    """MultiheadAttention returns (output, weights (B,H,Sq,Sk)) like the reference (nn/modules.py:1123-1216), also
    when key / value are longer or shorter than the query; with need_weights=False the fused kernel gives the
    same output."""
    np.random.seed(35)
    rng = np.random.default_rng(35)
    d, H, B = 96, 4, 2
    mha = nn.MultiheadAttention(d, H).to_backend(backend)
    for n, p in mha.named_parameters():
        p.data[...] = rng.standard_normal(p.shape) * (0.1 if n.endswith("weight") else 0.05)
    q = rng.standard_normal((B, Sq, d)).astype(np.float32)
    kv = q if Sk == Sq else rng.standard_normal((B, Sk, d)).astype(np.float32)
    mask = (np.arange(Sk)[None] < np.array([Sk, max(Sk // 2, 1)])[:, None]).astype(np.float32)
    out, w = mha(q, kv, kv, mask)
    P = {n: p.data.astype(np.float64) for n, p in mha.named_parameters()}
    proj = lambda t, n: t @ P[f"{n}.weight"].T + P[f"{n}.bias"]
    D = d // H
    qh = proj(q, "q_proj").reshape(B, Sq, H, D); kh = proj(kv, "k_proj").reshape(B, Sk, H, D); vh = proj(kv, "v_proj").reshape(B, Sk, H, D)
    sc = np.einsum("bqhd,bkhd->bhqk", qh, kh) / np.sqrt(D) + ((mask.astype(np.float64) - 1) * 1e9)[:, None, None, :]
    pw = np.exp(sc - sc.max(-1, keepdims=True)); pw /= pw.sum(-1, keepdims=True)
    ref = proj(np.einsum("bhqk,bkhd->bqhd", pw, vh).reshape(B, Sq, d), "out_proj")
    assert out.shape == (B, Sq, d) and w.shape == (B, H, Sq, Sk)
    assert O.max_rel(w, pw) < TOL_F32 and O.max_rel(out, ref) < TOL_F32
    np.testing.assert_allclose(w.sum(-1), 1.0, atol=1e-5)
    if Sq == Sk:
        out2, none = mha(q, kv, kv, mask, need_weights=False)
        assert none is None and O.max_rel(out2, ref) < TOL_F32


def test_nn_modules_randomized(backend):
    """Seeded sweep over the attention-bearing modules at random widths, head counts (head dims that run the MFMA
    kernels directly and head dims that run on padded copies), sequence lengths (query and key lengths apart for
    MultiheadAttention), FFN widths, activations and key masks, against the float64 composition of the pinned pieces."""
    from conftest import sweep_rounds
    rng = np.random.default_rng(55006)
    for case in range(12 * sweep_rounds()):
        np.random.seed(1000 + case)
        H = int(rng.choice([1, 2, 3, 4]))
        D = int(rng.choice([8, 24, 32, 64]))
        d, B = H * D, int(rng.integers(1, 4))
        if case % 2 == 0:
            S, ff = int(rng.choice([1, 9, 50, 130])), 8 * int(rng.integers(1, 60))
            act = ["gelu", "relu"][int(rng.integers(0, 2))]
            layer = nn.TransformerEncoderLayer(d, H, dim_feedforward=ff, activation=act).to_backend(backend).eval()
            for n, p in layer.named_parameters():
                if n.startswith("norm"):
                    p.data[...] = 1.0 + 0.1 * rng.standard_normal(p.shape) if n.endswith("weight") else 0.1 * rng.standard_normal(p.shape)
                else:
                    p.data[...] = rng.standard_normal(p.shape) * (0.08 if n.endswith("weight") else 0.05)
            x = rng.standard_normal((B, S, d)).astype(np.float32)
            mask = None
            if rng.random() < 0.6:
                mask = (np.arange(S)[None] < rng.integers(1, S + 1, B)[:, None]).astype(np.float32)
            y = layer(x, mask)
            P = {n: p.data.astype(np.float64) for n, p in layer.named_parameters()}
            h = O.truth_layernorm(x, P["norm1.weight"], P["norm1.bias"])
            proj = lambda t, n: t @ P[f"self_attn.{n}.weight"].T + P[f"self_attn.{n}.bias"]
            sh = (B, S, H, D)
            a = O.truth_attention(proj(h, "q_proj").reshape(sh), proj(h, "k_proj").reshape(sh), proj(h, "v_proj").reshape(sh), mask=mask)
            x1 = x + proj(a.reshape(B, S, d), "out_proj")
            h2 = O.truth_layernorm(x1, P["norm2.weight"], P["norm2.bias"])
            f = h2 @ P["linear1.weight"].T + P["linear1.bias"]
            f = O.truth_gelu(f) if act == "gelu" else np.maximum(f, 0)
            ref = x1 + f @ P["linear2.weight"].T + P["linear2.bias"]
            assert y.shape == (B, S, d)
            assert O.max_rel(y, ref) < TOL_F32, (case, "layer", d, H, ff, act, B, S, mask is not None)
        else:
            Sq, Sk = int(rng.choice([1, 7, 40, 100])), int(rng.choice([1, 9, 45, 130]))
            mha = nn.MultiheadAttention(d, H).to_backend(backend)
            for n, p in mha.named_parameters():
                p.data[...] = rng.standard_normal(p.shape) * (0.1 if n.endswith("weight") else 0.05)
            q = rng.standard_normal((B, Sq, d)).astype(np.float32)
            kv = rng.standard_normal((B, Sk, d)).astype(np.float32)
            mask = (np.arange(Sk)[None] < rng.integers(1, Sk + 1, B)[:, None]).astype(np.float32)
            out, w = mha(q, kv, kv, mask)
            P = {n: p.data.astype(np.float64) for n, p in mha.named_parameters()}
            proj = lambda t, n: t @ P[f"{n}.weight"].T + P[f"{n}.bias"]
            qh = proj(q, "q_proj").reshape(B, Sq, H, D); kh = proj(kv, "k_proj").reshape(B, Sk, H, D); vh = proj(kv, "v_proj").reshape(B, Sk, H, D)
            sc = np.einsum("bqhd,bkhd->bhqk", qh, kh) / np.sqrt(D) + ((mask.astype(np.float64) - 1) * 1e9)[:, None, None, :]
            pw = np.exp(sc - sc.max(-1, keepdims=True)); pw /= pw.sum(-1, keepdims=True)
            ref = proj(np.einsum("bhqk,bkhd->bqhd", pw, vh).reshape(B, Sq, d), "out_proj")
            assert out.shape == (B, Sq, d) and w.shape == (B, H, Sq, Sk)
            assert O.max_rel(w, pw) < TOL_F32 and O.max_rel(out, ref) < TOL_F32, (case, "mha", d, H, B, Sq, Sk)
        if case and case % 20 == 0:
            print("sweep case", case, flush=True)
