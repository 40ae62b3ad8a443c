"""Host logic of the nn adapters (grilly_amd/nn.py) against a recording stand-in backend: routing,
shapes, parameter names, error behaviour.  No GPU: the stand-in computes in numpy inside this test only."""
import numpy as np
import pytest

from grilly_amd import nn
from oracle import oracle_np as O


class _FNN:
    def __init__(self, log):
        self.log = log

    def gemm(self, A, B):
        self.log.append(("gemm", A.shape, B.shape, B.base is not None and B.T.flags["C_CONTIGUOUS"]))
        return (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)

    def linear(self, x, W, b=None):
        self.log.append(("linear", x.shape, W.shape, b is not None))
        return O.truth_linear(x, W, b).astype(np.float32)

    def layernorm(self, x, g, b, eps=1e-5):
        self.log.append(("layernorm", x.shape, eps))
        return O.truth_layernorm(x, g, b, eps).astype(np.float32)

    def activation_gelu(self, x):
        self.log.append(("gelu", x.shape)); return O.truth_gelu(x).astype(np.float32)

    def activation_silu(self, x):
        self.log.append(("silu", x.shape)); return O.truth_silu(x).astype(np.float32)

    def activation_relu(self, x):
        self.log.append(("relu", x.shape)); return np.maximum(x, 0).astype(np.float32)


class _Att:
    def __init__(self, log):
        self.log = log

    def flash_attention2(self, q, k, v, H, D, mask=None):
        self.log.append(("fa2", q.shape, H, D, mask is not None))
        return O.truth_attention(q, k, v, mask=mask).astype(np.float32)

    def flash_attention2_rope(self, q, k, v, H, D, mask=None):
        self.log.append(("fa2_rope", q.shape, H, D, mask is not None))
        return O.truth_attention(q, k, v, mask=mask, rope="interleaved").astype(np.float32)


class FakeBackend:
    def __init__(self):
        self.log = []
        self.fnn, self.attention = _FNN(self.log), _Att(self.log)


def test_linear_routing_shapes_and_errors():
    be = FakeBackend()
    np.random.seed(0)
    lin = nn.Linear(24, 16).to_backend(be)
    lin.bias.data[:] = np.arange(16)
    assert lin.weight.shape == (16, 24) and abs(lin.weight.data).max() <= np.sqrt(6 / 40) + 1e-7
    x = np.random.default_rng(1).standard_normal((8, 24)).astype(np.float32)
    y = lin(x)                                       # 8*16 = 128 < 4096 -> fused linear with the bias inside
    assert be.log[-1] == ("linear", (8, 24), (16, 24), True) and y.shape == (8, 16)
    np.testing.assert_allclose(y, x @ lin.weight.data.T + lin.bias.data, rtol=1e-5, atol=1e-5)
    x3 = np.random.default_rng(2).standard_normal((4, 64, 24)).astype(np.float32)
    y3 = lin(x3)                                     # 256*16 = 4096 -> gemm(x, W.T), bias on the host
    assert be.log[-1][0] == "gemm" and be.log[-1][1:3] == ((256, 24), (24, 16)) and be.log[-1][3]
    assert y3.shape == (4, 64, 16)
    np.testing.assert_allclose(y3, x3 @ lin.weight.data.T + lin.bias.data, rtol=1e-5, atol=1e-5)
    nb = nn.Linear(24, 16, bias=False).to_backend(be)
    assert nb.bias is None and [n for n, _ in nb.named_parameters()] == ["weight"]
    for bad in (np.zeros(24, np.float32), np.zeros((2, 2, 2, 24), np.float32)):
        with pytest.raises(ValueError):
            lin(bad)
    with pytest.raises(ValueError):
        lin(np.zeros((3, 23), np.float32))


def test_modules_register_and_toggle():
    layer = nn.TransformerEncoderLayer(32, 4, dim_feedforward=48, dropout=0.25)
    names = [n for n, _ in layer.named_parameters()]
    for want in ("self_attn.q_proj.weight", "self_attn.out_proj.bias", "linear1.weight", "linear2.bias", "norm1.weight", "norm2.bias"):
        assert want in names
    assert len(list(layer.parameters())) == 16
    assert layer.training and layer.dropout1.training
    layer.eval()
    assert not layer.training and not layer.self_attn.q_proj.training and not layer.dropout2.training
    assert layer.dim_feedforward == 48 and nn.TransformerEncoderLayer(32, 4).dim_feedforward == 128
    with pytest.raises(ValueError):
        nn.TransformerEncoderLayer(32, 4, activation="tanh")
    with pytest.raises(NotImplementedError):
        nn.TransformerEncoderLayer(32, 4, use_prosody=True)
    with pytest.raises(ValueError):
        nn.FlashAttention2(30, 4)
    with pytest.raises(ValueError):
        nn.MultiheadAttention(30, 4)


def test_dropout_modes():
    d = nn.Dropout(0.5)
    x = np.ones((64, 64), np.float32)
    np.random.seed(3)
    y = d(x)
    assert set(np.unique(y)) <= {0.0, 2.0} and 0.3 < (y == 0).mean() < 0.7
    assert d.eval()(x) is x and nn.Dropout(0.0)(x) is x


def test_flash_attention_module_reshapes():
    be = FakeBackend()
    fa = nn.FlashAttention2(32, 4).to_backend(be)
    rng = np.random.default_rng(4)
    q, k, v = (rng.standard_normal((2, 10, 32)).astype(np.float32) for _ in range(3))
    o = fa(q, k, v)
    assert o.shape == (2, 10, 4, 8) and be.log[-1] == ("fa2", (2, 10, 4, 8), 4, 8, False)
    nn.FlashAttention2(32, 4, use_rope=True).to_backend(be)(q.reshape(2, 10, 4, 8), k.reshape(2, 10, 4, 8), v.reshape(2, 10, 4, 8))
    assert be.log[-1][0] == "fa2_rope"


@pytest.mark.parametrize("act", ["gelu", "relu", "silu"])
def test_encoder_layer_wiring(act):
    """pre-LN: x + attn(norm1 x), then x + linear2(act(linear1(norm2 x))) (reference nn/transformer.py:355-369)"""
    be = FakeBackend()
    np.random.seed(5)
    layer = nn.TransformerEncoderLayer(32, 4, dim_feedforward=64, activation=act).to_backend(be).eval()
    rng = np.random.default_rng(6)
    for _, p in layer.named_parameters():
        p.data[...] = rng.standard_normal(p.shape) * 0.2
    x = rng.standard_normal((2, 12, 32)).astype(np.float32)
    mask = (np.arange(12)[None] < np.array([12, 7])[:, None]).astype(np.float32)
    y = layer(x, mask)
    P = {n: p.data.astype(np.float64) for n, p in layer.named_parameters()}
    h = O.truth_layernorm(x, P["norm1.weight"], P["norm1.bias"])
    q = h @ P["self_attn.q_proj.weight"].T + P["self_attn.q_proj.bias"]
    k = h @ P["self_attn.k_proj.weight"].T + P["self_attn.k_proj.bias"]
    v = h @ P["self_attn.v_proj.weight"].T + P["self_attn.v_proj.bias"]
    a = O.truth_attention(q.reshape(2, 12, 4, 8), k.reshape(2, 12, 4, 8), v.reshape(2, 12, 4, 8), mask=mask).reshape(2, 12, 32)
    x1 = x + a @ P["self_attn.out_proj.weight"].T + P["self_attn.out_proj.bias"]
    h2 = O.truth_layernorm(x1, P["norm2.weight"], P["norm2.bias"])
    f = h2 @ P["linear1.weight"].T + P["linear1.bias"]
    f = {"gelu": O.truth_gelu, "silu": O.truth_silu, "relu": lambda t: np.maximum(t, 0)}[act](f)
    ref = x1 + f @ P["linear2.weight"].T + P["linear2.bias"]
    assert O.max_rel(y, ref) < 1e-5
    kinds = [e[0] for e in be.log]
    assert kinds.count("layernorm") == 2 and kinds.count("fa2") == 1 and kinds.count(act) == 1
