"""Forward-only `nn`-style adapters over the HIP facade, so Module code written against the
reference (nn/module.py:39-140, nn/modules.py, nn/transformer.py:240-372) runs on this backend:
same class names, constructor arguments, parameter names and call conventions.

Differences, all on purpose:
  * forward only (the reference's backward methods belong to its autograd path);
  * no CPU fallback: a failing backend call raises instead of silently recomputing in numpy;
  * MultiheadAttention with need_weights=False goes through the fused attention kernel (which never forms
    the weights) and returns (output, None); with need_weights=True, or key / value of another length than the
    query, it takes the score GEMM -> softmax -> output GEMM route and returns (output, weights (B,H,Sq,Sk)).
"""
import numpy as np

_default_backend = None


def _backend():
    global _default_backend
    if _default_backend is None:
        from . import Compute
        _default_backend = Compute()
    return _default_backend


class Parameter:
    """numpy array with a .grad slot (reference nn/modules.py:50-83 ParamWrapper)."""

    def __init__(self, data, requires_grad=True):
        self.data = np.array(data, dtype=np.float32)
        self.grad = None
        self.requires_grad = requires_grad

    def __array__(self, dtype=None, copy=None):
        return self.data if dtype is None else self.data.astype(dtype)

    def __getitem__(self, key):
        return self.data[key]

    def __setitem__(self, key, value):
        self.data[key] = value

    @property
    def shape(self):
        return self.data.shape

    @property
    def dtype(self):
        return self.data.dtype

    def copy(self):
        return Parameter(self.data.copy(), self.requires_grad)

    def zero_grad(self):
        self.grad = np.zeros_like(self.data)


def _array(p):
    return p.data if isinstance(p, Parameter) else np.asarray(p, dtype=np.float32)


class Module:
    """Reference nn/module.py:39-140."""

    def __init__(self):
        self.training = True
        self._parameters = {}
        self._buffers = {}
        self._modules = {}
        self._backend = None

    def _get_backend(self):
        return self._backend if self._backend is not None else _backend()

    def to_backend(self, backend):
        """Use `backend` (a grilly_amd.Compute) for this module and its children."""
        self._backend = backend
        for m in self._modules.values():
            m.to_backend(backend)
        return self

    def register_parameter(self, name, param):
        self._parameters[name] = param

    @staticmethod
    def _convert_input(x):
        # torch / TF tensors arrive as numpy (reference nn/module.py:55-94)
        if isinstance(x, np.ndarray) or x is None:
            return x
        if hasattr(x, "detach") and hasattr(x, "cpu"):
            return x.detach().cpu().numpy()
        if hasattr(x, "numpy"):
            return x.numpy()
        return x

    def forward(self, *args, **kwargs):
        raise NotImplementedError

    def __call__(self, *args, **kwargs):
        args = tuple(self._convert_input(a) for a in args)
        kwargs = {k: self._convert_input(v) for k, v in kwargs.items()}
        return self.forward(*args, **kwargs)

    def train(self, mode=True):
        self.training = mode
        for m in self._modules.values():
            m.train(mode)
        return self

    def eval(self):
        return self.train(False)

    def parameters(self):
        yield from self._parameters.values()
        for m in self._modules.values():
            yield from m.parameters()

    def named_parameters(self):
        yield from self._parameters.items()
        for prefix, m in self._modules.items():
            for name, p in m.named_parameters():
                yield f"{prefix}.{name}", p

    def __setattr__(self, name, value):
        # child modules register themselves (the reference fills _modules by hand)
        if isinstance(value, Module) and "_modules" in self.__dict__:
            self._modules[name] = value
        object.__setattr__(self, name, value)


class Linear(Module):
    """y = x.W^T + b, W (out_features, in_features) (reference nn/modules.py:20-180).
    Rank-2 / rank-3 inputs; `batch_seq * out_features >= 4096` takes the gemm(x, W.T) route with the
    bias added on the host, smaller problems the fused linear (reference :146-170).  On this backend
    both routes end in the same GEMM kernel (gemm recognises the transposed view)."""

    GEMM_SWITCH = 4096

    def __init__(self, in_features, out_features, bias=True):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        limit = np.sqrt(6.0 / (in_features + out_features))       # Xavier uniform, reference :41-43
        self.weight = Parameter(np.random.uniform(-limit, limit, (out_features, in_features)))
        self.bias = Parameter(np.zeros(out_features)) if bias else None
        self.register_parameter("weight", self.weight)
        if self.bias is not None:
            self.register_parameter("bias", self.bias)

    def forward(self, x):
        backend = self._get_backend()
        W = _array(self.weight)
        b = _array(self.bias) if self.bias is not None else None
        x = np.asarray(x, dtype=np.float32)
        if x.ndim == 2:
            x2 = x
        elif x.ndim == 3:
            x2 = x.reshape(x.shape[0] * x.shape[1], x.shape[2])
        else:
            raise ValueError(f"Linear expects 2D or 3D input, got shape {x.shape}")
        if x2.shape[1] != self.in_features:
            raise ValueError(f"Linear expects {self.in_features} input features, got {x2.shape[1]}")
        if x2.shape[0] * self.out_features >= self.GEMM_SWITCH:
            out = backend.fnn.gemm(x2, W.T)
            if b is not None:
                out += b.reshape(1, self.out_features)
        else:
            out = backend.fnn.linear(x2, W, b)
        return out if x.ndim == 2 else out.reshape(x.shape[0], x.shape[1], self.out_features)

    def __repr__(self):
        return f"Linear(in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None})"


class LayerNorm(Module):
    """Reference nn/modules.py:340-366."""

    def __init__(self, normalized_shape, eps=1e-5):
        super().__init__()
        self.normalized_shape, self.eps = normalized_shape, eps
        self.weight = Parameter(np.ones(normalized_shape))
        self.bias = Parameter(np.zeros(normalized_shape))
        self.register_parameter("weight", self.weight)
        self.register_parameter("bias", self.bias)

    def forward(self, x):
        return self._get_backend().fnn.layernorm(x, _array(self.weight), _array(self.bias), eps=self.eps)


class Dropout(Module):
    """Identity in eval mode; in training mode a host-side Bernoulli mask scaled by 1/(1-p), which is
    what the reference does as well (nn/modules.py:450-471)."""

    def __init__(self, p=0.5, inplace=False):
        super().__init__()
        self.p, self.inplace = p, inplace
        self._mask = None

    def forward(self, x):
        if not self.training or self.p == 0.0:
            self._mask = None
            return x
        self._mask = np.random.binomial(1, 1 - self.p, size=np.shape(x)).astype(np.float32)
        return np.asarray(x, np.float32) * self._mask / (1 - self.p)


class ReLU(Module):
    def __init__(self, inplace=False):
        super().__init__()
        self.inplace = inplace

    def forward(self, x):
        return self._get_backend().fnn.activation_relu(x)


class GELU(Module):
    def forward(self, x):
        return self._get_backend().fnn.activation_gelu(x)


class SiLU(Module):
    def forward(self, x):
        return self._get_backend().fnn.activation_silu(x)


class FlashAttention2(Module):
    """Reference nn/modules.py:1361-1412: q, k, v as (batch, seq, heads, head_dim) or (batch, seq, embed);
    the result is always (batch, seq, heads, head_dim), as the reference returns it."""

    def __init__(self, embed_dim, num_heads, use_rope=False):
        super().__init__()
        if embed_dim % num_heads != 0:
            raise ValueError(f"embed_dim ({embed_dim}) must be divisible by num_heads ({num_heads})")
        self.embed_dim, self.num_heads, self.head_dim, self.use_rope = embed_dim, num_heads, embed_dim // num_heads, use_rope

    def forward(self, q, k, v, mask=None):
        q, k, v = (np.asarray(t, dtype=np.float32) for t in (q, k, v))
        if q.ndim == 3:
            B, S, _ = q.shape
            q, k, v = (t.reshape(B, S, self.num_heads, self.head_dim) for t in (q, k, v))
        att = self._get_backend().attention
        fn = att.flash_attention2_rope if self.use_rope else att.flash_attention2
        return fn(q, k, v, self.num_heads, self.head_dim, mask=mask)


class MultiheadAttention(Module):
    """q/k/v/out projections around attention (reference nn/modules.py:1085-1222 builds the block from separate
    score / softmax / output steps).  Returns (output, attention_weights) with weights (batch, heads, query_len,
    key_len) like the reference; key and value may be longer or shorter than the query.  `mask` is a
    (batch, key_len) keep-mask (1 keep, 0 drop).  With need_weights=False the fused kernel runs (query and key
    of the same length) and the second result is None."""

    def __init__(self, embed_dim, num_heads, dropout=0.0):
        super().__init__()
        if embed_dim % num_heads != 0:
            raise ValueError(f"embed_dim ({embed_dim}) must be divisible by num_heads ({num_heads})")
        self.embed_dim, self.num_heads, self.head_dim, self.dropout = embed_dim, num_heads, embed_dim // num_heads, dropout
        self.q_proj = Linear(embed_dim, embed_dim)
        self.k_proj = Linear(embed_dim, embed_dim)
        self.v_proj = Linear(embed_dim, embed_dim)
        self.out_proj = Linear(embed_dim, embed_dim)

    def forward(self, query, key, value, mask=None, need_weights=True):
        q, k, v = self.q_proj(query), self.k_proj(key), self.v_proj(value)
        B, S, _ = q.shape
        Sk = k.shape[1]
        if v.shape[1] != Sk:
            raise ValueError("key and value must have the same length")
        qs, ks = (B, S, self.num_heads, self.head_dim), (B, Sk, self.num_heads, self.head_dim)
        att = self._get_backend().attention
        if need_weights or Sk != S:
            o, w = att.attention_with_weights(q.reshape(qs), k.reshape(ks), v.reshape(ks), mask=mask)
        else:
            o, w = att.flash_attention2(q.reshape(qs), k.reshape(ks), v.reshape(ks), self.num_heads, self.head_dim, mask=mask), None
        return self.out_proj(o.reshape(B, S, self.embed_dim)), w

    def __repr__(self):
        return f"MultiheadAttention(embed_dim={self.embed_dim}, num_heads={self.num_heads})"


class TransformerEncoderLayer(Module):
    """Pre-LN encoder layer of the reference (nn/transformer.py:264-372):
    x = x + dropout1(attn(norm1(x)));  x = x + linear2(dropout2(act(linear1(norm2(x)))))."""

    def __init__(self, d_model, nhead, dim_feedforward=None, dropout=0.1, activation="gelu", use_rope=False,
                 use_prosody=False):
        super().__init__()
        if use_prosody:
            raise NotImplementedError("prosody-modulated attention is outside this backend's path")
        self.d_model, self.nhead = d_model, nhead
        self.dim_feedforward = dim_feedforward or 4 * d_model
        self.dropout, self.use_rope, self.use_prosody = dropout, use_rope, use_prosody
        self.self_attn = MultiheadAttention(d_model, nhead, dropout=dropout)
        self.linear1 = Linear(d_model, self.dim_feedforward)
        self.linear2 = Linear(self.dim_feedforward, d_model)
        self.norm1, self.norm2 = LayerNorm(d_model), LayerNorm(d_model)
        self.dropout1, self.dropout2 = Dropout(dropout), Dropout(dropout)
        acts = {"gelu": GELU, "relu": ReLU, "silu": SiLU}
        if activation not in acts:
            raise ValueError(f"Unknown activation: {activation}")
        self.activation = acts[activation]()

    def forward(self, src, src_mask=None, prosody=None):
        src = np.asarray(src, dtype=np.float32)
        src2 = self.norm1(src)
        src2, _ = self.self_attn(src2, src2, src2, src_mask, need_weights=False)
        src = src + self.dropout1(src2)
        src2 = self.norm2(src)
        src2 = self.linear2(self.dropout2(self.activation(self.linear1(src2))))
        return src + src2

    def __repr__(self):
        return f"TransformerEncoderLayer(d_model={self.d_model}, nhead={self.nhead})"
