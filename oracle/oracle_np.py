"""Oracle for grilly's transformer-forward path -- TEST INFRASTRUCTURE, NOT PRODUCT.

Two layers:

* ``truth_*``: the closed forms in float64 numpy.  These are the parity reference
  (y_ref = float64 result rounded to fp32).  Each cites the reference text it restates.
* ``C``: ctypes access to oracle/liboracle.so, the fp32 shader-order restatement in C
  (used for the cross-check truth-vs-shader-order and as the CPU baseline that is timed).

Pinned by tests/test_oracle.py against the reference's own known answers and against
invariants; see the header of oracle.c for the list.  The reference has no numeric test for
flash_attention2, fused linears, fused_swiglu or fused QKV: at the level of the reference's
own tests those are "parity unpinned"; here they are pinned by closed forms and invariants.
"""
import ctypes
import os
import subprocess
import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


# ---------------------------------------------------------------- bf16 helpers
def bf16_round(x):
    """fp32 -> nearest bf16 (ties to even) -> fp32, the storage rounding of the bf16 path."""
    a = np.ascontiguousarray(x, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32).reshape(a.shape)
    return np.where(np.isnan(a), a, out)


def to_bf16_bits(x):
    a = np.ascontiguousarray(x, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return (r & 0xFFFF).astype(np.uint16).reshape(a.shape)


def from_bf16_bits(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------- float64 closed forms
def truth_gelu(x):
    """shaders/activation-gelu.glsl:33-50 / fused-linear-gelu.glsl:45-63 (outer factor unclamped)."""
    x = np.asarray(x, dtype=np.float64)
    c = np.clip(x, -50.0, 50.0)
    r = 0.5 * x * (1.0 + np.tanh(0.7978845608028654 * (c + 0.044715 * c ** 3)))
    return np.where(np.abs(x) > 50.0, np.where(x > 0, x, 0.0), r)


def truth_silu_clamped(x):
    """shaders/fused-linear-silu.glsl:43-48"""
    x = np.asarray(x, dtype=np.float64)
    return x / (1.0 + np.exp(-np.clip(x, -88.0, 88.0)))


def truth_silu(x):
    """x*sigmoid(x): shaders/fused-swiglu.glsl:44-46, backend/fnn.py:344-391"""
    x = np.asarray(x, dtype=np.float64)
    with np.errstate(over="ignore"):
        return x / (1.0 + np.exp(-x))


def truth_linear(x, W, b=None, epi="none", alpha=1.0, beta=1.0):
    """x.W^T + b: shaders/fnn-linear.glsl:42-57; W is (out,in) (backend/fnn.py:1394-1419)."""
    y = np.asarray(x, np.float64) @ np.asarray(W, np.float64).T
    if b is not None:
        y = y + np.asarray(b, np.float64)
    if epi == "gelu":
        y = truth_gelu(y)
    elif epi == "silu":
        y = truth_silu_clamped(y)
    elif epi == "relu":          # shaders/fused-linear-relu.glsl:63
        y = np.maximum(y, 0.0)
    elif epi == "gcu":           # shaders/fused-linear-gcu.glsl:44-46
        y = y * np.cos(y)
    elif epi == "roswish":       # shaders/fused-linear-roswish.glsl:46-58
        y = truth_roswish(y, alpha, beta)
    elif epi != "none":
        raise ValueError(epi)
    return y


def truth_roswish(x, alpha=1.0, beta=1.0):
    """(x+alpha)*sigmoid(beta*x) - alpha/2: shaders/fused-linear-roswish.glsl:46-58"""
    x = np.asarray(x, np.float64)
    with np.errstate(over="ignore"):
        return (x + alpha) / (1.0 + np.exp(-beta * x)) - 0.5 * alpha


def truth_gelu_plain(x):
    """tanh GELU without the clamp rule: shaders/fused-geglu.glsl:44-49"""
    x = np.asarray(x, np.float64)
    return 0.5 * x * (1.0 + np.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))


def truth_fused_glu(x, Wg, Wu, bg=None, bu=None, act="silu"):
    """gate*act(up) for act silu / relu / gelu: shaders/fused-swiglu.glsl:54-78, fused-reglu.glsl:42-75,
    fused-geglu.glsl:43-82; biases only if both given (backend/_glu_append.py:68).  Returns (out, gate, up)."""
    g = np.asarray(x, np.float64) @ np.asarray(Wg, np.float64).T
    u = np.asarray(x, np.float64) @ np.asarray(Wu, np.float64).T
    if bg is not None and bu is not None:
        g = g + np.asarray(bg, np.float64)
        u = u + np.asarray(bu, np.float64)
    a = {"silu": truth_silu, "relu": lambda t: np.maximum(t, 0.0), "gelu": truth_gelu_plain}[act](u)
    return g * a, g, u


def truth_gemm(A, B):
    """A.B: shaders/gemm_mnk.glsl:35-88, backend/fnn.py:104-124"""
    return np.asarray(A, np.float64) @ np.asarray(B, np.float64)


def truth_fused_swiglu(x, Wg, Wu, bg=None, bu=None):
    """gate*silu(up), SiLU on the UP projection: shaders/fused-swiglu.glsl:54-78;
    biases only if both given (backend/_glu_append.py:68).  Returns (out, gate, up)."""
    g = np.asarray(x, np.float64) @ np.asarray(Wg, np.float64).T
    u = np.asarray(x, np.float64) @ np.asarray(Wu, np.float64).T
    if bg is not None and bu is not None:
        g = g + np.asarray(bg, np.float64)
        u = u + np.asarray(bu, np.float64)
    return g * truth_silu(u), g, u


def truth_swiglu_act(x):
    """last dim 2h -> h: x1*silu(x2): shaders/activation-swiglu.glsl:32-51; the reference's own
    test formula x1*x2/(1+exp(-x2)) (tests/test_gpu_operations.py:169-195)."""
    x = np.asarray(x, np.float64)
    h = x.shape[-1] // 2
    return x[..., :h] * truth_silu(x[..., h:])


def truth_layernorm(x, gamma=None, beta=None, eps=1e-5, residual=None):
    """shaders/fnn-layernorm.glsl:44-103: biased variance, eps inside the root."""
    t = np.asarray(x, np.float64)
    if residual is not None:
        t = t + np.asarray(residual, np.float64)
    mu = t.mean(-1, keepdims=True)
    var = ((t - mu) ** 2).mean(-1, keepdims=True)
    y = (t - mu) / np.sqrt(var + eps)
    if gamma is not None:
        y = y * np.asarray(gamma, np.float64)
    if beta is not None:
        y = y + np.asarray(beta, np.float64)
    return y


def rope_angles(S, D, base=10000.0, scaling=1.0, style="interleaved", position_ids=None):
    """theta[pos,p] formed in fp32 in the shaders' operation order, with the power correctly
    rounded: half style (pos/scaling)*freq (shaders/rope.glsl:114-118), interleaved style
    (pos*freq)/scaling (shaders/flash-attention2-rope.glsl:75-78,124-125)."""
    p = np.arange(D // 2, dtype=np.float32)
    fe = (np.float32(-2.0) * p) / np.float32(D)
    freq = np.power(np.float64(base), fe.astype(np.float64)).astype(np.float32)
    pos = (np.arange(S) if position_ids is None else np.asarray(position_ids)).astype(np.float32)
    sc = np.float32(scaling)
    if style == "half":
        th = (pos[..., None] / sc) * freq
    else:
        th = (pos[..., None] * freq) / sc
    return th.astype(np.float32)  # (..., S, D/2)


def truth_rope(x, base=10000.0, scaling=1.0, style="half", position_ids=None):
    """x (B,S,H,D).  half: shaders/rope.glsl:74-125, backend/attention.py:795-835;
    interleaved: shaders/flash-attention2-rope.glsl:84-90,122-137 and
    backend/capsule_transformer.py:775-787."""
    x = np.asarray(x, np.float64)
    B, S, H, D = x.shape
    th = rope_angles(S, D, base, scaling, style, position_ids).astype(np.float64)
    if th.ndim == 2:
        th = np.broadcast_to(th, (B, S, D // 2))
    c = np.cos(th)[:, :, None, :]
    s = np.sin(th)[:, :, None, :]
    y = np.empty_like(x)
    if style == "half":
        a, b = x[..., : D // 2], x[..., D // 2:]
        y[..., : D // 2] = a * c - b * s
        y[..., D // 2:] = b * c + a * s
    else:
        a, b = x[..., 0::2], x[..., 1::2]
        y[..., 0::2] = a * c - b * s
        y[..., 1::2] = a * s + b * c
    return y


def truth_attention(q, k, v, scale=None, mask=None, causal=False, rope=None, base=10000.0, scaling=1.0):
    """softmax(scale*QK^T + (mask-1)*1e9).V, layout (B,S,H,D): backend/attention.py:374-395,
    nn/modules.py:1421-1456, utils/vulkan_sentence_transformer.py:1069-1107.  The mask bias is
    added in fp32 as the shader does (flash-attention2.glsl:150-154): a fully masked row then
    degenerates to the uniform mean.  causal: k>q excluded (attention-mask.glsl:42-46)."""
    q = np.asarray(q, np.float64); k = np.asarray(k, np.float64); v = np.asarray(v, np.float64)
    B, S, H, D = q.shape
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    if rope:
        q = truth_rope(q, base, scaling, rope)
        k = truth_rope(k, base, scaling, rope)
    s = np.einsum("bihd,bjhd->bhij", q, k) * float(np.float32(scale))
    if mask is not None:
        bias = (np.asarray(mask, np.float32) - np.float32(1.0)) * np.float32(1e9)
        s = (s.astype(np.float32) + bias[:, None, None, :]).astype(np.float64)
    if causal:
        s = np.where(np.triu(np.ones((S, S), bool), 1)[None, None], -np.inf, s)
    m = np.maximum(s.max(-1, keepdims=True), -1e10)
    p = np.exp(s - m)
    l = np.maximum(p.sum(-1, keepdims=True), 1e-10)
    return np.einsum("bhij,bjhd->bihd", p / l, v)


def truth_embed(ids, tok, pos, typ):
    """tok[ids] + type[0] + pos[:S]: utils/vulkan_sentence_transformer.py:563-707"""
    ids = np.asarray(ids)
    S = ids.shape[1]
    return np.asarray(tok, np.float64)[ids] + np.asarray(typ, np.float64)[0] + np.asarray(pos, np.float64)[:S][None]


def truth_mean_pool(x, mask=None, l2=True):
    """utils/vulkan_sentence_transformer.py:1177-1201"""
    x = np.asarray(x, np.float64)
    m = np.ones(x.shape[:2]) if mask is None else np.asarray(mask, np.float64)
    out = (x * m[..., None]).sum(1) / np.maximum(m.sum(1, keepdims=True), 1e-9)
    if l2:
        out = out / np.maximum(np.linalg.norm(out, axis=-1, keepdims=True), 1e-12)
    return out


def truth_bert_layer(x, w, mask, H, eps=1e-5, quant=None):
    """utils/vulkan_sentence_transformer.py:972-1035 (post-LN).  ``quant`` (e.g. bf16_round) is
    applied wherever the device path stores an activation, so the bf16 reference sees the same
    storage roundings and only accumulation differences remain."""
    qf = (lambda a: a) if quant is None else (lambda a: quant(np.asarray(a, np.float32)).astype(np.float64))
    x = np.asarray(x, np.float64)
    B, S, d = x.shape
    D = d // H
    qkv = qf(truth_linear(x, w["w_qkv"], w["b_qkv"]))
    q, k, v = (qkv[..., i * d:(i + 1) * d].reshape(B, S, H, D) for i in range(3))
    a = qf(truth_attention(q, k, v, mask=mask)).reshape(B, S, d)
    proj = qf(truth_linear(a, w["w_o"], w["b_o"]))
    x1 = qf(truth_layernorm(x, w["ln1_g"], w["ln1_b"], eps, residual=proj))
    ff = qf(truth_linear(x1, w["w_ff1"], w["b_ff1"], "gelu"))
    ff2 = qf(truth_linear(ff, w["w_ff2"], w["b_ff2"]))
    return qf(truth_layernorm(x1, w["ln2_g"], w["ln2_b"], eps, residual=ff2))


def truth_prenorm_geglu_layer(x, w, mask, H, eps=1e-5, rope_base=10000.0, rope_scaling=1.0, quant=None):
    """Pre-norm layer with rotary positions and a GeGLU MLP, utils/vulkan_sentence_transformer.py:799-970:
    x += Wo.Attn(rope(Wq x), rope(Wk x), Wv x; key mask) (:806-893, no norm in front of the attention:
    the reference skips attn_norm in every layer); x += W2.(gelu(Wi_in.LN(x)) * (Wi_gate.LN(x))) (:901-945),
    rotate-half RoPE on positions 0..S-1 (:829-846, backend/attention.py:795-835), tanh GELU (:933).
    The +-50 / +-1e6 clips of :924-930 are left out (no effect below those magnitudes)."""
    qf = (lambda a: a) if quant is None else (lambda a: quant(np.asarray(a, np.float32)).astype(np.float64))
    x = np.asarray(x, np.float64)
    B, S, d = x.shape
    D = d // H
    q, k, v = (qf(truth_linear(x, w["w_qkv"][i * d:(i + 1) * d], w["b_qkv"][i * d:(i + 1) * d])).reshape(B, S, H, D)
               for i in range(3))
    a = qf(truth_attention(q, k, v, mask=mask, rope="half", base=rope_base, scaling=rope_scaling)).reshape(B, S, d)
    x = qf(x + qf(truth_linear(a, w["w_o"], w["b_o"])))
    xn = qf(truth_layernorm(x, w["ffn_ln_g"], w["ffn_ln_b"], eps))
    # truth_fused_glu activates its "up" operand: that is the first half of Wi here
    h = qf(truth_fused_glu(xn, w["w_ff_gate"], w["w_ff_in"], w["b_ff_gate"], w["b_ff_in"], act="gelu")[0])
    return qf(x + qf(truth_linear(h, w["w_ff2"], w["b_ff2"])))


# ---------------------------------------------------------------- error metrics
def max_rel(y, ref):
    """max|y-ref| / max|ref|: the scale-relative error the tolerances (1e-4 fp32, 2e-2 bf16) use."""
    ref = np.asarray(ref, np.float64)
    den = np.max(np.abs(ref))
    num = np.max(np.abs(np.asarray(y, np.float64) - ref)) if ref.size else 0.0
    return float(num / den) if den > 0 else float(num)


# ---------------------------------------------------------------- C oracle (shader order, fp32)
def build(force=False):
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "oracle.c")):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_F = ctypes.POINTER(ctypes.c_float)
_I = ctypes.POINTER(ctypes.c_int32)


def _fp(a):
    return None if a is None else a.ctypes.data_as(_F)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


class COracle:
    """fp32 shader-order restatement (oracle.c) behind numpy-in / numpy-out helpers."""

    def __init__(self):
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError("oracle/liboracle.so is not built; run `make -C oracle` (or __graft_entry__.build())")
        self.lib = ctypes.CDLL(_LIB_PATH)
        L, i64, f, ci = self.lib, ctypes.c_int64, ctypes.c_float, ctypes.c_int
        L.orc_linear.argtypes = [_F, _F, _F, _F, i64, i64, i64, ci]
        L.orc_linear_act.argtypes = [_F, _F, _F, _F, i64, i64, i64, ci, f, f]
        L.orc_fused_glu.argtypes = [_F, _F, _F, _F, _F, _F, _F, _F, i64, i64, i64, ci]
        L.orc_gemm_nn.argtypes = [_F, _F, _F, i64, i64, i64]
        L.orc_fused_swiglu.argtypes = [_F, _F, _F, _F, _F, _F, _F, _F, i64, i64, i64]
        L.orc_layernorm.argtypes = [_F, _F, _F, _F, _F, i64, i64, f]
        L.orc_residual.argtypes = [_F, _F, _F, i64]
        L.orc_gelu.argtypes = [_F, _F, i64]
        L.orc_silu.argtypes = [_F, _F, i64]
        L.orc_swiglu_act.argtypes = [_F, _F, i64, i64]
        L.orc_rope.argtypes = [_F, _I, _F, i64, i64, i64, i64, ci, f, f]
        L.orc_attention.argtypes = [_F, _F, _F, _F, _F, i64, i64, i64, i64, f, ci, ci, f, f]
        L.orc_embed.argtypes = [_I, _F, _F, _F, _F, i64, i64, i64]
        L.orc_mean_pool.argtypes = [_F, _F, _F, i64, i64, i64, ci]
        L.orc_bert_layer.argtypes = [_F, _F, i64, i64, i64, i64, i64] + [_F] * 12 + [f, _F]
        L.orc_num_threads.restype = ci
        for n in ("orc_linear", "orc_linear_act", "orc_fused_glu", "orc_gemm_nn", "orc_fused_swiglu", "orc_layernorm", "orc_residual", "orc_gelu",
                  "orc_silu", "orc_swiglu_act", "orc_rope", "orc_attention", "orc_embed", "orc_mean_pool", "orc_bert_layer"):
            getattr(L, n).restype = None

    def num_threads(self):
        return int(self.lib.orc_num_threads())

    def linear(self, x, W, b=None, epi="none", alpha=1.0, beta=1.0):
        x, W, b = _f32(x), _f32(W), _f32(b)
        M, K = x.shape; N = W.shape[0]
        y = np.empty((M, N), np.float32)
        code = {"none": 0, "gelu": 1, "silu": 2, "relu": 3, "gcu": 4, "roswish": 5}[epi]
        self.lib.orc_linear_act(_fp(x), _fp(W), _fp(b), _fp(y), M, K, N, code, alpha, beta)
        return y

    def fused_glu(self, x, Wg, Wu, bg=None, bu=None, act="silu"):
        x, Wg, Wu, bg, bu = _f32(x), _f32(Wg), _f32(Wu), _f32(bg), _f32(bu)
        M, K = x.shape; N = Wg.shape[0]
        out, g, u = (np.empty((M, N), np.float32) for _ in range(3))
        self.lib.orc_fused_glu(_fp(x), _fp(Wg), _fp(Wu), _fp(bg), _fp(bu), _fp(out), _fp(g), _fp(u), M, K, N,
                               {"silu": 2, "relu": 3, "gelu": 1}[act])
        return out, g, u

    def gemm(self, A, B):
        A, B = _f32(A), _f32(B)
        M, K = A.shape; N = B.shape[1]
        C = np.empty((M, N), np.float32)
        self.lib.orc_gemm_nn(_fp(A), _fp(B), _fp(C), M, K, N)
        return C

    def fused_swiglu(self, x, Wg, Wu, bg=None, bu=None):
        x, Wg, Wu, bg, bu = _f32(x), _f32(Wg), _f32(Wu), _f32(bg), _f32(bu)
        M, K = x.shape; N = Wg.shape[0]
        out, g, u = (np.empty((M, N), np.float32) for _ in range(3))
        self.lib.orc_fused_swiglu(_fp(x), _fp(Wg), _fp(Wu), _fp(bg), _fp(bu), _fp(out), _fp(g), _fp(u), M, K, N)
        return out, g, u

    def layernorm(self, x, gamma, beta, eps=1e-5, residual=None):
        x, r = _f32(x), _f32(residual)
        F = x.shape[-1]
        y = np.empty_like(x)
        self.lib.orc_layernorm(_fp(x), _fp(r), _fp(_f32(gamma)), _fp(_f32(beta)), _fp(y), x.size // F, F, eps)
        return y

    def residual(self, a, b):
        a, b = _f32(a), _f32(b)
        o = np.empty_like(a)
        self.lib.orc_residual(_fp(a), _fp(b), _fp(o), a.size)
        return o

    def gelu(self, x):
        x = _f32(x); y = np.empty_like(x)
        self.lib.orc_gelu(_fp(x), _fp(y), x.size)
        return y

    def silu(self, x):
        x = _f32(x); y = np.empty_like(x)
        self.lib.orc_silu(_fp(x), _fp(y), x.size)
        return y

    def swiglu_act(self, x):
        x = _f32(x)
        h = x.shape[-1] // 2
        y = np.empty(x.shape[:-1] + (h,), np.float32)
        self.lib.orc_swiglu_act(_fp(x), _fp(y), x.size // (2 * h), h)
        return y

    def rope(self, x, style="half", base=10000.0, scaling=1.0, position_ids=None):
        x = _f32(x)
        B, S, H, D = x.shape
        y = np.empty_like(x)
        pid = None if position_ids is None else np.ascontiguousarray(position_ids, np.int32)
        self.lib.orc_rope(_fp(x), None if pid is None else pid.ctypes.data_as(_I), _fp(y), B, S, H, D,
                          2 if style == "half" else 1, base, scaling)
        return y

    def attention(self, q, k, v, scale=None, mask=None, causal=False, rope=None, base=10000.0, scaling=1.0):
        q, k, v, mask = _f32(q), _f32(k), _f32(v), _f32(mask)
        B, S, H, D = q.shape
        if scale is None:
            scale = 1.0 / np.sqrt(D)
        o = np.empty_like(q)
        self.lib.orc_attention(_fp(q), _fp(k), _fp(v), _fp(mask), _fp(o), B, S, H, D, float(scale), int(bool(causal)),
                               {None: 0, "interleaved": 1, "half": 2}[rope], base, scaling)
        return o

    def embed(self, ids, tok, pos, typ):
        ids = np.ascontiguousarray(ids, np.int32)
        tok, pos, typ = _f32(tok), _f32(pos), _f32(typ)
        B, S = ids.shape; F = tok.shape[1]
        x = np.empty((B, S, F), np.float32)
        self.lib.orc_embed(ids.ctypes.data_as(_I), _fp(tok), _fp(pos), _fp(typ), _fp(x), B, S, F)
        return x

    def mean_pool(self, x, mask=None, l2=True):
        x, mask = _f32(x), _f32(mask)
        B, S, F = x.shape
        o = np.empty((B, F), np.float32)
        self.lib.orc_mean_pool(_fp(x), _fp(mask), _fp(o), B, S, F, int(l2))
        return o

    def bert_layer(self, x, w, mask, H, eps=1e-5):
        x = _f32(x).copy()
        B, S, d = x.shape
        dff = w["w_ff1"].shape[0]
        ws = [_f32(w[k]) for k in ("w_qkv", "b_qkv", "w_o", "b_o", "ln1_g", "ln1_b", "w_ff1", "b_ff1", "w_ff2", "b_ff2", "ln2_g", "ln2_b")]
        scratch = np.empty(B * S * (3 * d + 2 * d + dff), np.float32)
        self.lib.orc_bert_layer(_fp(x), _fp(_f32(mask)), B, S, H, d // H, dff, *[_fp(a) for a in ws], eps, _fp(scratch))
        return x
