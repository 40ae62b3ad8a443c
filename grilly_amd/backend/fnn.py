"""`backend.fnn.*` of grilly on MI355X: same method names, positional order, defaults, output
shapes and float32 results as VulkanFNN (reference backend/fnn.py), numpy in / numpy out.

Every method copies its inputs to the device, runs hand-written gfx950 kernels through the C
ABI, and copies the result back; inputs are never modified.  Extra keyword `dtype` ("fp32" or
"bf16") selects the storage type of activations and weights on the device (accumulation is
always fp32; results come back as float32).  There is no CPU path: a missing library or
device raises.
"""
import numpy as np

from .. import _lib as L
from .core import dtype_code


class _PoolView:
    """`backend.fnn.buffer_pool.get_stats()` of the reference (backend/buffer_pool.py:627-640)."""

    def __init__(self, core):
        self._core = core

    def get_stats(self):
        return self._core.pool_stats()


def _as2d(x, K):
    x = np.asarray(x)
    if x.ndim == 0:
        raise ValueError("input must have at least one dimension")
    if x.shape[-1] != K:
        raise ValueError(f"last dimension of x ({x.shape[-1]}) does not match in_features ({K})")
    return x.reshape(-1, K)


class HipFNN:
    def __init__(self, core):
        self.core = core
        self.buffer_pool = _PoolView(core)

    def get_buffer_pool_stats(self):
        """backend/fnn.py:90-102"""
        return self.core.pool_stats()

    # ------------------------------------------------------------------ GEMM family
    def fused_linear_residual(self, x, weights, bias, residual, dtype="fp32"):
        """residual + x.W^T + b in one kernel: the reference's linear followed by residual
        (backend/fnn.py:1394-1496 then :1950-2014), as its encoder recipes chain them.  Not a method of the
        reference's VulkanFNN; same shape rules as linear, residual shaped like the result."""
        code = dtype_code(dtype)
        x = np.asarray(x)
        W = np.asarray(weights)
        if W.ndim != 2:
            raise ValueError("weights must be (out_features, in_features)")
        N, K = W.shape
        x2 = _as2d(x, K)
        M = x2.shape[0]
        r = np.asarray(residual)
        if r.size != M * N:
            raise ValueError(f"residual has {r.size} elements, expected {M * N}")
        if bias is not None and np.asarray(bias).size != N:
            raise ValueError(f"bias has {np.asarray(bias).size} elements, expected {N}")
        c = self.core
        dx, dw, dr = c.upload(x2, code), c.upload(W, code), c.upload(r.reshape(M, N), code)
        db = c.upload(np.asarray(bias).reshape(-1)) if bias is not None else None
        try:
            L.check(c.lib.grl_gemm_nt_res(c.ctx, code, code, M, N, K, dx.ptr, dw.ptr, db.ptr if db else None, dr.ptr,
                                          dr.ptr), "gemm_nt_res")          # in place on the residual buffer
            return c.download(dr, (M, N), code).reshape(r.shape)
        finally:
            for b in (dx, dw, db, dr):
                if b is not None:
                    b.free()

    def _linear_impl(self, x, weights, bias, epi, dtype, alpha=1.0, beta=1.0):
        code = dtype_code(dtype)
        W = np.asarray(weights)
        if W.ndim != 2:
            raise ValueError("weights must be (out_features, in_features)")
        N, K = W.shape
        x2 = _as2d(x, K)
        M = x2.shape[0]
        if bias is not None and np.asarray(bias).size != N:
            raise ValueError(f"bias has {np.asarray(bias).size} elements, expected {N}")
        c = self.core
        dx, dw = c.upload(x2, code), c.upload(W, code)
        db = c.upload(np.asarray(bias).reshape(-1)) if bias is not None else None
        dy = c.alloc(M * N * (2 if code == L.GRL_BF16 else 4))
        try:
            L.check(c.lib.grl_gemm_nt_act(c.ctx, code, code, M, N, K, dx.ptr, dw.ptr, db.ptr if db else None, dy.ptr, epi,
                                          float(alpha), float(beta)), "gemm_nt")
            return c.download(dy, (M, N), code)
        finally:
            for b in (dx, dw, db, dy):
                if b is not None:
                    b.free()

    def linear(self, x, weights, bias=None, dtype="fp32"):
        """y = x.W^T + b (reference backend/fnn.py:1394-1496).  Leading dimensions of x are kept
        (:1421-1427, :1491-1496)."""
        x = np.asarray(x)
        y = self._linear_impl(x, weights, bias, L.EPI_NONE, dtype)
        N = y.shape[1]
        if x.ndim > 2:
            return y.reshape(x.shape[:-1] + (N,))
        if x.ndim == 1:
            return y.reshape(N)
        return y

    def _fused_shape(self, x, y):
        # rank-1 input is one row and comes back as (1,N): backend/fnn.py:2055-2060, 2119-2123
        if x.ndim > 2:
            return y.reshape(x.shape[:-1] + (y.shape[1],))
        return y

    def fused_linear_gelu(self, x, weights, bias=None, dtype="fp32"):
        """GELU_tanh(x.W^T + b) in one kernel (reference backend/fnn.py:2022-2123)."""
        x = np.asarray(x)
        return self._fused_shape(x, self._linear_impl(x, weights, bias, L.EPI_GELU, dtype))

    def fused_linear_silu(self, x, weights, bias=None, dtype="fp32"):
        """SiLU(x.W^T + b) in one kernel (reference backend/fnn.py:2214-2303)."""
        x = np.asarray(x)
        return self._fused_shape(x, self._linear_impl(x, weights, bias, L.EPI_SILU, dtype))

    def fused_linear_relu(self, x, weights, bias=None, dtype="fp32"):
        """ReLU(x.W^T + b) in one kernel (reference backend/fnn.py:2125-2212)."""
        x = np.asarray(x)
        return self._fused_shape(x, self._linear_impl(x, weights, bias, L.EPI_RELU, dtype))

    def fused_linear_gcu(self, x, weights, bias=None, dtype="fp32"):
        """GCU(s) = s*cos(s) on s = x.W^T + b in one kernel (reference backend/fnn.py:2307-2383)."""
        x = np.asarray(x)
        return self._fused_shape(x, self._linear_impl(x, weights, bias, L.EPI_GCU, dtype))

    def fused_linear_roswish(self, x, weights, bias=None, alpha=1.0, beta=1.0, dtype="fp32"):
        """RoSwish(s) = (s+alpha)*sigmoid(beta*s) - alpha/2 on s = x.W^T + b in one kernel
        (reference backend/fnn.py:2385-2470)."""
        x = np.asarray(x)
        return self._fused_shape(x, self._linear_impl(x, weights, bias, L.EPI_ROSWISH, dtype, alpha, beta))

    def fused_layernorm_linear(self, x, gamma, beta, weights, bias=None, eps=1e-5, dtype="fp32"):
        """Linear(LayerNorm(x)) (reference shaders/fused-layernorm-linear.glsl:67-128; the reference has no host
        wrapper for it).  The normalised rows are never formed: gamma is folded into the weight, beta into the bias
        (grl_ln_fold, once per call here, once per model in the encoder classes), one pass over x leaves
        {rstd, rstd*mean} per row, and the GEMM on the raw rows applies them in its epilogue."""
        code = dtype_code(dtype)
        W = np.asarray(weights)
        if W.ndim != 2:
            raise ValueError("weights must be (out_features, in_features)")
        N, K = W.shape
        x = np.asarray(x)
        x2 = _as2d(x, K)
        M = x2.shape[0]
        g, bt = np.asarray(gamma, np.float32).reshape(-1), np.asarray(beta, np.float32).reshape(-1)
        if g.size != K or bt.size != K:
            raise ValueError("gamma/beta must have `in_features` elements")
        if bias is not None and np.asarray(bias).size != N:
            raise ValueError(f"bias has {np.asarray(bias).size} elements, expected {N}")
        c = self.core
        es = 2 if code == L.GRL_BF16 else 4
        if M == 0 or N == 0 or K == 0:
            return self._fused_shape(x, np.zeros((M, N), np.float32))
        dx, dw, dg, dbt = c.upload(x2, code), c.upload(W, code), c.upload(g), c.upload(bt)
        db = c.upload(np.asarray(bias, np.float32).reshape(-1)) if bias is not None else None
        dws, dcs, dbf = c.alloc(N * K * es), c.alloc(N * 4), c.alloc(N * 4)
        dst, dy = c.alloc(M * 8), c.alloc(M * N * es)
        try:
            L.check(c.lib.grl_ln_fold(c.ctx, code, N, K, dw.ptr, dg.ptr, dbt.ptr, db.ptr if db else None, dws.ptr, dcs.ptr, dbf.ptr), "ln_fold")
            L.check(c.lib.grl_ln_gemm_nt(c.ctx, code, code, M, N, K, dx.ptr, dws.ptr, dcs.ptr, dbf.ptr, float(eps), dst.ptr, dy.ptr), "ln_gemm_nt")
            return self._fused_shape(x, c.download(dy, (M, N), code))
        finally:
            for t in (dx, dw, dg, dbt, db, dws, dcs, dbf, dst, dy):
                if t is not None:
                    t.free()

    def fused_qkv_projection(self, x, W_qkv, b_qkv=None, num_heads=None, head_dim=None, dtype="fp32"):
        """QKV = x.[Wq;Wk;Wv]^T + [bq;bk;bv] -> (..., 3*H*D); Q is columns [0,H*D), K the next
        H*D, V the last (reference shaders/fused-qkv-projection.glsl:48-74; the reference has no
        host wrapper for this shader)."""
        W = np.asarray(W_qkv)
        if num_heads is not None and head_dim is not None and W.shape[0] != 3 * num_heads * head_dim:
            raise ValueError(f"W_qkv has {W.shape[0]} rows, expected 3*num_heads*head_dim = {3 * num_heads * head_dim}")
        if W.shape[0] % 3:
            raise ValueError("W_qkv must stack Wq, Wk, Wv row-wise")
        return self.linear(x, W, b_qkv, dtype=dtype)

    def gemm(self, A, B, dtype="fp32"):
        """C = A.B, A (M,K), B (K,N) (reference backend/fnn.py:104-166).  When B is a transposed
        view of a C-contiguous (N,K) array -- how nn.Linear calls it with W.T
        (nn/modules.py:153-160) -- the weight is used in place; otherwise B is transposed once on
        the device."""
        code = dtype_code(dtype)
        A = np.asarray(A); B = np.asarray(B)
        if A.ndim != 2 or B.ndim != 2:
            raise ValueError("gemm expects 2-D operands")
        M, K = A.shape
        K2, N = B.shape
        assert K == K2      # the reference's own check (backend/fnn.py:118)
        if B.T.flags.c_contiguous and not B.flags.c_contiguous:
            return self._linear_impl(A, B.T, None, L.EPI_NONE, dtype)
        c = self.core
        da, db = c.upload(A, code), c.upload(B, code)
        dc = c.alloc(M * N * (2 if code == L.GRL_BF16 else 4))
        try:
            L.check(c.lib.grl_gemm_nn(c.ctx, code, code, M, N, K, da.ptr, db.ptr, dc.ptr, None), "gemm_nn")
            return c.download(dc, (M, N), code)
        finally:
            for b in (da, db, dc):
                b.free()

    def fused_swiglu(self, x, W_gate, W_up, b_gate=None, b_up=None, return_cache=False, dtype="fp32"):
        """(x.Wg^T + bg) * SiLU(x.Wu^T + bu), output always 2-D (M, hidden)
        (reference backend/_glu_append.py:8-129; SiLU is on the UP projection,
        shaders/fused-swiglu.glsl:76-78; biases only when both are given, :68)."""
        return self._glu_impl(x, W_gate, W_up, b_gate, b_up, return_cache, dtype, L.EPI_SILU)

    def fused_reglu(self, x, W_gate, W_up, b_gate=None, b_up=None, return_cache=False, dtype="fp32"):
        """(x.Wg^T + bg) * ReLU(x.Wu^T + bu) (reference backend/_glu_append.py:131-222, shaders/fused-reglu.glsl:42-75)."""
        return self._glu_impl(x, W_gate, W_up, b_gate, b_up, return_cache, dtype, L.EPI_RELU)

    def fused_geglu(self, x, W_gate, W_up, b_gate=None, b_up=None, return_cache=False, dtype="fp32"):
        """(x.Wg^T + bg) * GELU_tanh(x.Wu^T + bu) (reference backend/_glu_append.py:224-315, shaders/fused-geglu.glsl:43-82)."""
        return self._glu_impl(x, W_gate, W_up, b_gate, b_up, return_cache, dtype, L.EPI_GELU)

    def _glu_impl(self, x, W_gate, W_up, b_gate, b_up, return_cache, dtype, act):
        code = dtype_code(dtype)
        Wg, Wu = np.asarray(W_gate), np.asarray(W_up)
        if Wg.shape != Wu.shape or Wg.ndim != 2:
            raise ValueError("W_gate and W_up must both be (hidden_dim, input_dim)")
        N, K = Wg.shape
        x2 = _as2d(x, K)
        M = x2.shape[0]
        c = self.core
        es = 2 if code == L.GRL_BF16 else 4
        dx, dg, du = c.upload(x2, code), c.upload(Wg, code), c.upload(Wu, code)
        both = b_gate is not None and b_up is not None
        dbg = c.upload(np.asarray(b_gate).reshape(-1)) if both else None
        dbu = c.upload(np.asarray(b_up).reshape(-1)) if both else None
        dy = c.alloc(M * N * es)
        cg = c.alloc(M * N * 4) if return_cache else None
        cu = c.alloc(M * N * 4) if return_cache else None
        try:
            L.check(c.lib.grl_glu_nt(c.ctx, code, code, M, N, K, dx.ptr, dg.ptr, du.ptr,
                                     dbg.ptr if dbg else None, dbu.ptr if dbu else None, dy.ptr,
                                     cg.ptr if cg else None, cu.ptr if cu else None, act), "glu_nt")
            out = c.download(dy, (M, N), code)
            if return_cache:
                return out, c.download(cg, (M, N)), c.download(cu, (M, N))
            return out
        finally:
            for b in (dx, dg, du, dbg, dbu, dy, cg, cu):
                if b is not None:
                    b.free()

    # ------------------------------------------------------------------ row / element kernels
    def layernorm(self, x, gamma=None, beta=None, eps=1e-5, dtype="fp32"):
        """Reference backend/fnn.py:1285-1389: ranks 1..3, normalises the last dimension."""
        code = dtype_code(dtype)
        x = np.asarray(x)
        if x.ndim < 1 or x.ndim > 3:
            raise ValueError("layernorm accepts (features,), (batch, features) or (batch, seq, features)")
        F = x.shape[-1]
        g = np.ones(F, np.float32) if gamma is None else np.asarray(gamma, np.float32).reshape(-1)
        b = np.zeros(F, np.float32) if beta is None else np.asarray(beta, np.float32).reshape(-1)
        if g.size != F or b.size != F:
            raise ValueError("gamma/beta must have `features` elements")
        rows = x.size // F if F else 0
        c = self.core
        dx, dg, db = c.upload(x, code), c.upload(g), c.upload(b)
        dy = c.alloc(max(x.size, 1) * (2 if code == L.GRL_BF16 else 4))
        try:
            L.check(c.lib.grl_layernorm(c.ctx, code, rows, F, dx.ptr, None, dg.ptr, db.ptr, float(eps), dy.ptr), "layernorm")
            return c.download(dy, x.shape, code)
        finally:
            for t in (dx, dg, db, dy):
                t.free()

    def _unary(self, fn, x, dtype, what, *params):
        code = dtype_code(dtype)
        x = np.asarray(x)
        c = self.core
        dx = c.upload(x, code)
        dy = c.alloc(max(x.size, 1) * (2 if code == L.GRL_BF16 else 4))
        try:
            L.check(fn(c.ctx, code, x.size, dx.ptr, dy.ptr, *params), what)
            return c.download(dy, x.shape, code)
        finally:
            dx.free(); dy.free()

    def residual(self, x, module_output, dtype="fp32"):
        """x + module_output (reference backend/fnn.py:1950-2014)."""
        code = dtype_code(dtype)
        x = np.asarray(x); m = np.asarray(module_output)
        if x.size != m.size:
            raise ValueError("residual operands must have the same number of elements")
        c = self.core
        da, db = c.upload(x, code), c.upload(m, code)
        dy = c.alloc(max(x.size, 1) * (2 if code == L.GRL_BF16 else 4))
        try:
            L.check(c.lib.grl_add(c.ctx, code, x.size, da.ptr, db.ptr, dy.ptr), "add")
            return c.download(dy, x.shape, code)
        finally:
            da.free(); db.free(); dy.free()

    # the activations take the reference's argument name `input_data` (backend/fnn.py:232, 285, 344, 393, 442, 499, 574)
    def activation_gelu(self, input_data, dtype="fp32"):
        """Reference backend/fnn.py:285-342 (tanh form with the +-50 rule)."""
        return self._unary(self.core.lib.grl_gelu, input_data, dtype, "gelu")

    def activation_silu(self, input_data, dtype="fp32"):
        """Reference backend/fnn.py:344-391."""
        return self._unary(self.core.lib.grl_silu, input_data, dtype, "silu")

    def activation_relu(self, input_data, dtype="fp32"):
        """Reference backend/fnn.py:232-283."""
        return self._unary(self.core.lib.grl_relu, input_data, dtype, "relu")

    def activation_gcu(self, input_data, dtype="fp32"):
        """x*cos(x) (reference backend/fnn.py:393-440)."""
        return self._unary(self.core.lib.grl_gcu, input_data, dtype, "gcu")

    def activation_roswish(self, input_data, alpha=1.0, beta=1.0, dtype="fp32"):
        """(x+alpha)*sigmoid(beta*x) - alpha/2 (reference backend/fnn.py:442-497)."""
        return self._unary(self.core.lib.grl_roswish, input_data, dtype, "roswish", float(alpha), float(beta))

    def activation_softmax(self, input_data, axis=-1, dtype="fp32"):
        """exp(x - max) / sum over `axis` (reference backend/fnn.py:574-700; its shader normalises the last
        dimension, other axes are moved there and back)."""
        code = dtype_code(dtype)
        x = np.asarray(input_data, dtype=np.float32)
        if x.ndim == 0:
            raise ValueError("activation_softmax needs at least one dimension")
        xm = np.moveaxis(x, axis, -1)
        F = xm.shape[-1]
        if F == 0:
            return np.empty(x.shape, np.float32)
        rows = xm.size // F
        c = self.core
        dx = c.upload(xm, code)
        dy = c.alloc(max(xm.size, 1) * (2 if code == L.GRL_BF16 else 4))
        try:
            L.check(c.lib.grl_softmax(c.ctx, code, rows, F, dx.ptr, dy.ptr), "softmax")
            return np.ascontiguousarray(np.moveaxis(c.download(dy, xm.shape, code), -1, axis))
        finally:
            dx.free(); dy.free()

    def activation_swiglu(self, input_data, dtype="fp32"):
        """Last dim 2h -> h: x1 * silu(x2) (reference backend/fnn.py:499-572); any rank >= 1."""
        code = dtype_code(dtype)
        x = np.asarray(input_data)
        if x.ndim < 1 or x.shape[-1] % 2:
            raise ValueError("activation_swiglu needs an even last dimension")
        h = x.shape[-1] // 2
        rows = x.size // (2 * h) if h else 0
        c = self.core
        dx = c.upload(x, code)
        dy = c.alloc(max(rows * h, 1) * (2 if code == L.GRL_BF16 else 4))
        try:
            L.check(c.lib.grl_swiglu_act(c.ctx, code, rows, h, dx.ptr, dy.ptr), "swiglu_act")
            return c.download(dy, x.shape[:-1] + (h,), code)
        finally:
            dx.free(); dy.free()
