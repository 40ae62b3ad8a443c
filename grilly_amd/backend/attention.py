"""`backend.attention.flash_attention2` (+ fused-RoPE variant and apply_rope) of grilly on
MI355X, numpy in / numpy out, same signature and output layout as the reference
(backend/attention.py:361-597): inputs (B,S,H,D) or (B,S,H*D), output (B,S,H,D) float32.

The result is the attention the reference documents (softmax(scale.QK^T + mask bias).V,
docstring :374-395, CPU forms nn/modules.py:1421-1456); `causal=True` means the usual
lower-triangular rule (keys after the query are excluded, shaders/attention-mask.glsl:42-46).
"""
import numpy as np

from .. import _lib as L
from .core import dtype_code

_ROPE = {None: L.ROPE_NONE, "none": L.ROPE_NONE, "interleaved": L.ROPE_INTERLEAVED, "half": L.ROPE_HALF}


class HipAttention:
    def __init__(self, core, architecture=None):
        self.core = core
        self.architecture = architecture

    def _attn(self, queries, keys, values, num_heads, head_dim, scale, mask, causal, rope, rope_base,
              rope_scaling, dtype, layout):
        code = dtype_code(dtype)
        q, k, v = (np.asarray(t, dtype=np.float32) for t in (queries, keys, values))
        if q.ndim == 3:     # flattened heads: reshaped with the given arguments (attention.py:403-408)
            B, S, _ = q.shape
            q, k, v = (t.reshape(B, S, num_heads, head_dim) for t in (q, k, v))
        elif q.ndim == 4:   # rank-4 input overrides num_heads/head_dim (attention.py:409-410)
            if layout == "bhsd":
                q, k, v = (t.transpose(0, 2, 1, 3) for t in (q, k, v))
            elif layout != "bshd":
                raise ValueError("layout must be 'bshd' or 'bhsd'")
            B, S, num_heads, head_dim = q.shape
        else:
            raise ValueError("queries must be (B,S,H,D) or (B,S,H*D)")
        if k.shape != q.shape or v.shape != q.shape:
            raise ValueError("queries, keys and values must have the same shape")
        if scale is None:
            scale = 1.0 / np.sqrt(head_dim)
        if mask is not None:
            mask = np.asarray(mask, dtype=np.float32)
            if mask.shape != (B, S):
                raise ValueError(f"mask must be (batch, seq_len) = {(B, S)}, got {mask.shape}")
        if rope not in _ROPE:
            raise ValueError("rope_style must be 'interleaved' or 'half'")
        c = self.core
        es = 2 if code == L.GRL_BF16 else 4
        dq, dk, dv = c.upload(q, code), c.upload(k, code), c.upload(v, code)
        dm = c.upload(mask) if mask is not None else None
        do = c.alloc(max(q.size, 1) * es)
        try:
            L.check(c.lib.grl_fa2_fwd(c.ctx, code, B, S, num_heads, head_dim, dq.ptr, dk.ptr, dv.ptr,
                                      dm.ptr if dm else None, do.ptr, float(scale), int(bool(causal)), _ROPE[rope],
                                      float(rope_base), float(rope_scaling), None), "fa2_fwd")
            return c.download(do, (B, S, num_heads, head_dim), code)
        finally:
            for b in (dq, dk, dv, dm, do):
                if b is not None:
                    b.free()

    def attention_with_weights(self, queries, keys, values, scale=None, mask=None):
        """Attention that also returns the softmax weights, for key / value sequences of any length: queries
        (B,Sq,H,D), keys and values (B,Sk,H,D), optional key keep-mask (B,Sk) -> (output (B,Sq,H,D), weights
        (B,H,Sq,Sk)).  What the reference's MultiheadAttention builds from separate score / softmax / output steps
        (nn/modules.py:1131-1216); here: one score GEMM and one output GEMM per (batch, head) on device-resident
        operands, one softmax kernel over all rows, fp32.  The fused kernel (flash_attention2) never forms the
        weights and is the fast path when they are not needed."""
        q, k, v = (np.asarray(t, dtype=np.float32) for t in (queries, keys, values))
        if q.ndim != 4 or k.ndim != 4 or v.shape != k.shape or q.shape[0] != k.shape[0] or q.shape[2:] != k.shape[2:]:
            raise ValueError("expected queries (B,Sq,H,D) and keys / values (B,Sk,H,D)")
        B, Sq, H, D = q.shape
        Sk = k.shape[1]
        if scale is None:
            scale = 1.0 / np.sqrt(D)
        bias = None
        if mask is not None:
            m = np.asarray(mask, dtype=np.float32)
            if m.shape != (B, Sk):
                raise ValueError(f"mask must be (batch, key_len) = {(B, Sk)}, got {m.shape}")
            bias = (m - np.float32(1.0)) * np.float32(1e9)
        if q.size == 0 or Sk == 0:
            return np.zeros((B, Sq, H, D), np.float32), np.zeros((B, H, Sq, Sk), np.float32)
        c, code = self.core, L.GRL_F32
        dq = c.upload(np.ascontiguousarray(q.transpose(0, 2, 1, 3)) * np.float32(scale))      # (B,H,Sq,D)
        dk = c.upload(np.ascontiguousarray(k.transpose(0, 2, 1, 3)))                           # (B,H,Sk,D)
        dvt = c.upload(np.ascontiguousarray(v.transpose(0, 2, 3, 1)))                          # (B,H,D,Sk)
        db = c.upload(bias) if bias is not None else None
        dsc, dw, do = c.alloc(B * H * Sq * Sk * 4), c.alloc(B * H * Sq * Sk * 4), c.alloc(B * H * Sq * D * 4)
        try:
            for bh in range(B * H):
                L.check(c.lib.grl_gemm_nt(c.ctx, code, code, Sq, Sk, D, dq.ptr + bh * Sq * D * 4, dk.ptr + bh * Sk * D * 4,
                                          db.ptr + (bh // H) * Sk * 4 if db else None, dsc.ptr + bh * Sq * Sk * 4, L.EPI_NONE), "scores")
            L.check(c.lib.grl_softmax(c.ctx, code, B * H * Sq, Sk, dsc.ptr, dw.ptr), "softmax")
            for bh in range(B * H):
                L.check(c.lib.grl_gemm_nt(c.ctx, code, code, Sq, D, Sk, dw.ptr + bh * Sq * Sk * 4, dvt.ptr + bh * D * Sk * 4,
                                          None, do.ptr + bh * Sq * D * 4, L.EPI_NONE), "weights x values")
            out = c.download(do, (B, H, Sq, D)).transpose(0, 2, 1, 3)
            return np.ascontiguousarray(out), c.download(dw, (B, H, Sq, Sk))
        finally:
            for t in (dq, dk, dvt, db, dsc, dw, do):
                if t is not None:
                    t.free()

    def flash_attention2(self, queries, keys, values, num_heads, head_dim, tile_size_q=64, tile_size_k=64,
                         scale=None, mask=None, causal=False, dtype="fp32", layout="bshd"):
        """tile_size_q / tile_size_k are accepted for call compatibility; the kernel's tiling is fixed."""
        return self._attn(queries, keys, values, num_heads, head_dim, scale, mask, causal, None, 10000.0, 1.0, dtype, layout)

    def flash_attention2_rope(self, queries, keys, values, num_heads, head_dim, scale=None, mask=None, causal=False,
                              rope_base=10000.0, rope_scaling=1.0, rope_style="interleaved", dtype="fp32", layout="bshd"):
        """Attention on RoPE-rotated Q and K, V unrotated (reference
        shaders/flash-attention2-rope.glsl:73-148, 230-236; interleaved pairs by default, the
        (d, d+D/2) pairing of shaders/rope.glsl with rope_style="half")."""
        return self._attn(queries, keys, values, num_heads, head_dim, scale, mask, causal, rope_style, rope_base,
                          rope_scaling, dtype, layout)

    def apply_rope(self, q_or_k, position_ids=None, rope_base=10000.0, rope_scaling=1.0, rope_style="half", dtype="fp32"):
        """Reference backend/attention.py:599-676 (rotate-half pairs, optional (B,S) position ids)."""
        code = dtype_code(dtype)
        x = np.asarray(q_or_k, dtype=np.float32)
        if x.ndim != 4:
            raise ValueError("apply_rope expects (batch, seq_len, num_heads, head_dim)")
        if rope_style not in ("half", "interleaved"):
            raise ValueError("rope_style must be 'interleaved' or 'half'")
        B, S, H, D = x.shape
        c = self.core
        dx = c.upload(x, code)
        dp = None
        if position_ids is not None:
            pid = np.ascontiguousarray(position_ids, dtype=np.int32)
            if pid.shape != (B, S):
                raise ValueError(f"position_ids must be (batch, seq_len) = {(B, S)}")
            dp = c.upload_raw(pid)
        dy = c.alloc(max(x.size, 1) * (2 if code == L.GRL_BF16 else 4))
        try:
            L.check(c.lib.grl_rope(c.ctx, code, B, S, H, D, dx.ptr, dp.ptr if dp else None, dy.ptr, _ROPE[rope_style],
                                   float(rope_base), float(rope_scaling)), "rope")
            return c.download(dy, x.shape, code)
        finally:
            for b in (dx, dp, dy):
                if b is not None:
                    b.free()
