"""`backend.learning.embedding_lookup` and `backend.pooling.mean_pool` of grilly on MI355X, numpy in / numpy out:
the two encoder steps either side of the layer stack (reference backend/learning.py:811-877 with
shaders/embedding-lookup.glsl:28-56, and backend/pooling.py:22-143 with shaders/embedding-pool.glsl:28-80).
The device-resident encoders call the same kernels (grl_embed / grl_mean_pool) without leaving HBM.
"""
import numpy as np

from .. import _lib as L


class HipLearning:
    """The embedding part of the reference's VulkanLearning namespace."""

    def __init__(self, core):
        self.core = core

    def embedding_lookup(self, token_ids, embedding_table):
        """token_ids (batch, seq_len) or (seq_len,), embedding_table (vocab, dim) -> float32 (batch, seq_len, dim).
        A 1-D id vector is one batch entry (learning.py:826-827).  The reference casts the ids to uint32 and its
        shader writes a zero row for any id >= vocab (embedding-lookup.glsl:38-46); negative ids wrap to large
        unsigned values, so they give zero rows too."""
        ids = np.asarray(token_ids)
        if ids.ndim == 1:
            ids = ids.reshape(1, -1)
        if ids.ndim != 2:
            raise ValueError("token_ids must be (batch, seq_len) or (seq_len,)")
        table = np.asarray(embedding_table, dtype=np.float32)
        if table.ndim != 2:
            raise ValueError("embedding_table must be (vocab_size, embedding_dim)")
        B, S = ids.shape
        V, F = table.shape
        out = np.zeros((B, S, F), np.float32)
        if out.size == 0 or V == 0:
            return out
        ids = ids.astype(np.int64)
        # one more table row of zeros stands for every id outside [0, vocab)
        ids32 = np.where((ids < 0) | (ids >= V), V, ids).astype(np.int32)
        c = self.core
        dt = c.alloc((V + 1) * F * 4)
        di = c.upload_raw(ids32)
        do = c.alloc(B * S * F * 4)
        try:
            tab = np.ascontiguousarray(table)
            L.check(c.lib.grl_h2d(c.ctx, dt.ptr, tab.ctypes.data, tab.nbytes), "upload table")
            L.check(c.lib.grl_memset(c.ctx, dt.ptr + V * F * 4, 0, F * 4), "zero row")
            L.check(c.lib.grl_embed(c.ctx, L.GRL_F32, B, S, F, V + 1, di.ptr, dt.ptr, None, None, do.ptr), "embed")
            return c.download(do, (B, S, F))
        finally:
            for b in (dt, di, do):
                b.free()


class HipPooling:
    """The sequence-pooling part of the reference's VulkanPooling namespace."""

    def __init__(self, core):
        self.core = core

    def mean_pool(self, embeddings, mask=None):
        """embeddings (batch, seq_len, dim), optional mask (batch, seq_len) -> float32 (batch, dim): the mean over
        the positions whose mask value exceeds 0.5, zeros for a sequence with none (embedding-pool.glsl:61-80: the
        mask is a threshold, not a weight); without a mask the plain mean over seq_len (pooling.py:98-143)."""
        x = np.asarray(embeddings, dtype=np.float32)
        if x.ndim != 3:
            raise ValueError("embeddings must be (batch, seq_len, dim)")
        B, S, F = x.shape
        if mask is not None:
            m = np.asarray(mask, dtype=np.float32)
            if m.shape != (B, S):
                raise ValueError(f"mask must be (batch, seq_len) = {(B, S)}, got {m.shape}")
            keep = (m > 0.5).astype(np.float32)
        else:
            keep = None
        if B == 0 or F == 0:
            return np.zeros((B, F), np.float32)
        if S == 0:
            return np.zeros((B, F), np.float32) if mask is not None else np.full((B, F), np.nan, np.float32)
        c = self.core
        dx = c.upload(x)
        dm = c.upload(keep) if keep is not None else None
        do = c.alloc(B * F * 4)
        try:
            L.check(c.lib.grl_mean_pool(c.ctx, L.GRL_F32, B, S, F, dx.ptr, dm.ptr if dm else None, do.ptr, 0), "mean_pool")
            return c.download(do, (B, F))
        finally:
            for b in (dx, dm, do):
                if b is not None:
                    b.free()
