"""Device-resident BERT-style (post-LN) encoder forward built from the hot-path kernels.

Mirrors the forward recipe of the reference's VulkanSentenceTransformer
(utils/vulkan_sentence_transformer.py): embeddings = token + token-type 0 + position, then
LayerNorm (:563-747); per layer the post-LN block of _forward_layer (:972-1035) with the
Q/K/V projections fused into one packed weight; masked mean pooling and L2 normalisation
(:1177-1201).  Weights and activations live in HBM for the whole forward; only token ids and
the attention mask go in and the pooled embeddings (or the hidden states) come out.
"""
import ctypes
from dataclasses import dataclass

import numpy as np

from . import _lib as L
from .backend.core import HipCore, dtype_code


@dataclass
class EncoderConfig:
    layers: int = 12
    d_model: int = 768
    heads: int = 12
    d_ff: int = 3072
    vocab: int = 30522
    max_pos: int = 512
    eps: float = 1e-5          # the reference hard-codes 1e-5 in the layer LayerNorms (:1004, :1026)

    @property
    def head_dim(self):
        return self.d_model // self.heads


BERT_BASE = EncoderConfig()
MINILM_L6 = EncoderConfig(layers=6, d_model=384, heads=12, d_ff=1536)

_MATS = ("w_qkv", "w_o", "w_ff1", "w_ff2")
_VECS = ("b_qkv", "b_o", "ln1_g", "ln1_b", "b_ff1", "b_ff2", "ln2_g", "ln2_b")


def random_bert_weights(cfg, seed=0, std=0.02):
    """Random-init weights in the reference's (out_features, in_features) layout: matrices
    ~N(0,std), biases 0, LayerNorm gamma 1 / beta 0."""
    rng = np.random.default_rng(seed)
    d, ff = cfg.d_model, cfg.d_ff
    n = lambda *s: (rng.standard_normal(s) * std).astype(np.float32)
    w = {"tok_emb": n(cfg.vocab, d), "pos_emb": n(cfg.max_pos, d), "type_emb": n(2, d),
         "emb_ln_g": np.ones(d, np.float32), "emb_ln_b": np.zeros(d, np.float32), "layers": []}
    for _ in range(cfg.layers):
        w["layers"].append({
            "w_qkv": n(3 * d, d), "b_qkv": np.zeros(3 * d, np.float32),
            "w_o": n(d, d), "b_o": np.zeros(d, np.float32),
            "ln1_g": np.ones(d, np.float32), "ln1_b": np.zeros(d, np.float32),
            "w_ff1": n(ff, d), "b_ff1": np.zeros(ff, np.float32),
            "w_ff2": n(d, ff), "b_ff2": np.zeros(d, np.float32),
            "ln2_g": np.ones(d, np.float32), "ln2_b": np.zeros(d, np.float32)})
    return w


class BertEncoder:
    def __init__(self, core, cfg, weights, dtype="fp32"):
        self.core = core.core if hasattr(core, "core") else core
        if not isinstance(self.core, HipCore):
            raise TypeError("BertEncoder needs a Compute() backend or its HipCore")
        if cfg.head_dim not in (32, 64, 128) or cfg.head_dim * cfg.heads != cfg.d_model:
            raise ValueError("d_model must be heads*head_dim with head_dim 32, 64 or 128")
        self.cfg, self.dtype, self.code = cfg, dtype, dtype_code(dtype)
        c = self.core
        self._keep = []                       # device buffers owned by the encoder
        up = lambda a, code=L.GRL_F32: self._own(c.upload(a, code))
        self.tok, self.pos, self.typ = up(weights["tok_emb"]), up(weights["pos_emb"]), up(weights["type_emb"])
        self.emb_g, self.emb_b = up(weights["emb_ln_g"]), up(weights["emb_ln_b"])
        self.layer_structs = []
        for lw in weights["layers"]:
            s = L.BertLayer()
            for k in _MATS:
                setattr(s, k, up(lw[k], self.code).ptr)
            for k in _VECS:
                setattr(s, k, up(np.asarray(lw[k]).reshape(-1)).ptr)
            self.layer_structs.append(s)
        self._shape = None

    def _own(self, buf):
        self._keep.append(buf)
        return buf

    # ---- device-side state for one (B,S): hidden states, workspace, ids, mask, pooled output
    def prepare(self, B, S):
        if self._shape == (B, S):
            return
        self.release_activations()
        cfg, c = self.cfg, self.core
        if S > cfg.max_pos:
            raise ValueError(f"sequence length {S} exceeds max_pos {cfg.max_pos}")
        es = 2 if self.code == L.GRL_BF16 else 4
        ws = c.lib.grl_bert_layer_workspace(self.code, B, S, cfg.heads, cfg.head_dim, cfg.d_ff)
        self.x = c.alloc(B * S * cfg.d_model * es)
        self.ws = c.alloc(ws)
        self.ids = c.alloc(B * S * 4)
        self.mask = c.alloc(B * S * 4)
        self.pooled = c.alloc(B * cfg.d_model * 4)
        self._shape = (B, S)

    def release_activations(self):
        if self._shape is not None:
            for b in (self.x, self.ws, self.ids, self.mask, self.pooled):
                b.free()
            self._shape = None

    def set_inputs(self, input_ids, attention_mask=None):
        ids = np.ascontiguousarray(input_ids, dtype=np.int32)
        if ids.ndim != 2:
            raise ValueError("input_ids must be (batch, seq_len)")
        if ids.size and (ids.min() < 0 or ids.max() >= self.cfg.vocab):
            raise IndexError("token id out of range")      # numpy indexing in the reference raises IndexError
        B, S = ids.shape
        self.prepare(B, S)
        c = self.core
        L.check(c.lib.grl_h2d(c.ctx, self.ids.ptr, ids.ctypes.data, ids.nbytes), "upload ids")
        self.has_mask = attention_mask is not None
        if self.has_mask:
            m = np.ascontiguousarray(attention_mask, dtype=np.float32)
            if m.shape != (B, S):
                raise ValueError("attention_mask must be (batch, seq_len)")
            L.check(c.lib.grl_h2d(c.ctx, self.mask.ptr, m.ctypes.data, m.nbytes), "upload mask")

    def launch(self, pool=True):
        """Enqueue one full forward on the context stream (no host synchronisation)."""
        B, S = self._shape
        cfg, c, lib = self.cfg, self.core, self.core.lib
        mask = self.mask.ptr if self.has_mask else None
        L.check(lib.grl_embed(c.ctx, self.code, B, S, cfg.d_model, cfg.vocab, self.ids.ptr, self.tok.ptr,
                              self.pos.ptr, self.typ.ptr, self.x.ptr), "embed")
        L.check(lib.grl_layernorm(c.ctx, self.code, B * S, cfg.d_model, self.x.ptr, None, self.emb_g.ptr,
                                  self.emb_b.ptr, cfg.eps, self.x.ptr), "embedding layernorm")
        for s in self.layer_structs:
            L.check(lib.grl_bert_layer_fwd(c.ctx, self.code, B, S, cfg.heads, cfg.head_dim, cfg.d_ff, ctypes.byref(s),
                                           mask, cfg.eps, self.x.ptr, self.ws.ptr), "bert_layer_fwd")
        if pool:
            L.check(lib.grl_mean_pool(c.ctx, self.code, B, S, cfg.d_model, self.x.ptr, mask, self.pooled.ptr, 1), "mean_pool")

    def forward(self, input_ids, attention_mask=None, pool=True):
        """pool=True -> L2-normalised mean-pooled embeddings (B, d); False -> hidden states (B,S,d)."""
        self.set_inputs(input_ids, attention_mask)
        self.launch(pool)
        B, S = self._shape
        if pool:
            return self.core.download(self.pooled, (B, self.cfg.d_model))
        return self.core.download(self.x, (B, S, self.cfg.d_model), self.code)

    def flops_per_forward(self, B, S):
        """2*M*N*K per GEMM + 4*B*H*S^2*D for attention (dense count)."""
        cfg = self.cfg
        M, d, ff = B * S, cfg.d_model, cfg.d_ff
        per_layer = 2 * M * d * 3 * d + 2 * M * d * d + 2 * 2 * M * d * ff + 4 * B * cfg.heads * S * S * cfg.head_dim
        return cfg.layers * per_layer
