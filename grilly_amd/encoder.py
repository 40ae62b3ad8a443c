"""Device-resident encoder forwards built from the hot-path kernels: the BERT-style post-LN encoder
(BertEncoder) and the pre-norm / rotary / GeGLU one (PreNormEncoder, further down).

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
    emb_eps: float = None      # embedding LayerNorm: the checkpoint's own eps in the reference (:729-736); None = eps

    @property
    def head_dim(self):
        return self.d_model // self.heads

    @property
    def embedding_eps(self):
        return self.eps if self.emb_eps is None else self.emb_eps


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
    """fused=None (default): both LayerNorms of every layer are folded into the GEMMs around them whenever the
    direct-to-LDS GEMM kernels take the layer's shapes (d_model and d_ff multiples of 64 in bf16, 32 in fp32) and the
    batch has at least FUSED_MIN_ROWS token rows: the residual stream then travels as raw rows plus row statistics and
    no LayerNorm pass runs over HBM between the embedding and the final LayerNorm (grl_bert_layer_fwd_fused).  Smaller
    batches run the seven-launch layer with its two LayerNorm passes (grl_bert_layer_fwd): a handful of token rows
    make a handful of tiles, the plain GEMMs then take 64 x 64 tiles while the fused layer's residual GEMM has none
    below 128 x 128, and the LayerNorm passes it saves cost next to nothing there (one sentence of 32 tokens in fp32:
    1.9 against 4.5 ms; level at 4096 rows; the fused layer 4 - 7 % ahead at 8192 - 16384 rows in bf16).  Both weight
    sets stay resident.  fused=False always takes the seven-launch layer;
    fused=True always the fused one, and raises for shapes it does not take."""
    FUSED_MIN_ROWS = 8192

    def __init__(self, core, cfg, weights, dtype="fp32", fused=None):
        self.core = core.core if hasattr(core, "core") else core
        if not isinstance(self.core, HipCore):
            raise TypeError("BertEncoder needs a Compute() backend or its HipCore")
        if cfg.head_dim * cfg.heads != cfg.d_model:
            raise ValueError("d_model must be heads*head_dim")
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
        slab = 64 if self.code == L.GRL_BF16 else 32
        eligible = cfg.d_model % slab == 0 and cfg.d_ff % slab == 0 and cfg.layers > 0
        if fused and not eligible:
            raise ValueError(f"the fused layer needs d_model and d_ff to be multiples of {slab} in {dtype}")
        self.fused = eligible if fused is None else bool(fused)
        self._fused_min_rows = self.FUSED_MIN_ROWS if fused is None else 0
        self.fused_structs = []
        if self.fused:
            # every GEMM that reads a LayerNorm's output gets that norm folded into its weight (once, here):
            # QKV of layer l reads the embedding norm (l = 0) or the second norm of layer l-1, FFN1 reads ln1
            d, ff = cfg.d_model, cfg.d_ff
            es = 2 if self.code == L.GRL_BF16 else 4

            def fold(w_ptr, b_ptr, g_ptr, bt_ptr, n, k):
                ws, cs, bf = self._own(c.alloc(n * k * es)), self._own(c.alloc(n * 4)), self._own(c.alloc(n * 4))
                L.check(c.lib.grl_ln_fold(c.ctx, self.code, n, k, w_ptr, g_ptr, bt_ptr, b_ptr, ws.ptr, cs.ptr, bf.ptr), "fold layernorm")
                return ws.ptr, cs.ptr, bf.ptr
            in_g, in_b = self.emb_g.ptr, self.emb_b.ptr
            for s in self.layer_structs:
                f = L.BertLayerFused()
                f.ws_qkv, f.c_qkv, f.bf_qkv = fold(s.w_qkv, s.b_qkv, in_g, in_b, 3 * d, d)
                f.in_g, f.in_b = in_g, in_b
                f.w_o, f.b_o, f.ln1_g, f.ln1_b = s.w_o, s.b_o, s.ln1_g, s.ln1_b
                f.ws_ff1, f.c_ff1, f.bf_ff1 = fold(s.w_ff1, s.b_ff1, s.ln1_g, s.ln1_b, ff, d)
                f.w_ff2, f.b_ff2 = s.w_ff2, s.b_ff2
                self.fused_structs.append(f)
                in_g, in_b = s.ln2_g, s.ln2_b
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
        self.fused_now = self.fused and B * S >= self._fused_min_rows        # which layer form this batch runs
        wsfn = c.lib.grl_bert_layer_fused_workspace if self.fused_now else c.lib.grl_bert_layer_workspace
        ws = wsfn(self.code, B, S, cfg.heads, cfg.head_dim, cfg.d_ff)
        self.x = c.alloc(B * S * cfg.d_model * es)
        self.stats = c.alloc(max(B * S, 1) * 8)        # {1/sd, mean/sd} per row of the raw residual stream (fused layers)
        self.ws = c.alloc(ws)
        self.ids = c.alloc(B * S * 4)
        self.mask = c.alloc(B * S * 4)
        self.pooled = c.alloc(B * cfg.d_model * 4)
        self._shape = (B, S)

    def release_activations(self):
        if self._shape is not None:
            for b in (self.x, self.stats, self.ws, self.ids, self.mask, self.pooled):
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
        if self.fused_now and B * S > 0:
            # raw embedding rows + their statistics; every layer consumes and produces (raw rows, statistics); the last
            # layer's second LayerNorm is the one pass that writes normalised rows
            L.check(lib.grl_embed(c.ctx, self.code, B, S, cfg.d_model, cfg.vocab, self.ids.ptr, self.tok.ptr, self.pos.ptr,
                                  self.typ.ptr, self.x.ptr), "embedding")
            L.check(lib.grl_ln_stats(c.ctx, self.code, B * S, cfg.d_model, self.x.ptr, cfg.embedding_eps, self.stats.ptr), "embedding statistics")
            for f in self.fused_structs:
                L.check(lib.grl_bert_layer_fwd_fused(c.ctx, self.code, B, S, cfg.heads, cfg.head_dim, cfg.d_ff, ctypes.byref(f),
                                                     mask, cfg.eps, self.x.ptr, self.stats.ptr, self.ws.ptr), "bert_layer_fwd_fused")
            last = self.layer_structs[-1]
            L.check(lib.grl_layernorm(c.ctx, self.code, B * S, cfg.d_model, self.x.ptr, None, last.ln2_g, last.ln2_b, cfg.eps,
                                      self.x.ptr), "final layernorm")
        else:
            L.check(lib.grl_embed_layernorm(c.ctx, self.code, B, S, cfg.d_model, cfg.vocab, self.ids.ptr, self.tok.ptr,
                                            self.pos.ptr, self.typ.ptr, self.emb_g.ptr, self.emb_b.ptr, cfg.embedding_eps,
                                            self.x.ptr), "embedding + layernorm")
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


# ------------------------------------------------------------------------------------------------
@dataclass
class PreNormEncoderConfig:
    """ModernBERT-shaped encoder: token embeddings only, rotary positions, GeGLU MLP."""
    layers: int = 22
    d_model: int = 768
    heads: int = 12
    d_ff: int = 1152           # width of each GeGLU half (Wi is (2*d_ff, d_model))
    vocab: int = 50368
    eps: float = 1e-5          # the reference hard-codes 1e-5 for the layer norm in front of the MLP (:901)
    emb_eps: float = 1e-5
    final_eps: float = 1e-5
    rope_base: float = 10000.0
    rope_scaling: float = 1.0

    @property
    def head_dim(self):
        return self.d_model // self.heads


def random_prenorm_weights(cfg, seed=0, std=0.02):
    """Random-init weights, (out_features, in_features) matrices ~N(0,std), biases 0, norms 1 / 0."""
    rng = np.random.default_rng(seed)
    d, ff = cfg.d_model, cfg.d_ff
    n = lambda *s: (rng.standard_normal(s) * std).astype(np.float32)
    one, zero = (lambda k: np.ones(k, np.float32)), (lambda k: np.zeros(k, np.float32))
    w = {"tok_emb": n(cfg.vocab, d), "emb_ln_g": one(d), "emb_ln_b": zero(d),
         "final_ln_g": one(d), "final_ln_b": zero(d), "layers": []}
    for _ in range(cfg.layers):
        w["layers"].append({
            "w_qkv": n(3 * d, d), "b_qkv": zero(3 * d), "w_o": n(d, d), "b_o": zero(d),
            "ffn_ln_g": one(d), "ffn_ln_b": zero(d),
            "w_ff_in": n(ff, d), "b_ff_in": zero(ff), "w_ff_gate": n(ff, d), "b_ff_gate": zero(ff),
            "w_ff2": n(d, ff), "b_ff2": zero(d)})
    return w


class PreNormEncoder:
    """Device-resident forward of the reference's pre-norm branch
    (utils/vulkan_sentence_transformer.py:799-970 per layer; encode :1146-1183 around it):

        x = LN(tok_emb[ids]; emb)                                              (:1153-1155, :749-785)
        per layer:  x += Wo.Attn(rope(Wq x), rope(Wk x), Wv x; key mask)       (:806-893, no norm in front)
                    x += W2.(gelu(Wi_in.LN(x)) * (Wi_gate.LN(x)))              (:901-945)
        x = LN(x; final)   (only if final_ln_g is given, :1166-1175)
        pooled = x[:, 0, :] (first token), L2-normalised                       (:1179-1183, :1194-1201)

    Built from the same entry points as the post-LN encoder: the projection GEMMs, attention with the
    rotate-half rotation fused, the dual GEMM with the GELU gate, and the GEMM that adds the residual stream in
    place.  The LayerNorm in front of the MLP is folded into that dual GEMM (gamma into the two weights, beta into
    the biases, once at construction; the GEMM reads the residual stream itself and applies each row's mean and
    1/sd in its epilogue), so the normalised rows are never written.
    The packed Wqkv is one GEMM; attention reads its three column blocks in place.  The +-50 / +-1e6 clips the
    reference puts around the gate (:924-930) are not applied: they only act beyond those magnitudes."""

    def __init__(self, core, cfg, weights, dtype="fp32", stats_from_gemm=None):
        self.core = core.core if hasattr(core, "core") else core
        if not isinstance(self.core, HipCore):
            raise TypeError("PreNormEncoder needs a Compute() backend or its HipCore")
        self._stats_from_gemm = stats_from_gemm        # None: wherever the kernel takes the width
        if cfg.head_dim * cfg.heads != cfg.d_model or cfg.head_dim % 2 or cfg.head_dim > 128:
            raise ValueError("d_model must be heads*head_dim with an even head_dim up to 128 (rotary positions)")
        self.cfg, self.dtype, self.code = cfg, dtype, dtype_code(dtype)
        c = self.core
        self._keep = []
        up = lambda a, code=L.GRL_F32: self._own(c.upload(a, code))
        vec = lambda a: up(np.asarray(a, np.float32).reshape(-1))
        self.tok = up(weights["tok_emb"])
        self.emb_g, self.emb_b = vec(weights["emb_ln_g"]), vec(weights["emb_ln_b"])
        self.final = None
        if weights.get("final_ln_g") is not None:
            self.final = (vec(weights["final_ln_g"]), vec(weights["final_ln_b"]))
        self.layers = []
        es = 2 if self.code == L.GRL_BF16 else 4
        d, ff = cfg.d_model, cfg.d_ff
        for lw in weights["layers"]:
            entry = {k: up(lw[k], self.code) for k in ("w_qkv", "w_o", "w_ff2")}
            entry.update({k: vec(lw[k]) for k in ("b_qkv", "b_o", "b_ff2")})
            g, bt = c.upload(np.asarray(lw["ffn_ln_g"], np.float32).reshape(-1)), c.upload(np.asarray(lw["ffn_ln_b"], np.float32).reshape(-1))
            for name in ("gate", "in"):
                raw = c.upload(lw["w_ff_" + name], self.code)
                b = c.upload(np.asarray(lw["b_ff_" + name], np.float32).reshape(-1))
                ws, cs, bf = self._own(c.alloc(ff * d * es)), self._own(c.alloc(ff * 4)), self._own(c.alloc(ff * 4))
                L.check(c.lib.grl_ln_fold(c.ctx, self.code, ff, d, raw.ptr, g.ptr, bt.ptr, b.ptr, ws.ptr, cs.ptr, bf.ptr), "fold mlp layernorm")
                entry["ws_" + name], entry["cs_" + name], entry["bf_" + name] = ws, cs, bf
                raw.free(); b.free()
            g.free(); bt.free()
            self.layers.append(entry)
        self._shape = None

    def _own(self, buf):
        self._keep.append(buf)
        return buf

    def prepare(self, B, S):
        if self._shape == (B, S):
            return
        self.release_activations()
        cfg, c = self.cfg, self.core
        es = 2 if self.code == L.GRL_BF16 else 4
        act = B * S * cfg.d_model * es
        self.x, self.att = (c.alloc(act) for _ in range(2))
        self.stats = c.alloc(B * S * 8)                # {1/sd, mean/sd} per row, for the GEMM that carries the MLP's LayerNorm
        # The row statistics come out of the epilogue of the output projection that writes the rows (the GEMM entry point
        # that adds LayerNorm(residual) and reduces the moments of what it stores, here with the identity in place of the
        # LayerNorm: statistics {1, 0}, scale 1, shift 0) where that kernel takes the shape; else from a pass over the rows.
        slab = 64 if self.code == L.GRL_BF16 else 32
        self.stats_from_gemm = cfg.d_model % slab == 0 if self._stats_from_gemm is None else bool(self._stats_from_gemm)
        if self.stats_from_gemm and cfg.d_model % slab:
            raise ValueError(f"row statistics out of the GEMM epilogue need d_model to be a multiple of {slab}")
        if self.stats_from_gemm:
            ident = np.zeros((B * S, 2), np.float32)
            ident[:, 0] = 1.0
            self.ident_stats = c.upload_raw(ident)
            self.ones, self.zeros = c.upload_raw(np.ones(cfg.d_model, np.float32)), c.upload_raw(np.zeros(cfg.d_model, np.float32))
            self.part = c.alloc(int(c.lib.grl_gemm_nt_resln_workspace(B * S, cfg.d_model)))
        self.qkv = c.alloc(3 * act)                    # packed (M, 3d): Q, K, V are its three column blocks
        self.h = c.alloc(B * S * cfg.d_ff * es)
        self.ids = c.alloc(B * S * 4)
        self.mask = c.alloc(B * S * 4)
        first = np.zeros((B, S), np.float32)
        first[:, 0] = 1.0                              # "mean" over the first token only = that token
        self.first = c.upload_raw(first)
        self.pooled = c.alloc(B * cfg.d_model * 4)
        self._shape = (B, S)

    def release_activations(self):
        if self._shape is not None:
            for b in (self.x, self.qkv, self.att, self.stats, self.h, self.ids, self.mask, self.first, self.pooled):
                b.free()
            if self.stats_from_gemm:
                for b in (self.ident_stats, self.ones, self.zeros, self.part):
                    b.free()
            self._shape = None

    def set_inputs(self, input_ids, attention_mask=None):
        ids = np.ascontiguousarray(input_ids, dtype=np.int32)
        if ids.ndim != 2 or ids.shape[1] == 0:
            raise ValueError("input_ids must be (batch, seq_len) with seq_len > 0")
        if ids.size and (ids.min() < 0 or ids.max() >= self.cfg.vocab):
            raise IndexError("token id out of range")
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
        cfg, c, lib, code = self.cfg, self.core, self.core.lib, self.code
        M, d, ff, H, D = B * S, cfg.d_model, cfg.d_ff, cfg.heads, cfg.head_dim
        es = 2 if code == L.GRL_BF16 else 4
        mask = self.mask.ptr if self.has_mask else None
        L.check(lib.grl_embed_layernorm(c.ctx, code, B, S, d, cfg.vocab, self.ids.ptr, self.tok.ptr, None, None,
                                        self.emb_g.ptr, self.emb_b.ptr, cfg.emb_eps, self.x.ptr), "embedding + layernorm")
        for w in self.layers:
            # one GEMM with the packed weight; attention reads Q, K, V as column blocks of its output and applies
            # the rotation itself (queries as they are loaded, keys once per row from the cached table)
            L.check(lib.grl_gemm_nt(c.ctx, code, code, M, 3 * d, d, self.x.ptr, w["w_qkv"].ptr, w["b_qkv"].ptr,
                                    self.qkv.ptr, L.EPI_NONE), "q/k/v projection")
            L.check(lib.grl_fa2_fwd_strided(c.ctx, code, B, S, H, D, self.qkv.ptr, self.qkv.ptr + d * es,
                                            self.qkv.ptr + 2 * d * es, mask, self.att.ptr, 3 * d, 3 * d, 3 * d, d,
                                            1.0 / float(np.sqrt(D)), 0, L.ROPE_HALF, cfg.rope_base, cfg.rope_scaling),
                    "attention")
            # LayerNorm + dual GEMM; the dual GEMM activates its second ("up") operand: that is the first half of Wi here
            if self.stats_from_gemm:
                L.check(lib.grl_gemm_nt_resln(c.ctx, code, M, d, d, self.att.ptr, w["w_o"].ptr, w["b_o"].ptr, self.x.ptr,
                                              self.ident_stats.ptr, self.ones.ptr, self.zeros.ptr, self.x.ptr, cfg.eps,
                                              self.stats.ptr, self.part.ptr), "output projection + residual + row statistics")
                L.check(lib.grl_ln_glu_nt_stats(c.ctx, code, code, M, ff, d, self.x.ptr, w["ws_gate"].ptr, w["ws_in"].ptr,
                                                w["cs_gate"].ptr, w["cs_in"].ptr, w["bf_gate"].ptr, w["bf_in"].ptr,
                                                self.stats.ptr, self.h.ptr, L.EPI_GELU), "mlp layernorm + geglu")
            else:
                L.check(lib.grl_gemm_nt_res(c.ctx, code, code, M, d, d, self.att.ptr, w["w_o"].ptr, w["b_o"].ptr, self.x.ptr,
                                            self.x.ptr), "output projection + residual")
                L.check(lib.grl_ln_glu_nt(c.ctx, code, code, M, ff, d, self.x.ptr, w["ws_gate"].ptr, w["ws_in"].ptr,
                                          w["cs_gate"].ptr, w["cs_in"].ptr, w["bf_gate"].ptr, w["bf_in"].ptr, cfg.eps,
                                          self.stats.ptr, self.h.ptr, L.EPI_GELU), "mlp layernorm + geglu")
            L.check(lib.grl_gemm_nt_res(c.ctx, code, code, M, d, ff, self.h.ptr, w["w_ff2"].ptr, w["b_ff2"].ptr, self.x.ptr,
                                        self.x.ptr), "mlp output + residual")
        if self.final is not None:
            L.check(lib.grl_layernorm(c.ctx, code, M, d, self.x.ptr, None, self.final[0].ptr, self.final[1].ptr,
                                      cfg.final_eps, self.x.ptr), "final layernorm")
        if pool:
            L.check(lib.grl_mean_pool(c.ctx, code, B, S, d, self.x.ptr, self.first.ptr, self.pooled.ptr, 1), "first-token pool")

    def forward(self, input_ids, attention_mask=None, pool=True):
        """pool=True -> L2-normalised first-token embeddings (B, d); False -> hidden states (B,S,d)."""
        self.set_inputs(input_ids, attention_mask)
        self.launch(pool)
        B, S = self._shape
        if pool:
            return self.core.download(self.pooled, (B, self.cfg.d_model))
        return self.core.download(self.x, (B, S, self.cfg.d_model), self.code)
