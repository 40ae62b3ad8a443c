"""grilly's transformer-forward hot path on AMD Instinct MI355X (gfx950).

    import grilly_amd
    backend = grilly_amd.Compute()
    y = backend.fnn.linear(x, W, b)
    o = backend.attention.flash_attention2(q, k, v, num_heads, head_dim)

Same numpy-in / numpy-out methods as the reference's `grilly.Compute()` for this path; the
work is done by hand-written HIP kernels in grilly_amd/lib/libgrilly_hip.so.  `grilly_amd.nn`
holds forward-only Module adapters (Linear, LayerNorm, FlashAttention2, TransformerEncoderLayer ...).
"""
from .backend.compute import HipCompute, Compute
from .encoder import (BertEncoder, EncoderConfig, PreNormEncoder, PreNormEncoderConfig, random_bert_weights,
                      random_prenorm_weights)

__all__ = ["Compute", "HipCompute", "BertEncoder", "EncoderConfig", "random_bert_weights",
           "PreNormEncoder", "PreNormEncoderConfig", "random_prenorm_weights"]
__version__ = "0.1.0"
