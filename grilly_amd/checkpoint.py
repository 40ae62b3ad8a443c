"""Weights of a BERT- or DistilBERT-style post-LN encoder (-> grilly_amd.BertEncoder) or of a
ModernBERT-style pre-norm one (-> grilly_amd.PreNormEncoder) from a local Hugging Face /
sentence-transformers checkpoint directory.

The reference pulls the same tensors out of a live torch model
(utils/vulkan_sentence_transformer.py:262-542 `_extract_layer_weights`, :563-708 embeddings); here
they are read straight from the files, offline, with loaders that execute nothing from them
(`safetensors`, or `torch.load(..., weights_only=True)` for a pytorch_model.bin).

    cfg, weights = load_encoder_checkpoint("/path/to/all-MiniLM-L6-v2")
    enc = grilly_amd.BertEncoder(grilly_amd.Compute(), cfg, weights, dtype="bf16")

Names follow PyTorch's (out_features, in_features) weight layout, which is also the reference's and
this library's, so nothing is transposed; the three attention projections are stacked into the packed
[Wq;Wk;Wv] of the fused QKV projection.  The activation is the reference's tanh GELU whatever
`hidden_act` says (its shaders have no erf GELU).  A ModernBERT checkpoint (tok_embeddings, Wqkv, Wi / Wo)
gives a PreNormEncoderConfig; as in the reference (:307-330, :426-452, :512-520) Wqkv stays packed as
[Wq;Wk;Wv], the first half of Wi is the half that goes through GELU, absent biases become zeros, and the
per-layer attn_norm is not used (the reference's forward skips it, :804-806).
"""
import json
import os

import numpy as np

from .encoder import EncoderConfig, PreNormEncoderConfig


def _find_dir(path):
    for sub in ("", "0_Transformer"):                       # sentence-transformers keeps the model in a sub-folder
        d = os.path.join(path, sub)
        if os.path.isfile(os.path.join(d, "config.json")):
            return d
    raise FileNotFoundError(f"no config.json under {path}")


def _load_tensors(d):
    st = os.path.join(d, "model.safetensors")
    if os.path.isfile(st):
        from safetensors.numpy import load_file
        return {k: np.asarray(v) for k, v in load_file(st).items()}
    pt = os.path.join(d, "pytorch_model.bin")
    if os.path.isfile(pt):
        import torch
        sd = torch.load(pt, map_location="cpu", weights_only=True)
        return {k: v.detach().to(torch.float32).numpy() for k, v in sd.items() if hasattr(v, "detach")}
    raise FileNotFoundError(f"neither model.safetensors nor pytorch_model.bin in {d}")


def _f32(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def load_encoder_checkpoint(path):
    """-> (EncoderConfig, weights dict).  Raises FileNotFoundError / ValueError with the missing piece named."""
    d = _find_dir(path)
    with open(os.path.join(d, "config.json")) as f:
        hf = json.load(f)
    T = _load_tensors(d)
    if any(k.endswith("embeddings.tok_embeddings.weight") for k in T):
        return _load_prenorm(hf, T)
    anchor = [k for k in T if k.endswith("embeddings.word_embeddings.weight")]
    if not anchor:
        raise ValueError("checkpoint has no embeddings.word_embeddings.weight: not a BERT / DistilBERT encoder")
    prefix = anchor[0][: -len("embeddings.word_embeddings.weight")]

    def get(*names, optional=False):
        for n in names:
            for cand in (prefix + n, prefix + n.replace(".weight", ".gamma").replace(".bias", ".beta")):
                if cand in T:
                    return _f32(T[cand])
        if optional:
            return None
        raise ValueError(f"checkpoint lacks {prefix}{names[0]}")

    distil = any(k.startswith(prefix + "transformer.layer.") for k in T)
    if distil:
        L_, dm, H, ff = hf["n_layers"], hf["dim"], hf["n_heads"], hf["hidden_dim"]
    else:
        L_, dm, H, ff = hf["num_hidden_layers"], hf["hidden_size"], hf["num_attention_heads"], hf["intermediate_size"]
    # the embedding LayerNorm runs with the model's own eps (utils/vulkan_sentence_transformer.py:729-736: BERT and
    # DistilBERT configurations say 1e-12), the layer norms with the reference's hard-coded 1e-5 (:1004, :1026)
    cfg = EncoderConfig(layers=L_, d_model=dm, heads=H, d_ff=ff, vocab=hf["vocab_size"],
                        max_pos=hf["max_position_embeddings"], emb_eps=float(hf.get("layer_norm_eps", 1e-12)))
    tok = get("embeddings.word_embeddings.weight")
    pos = get("embeddings.position_embeddings.weight")
    typ = get("embeddings.token_type_embeddings.weight", optional=True)
    if typ is None:
        typ = np.zeros((2, dm), np.float32)                # DistilBERT has no segment embeddings
    w = {"tok_emb": tok, "pos_emb": pos, "type_emb": typ,
         "emb_ln_g": get("embeddings.LayerNorm.weight"), "emb_ln_b": get("embeddings.LayerNorm.bias"), "layers": []}
    if tok.shape != (cfg.vocab, dm) or pos.shape[1] != dm:
        raise ValueError(f"embedding shapes {tok.shape}, {pos.shape} do not match config ({cfg.vocab}, {dm})")
    for i in range(L_):
        if distil:
            p = f"transformer.layer.{i}."
            names = {"q": p + "attention.q_lin", "k": p + "attention.k_lin", "v": p + "attention.v_lin",
                     "o": p + "attention.out_lin", "ln1": p + "sa_layer_norm", "ff1": p + "ffn.lin1",
                     "ff2": p + "ffn.lin2", "ln2": p + "output_layer_norm"}
        else:
            p = f"encoder.layer.{i}."
            names = {"q": p + "attention.self.query", "k": p + "attention.self.key", "v": p + "attention.self.value",
                     "o": p + "attention.output.dense", "ln1": p + "attention.output.LayerNorm",
                     "ff1": p + "intermediate.dense", "ff2": p + "output.dense", "ln2": p + "output.LayerNorm"}
        wq, wk, wv = (get(names[t] + ".weight") for t in "qkv")
        bq, bk, bv = (get(names[t] + ".bias") for t in "qkv")
        lw = {"w_qkv": np.concatenate([wq, wk, wv], 0), "b_qkv": np.concatenate([bq, bk, bv], 0),
              "w_o": get(names["o"] + ".weight"), "b_o": get(names["o"] + ".bias"),
              "ln1_g": get(names["ln1"] + ".weight"), "ln1_b": get(names["ln1"] + ".bias"),
              "w_ff1": get(names["ff1"] + ".weight"), "b_ff1": get(names["ff1"] + ".bias"),
              "w_ff2": get(names["ff2"] + ".weight"), "b_ff2": get(names["ff2"] + ".bias"),
              "ln2_g": get(names["ln2"] + ".weight"), "ln2_b": get(names["ln2"] + ".bias")}
        want = {"w_qkv": (3 * dm, dm), "w_o": (dm, dm), "w_ff1": (ff, dm), "w_ff2": (dm, ff)}
        for k, shp in want.items():
            if lw[k].shape != shp:
                raise ValueError(f"layer {i}: {k} has shape {lw[k].shape}, config says {shp}")
        w["layers"].append(lw)
    return cfg, w


def _load_prenorm(hf, T):
    """ModernBERT names -> (PreNormEncoderConfig, weights for PreNormEncoder)."""
    anchor = [k for k in T if k.endswith("embeddings.tok_embeddings.weight")][0]
    prefix = anchor[: -len("embeddings.tok_embeddings.weight")]
    dm, ff, L_ = hf["hidden_size"], hf["intermediate_size"], hf["num_hidden_layers"]

    def get(name, zeros=None):
        if prefix + name in T:
            return _f32(T[prefix + name])
        if zeros is not None:
            return np.zeros(zeros, np.float32)
        raise ValueError(f"checkpoint lacks {prefix}{name}")

    rope_base = hf.get("local_rope_theta") or hf.get("rope_theta") or 10000.0      # reference :830-833
    scaling = hf.get("rope_scaling")
    cfg = PreNormEncoderConfig(layers=L_, d_model=dm, heads=hf["num_attention_heads"], d_ff=ff, vocab=hf["vocab_size"],
                               emb_eps=hf.get("norm_eps", 1e-5), final_eps=hf.get("norm_eps", 1e-5),
                               rope_base=float(rope_base),
                               rope_scaling=float(scaling.get("factor", 1.0)) if isinstance(scaling, dict) else 1.0)
    tok = get("embeddings.tok_embeddings.weight")
    if tok.shape != (cfg.vocab, dm):
        raise ValueError(f"embedding shape {tok.shape} does not match config ({cfg.vocab}, {dm})")
    w = {"tok_emb": tok, "emb_ln_g": get("embeddings.norm.weight"), "emb_ln_b": get("embeddings.norm.bias", dm),
         "final_ln_g": get("final_norm.weight") if prefix + "final_norm.weight" in T else None,
         "final_ln_b": get("final_norm.bias", dm), "layers": []}
    for i in range(L_):
        p = f"layers.{i}."
        wi, bi = get(p + "mlp.Wi.weight"), get(p + "mlp.Wi.bias", 2 * ff)
        lw = {"w_qkv": get(p + "attn.Wqkv.weight"), "b_qkv": get(p + "attn.Wqkv.bias", 3 * dm),
              "w_o": get(p + "attn.Wo.weight"), "b_o": get(p + "attn.Wo.bias", dm),
              "ffn_ln_g": get(p + "mlp_norm.weight"), "ffn_ln_b": get(p + "mlp_norm.bias", dm),
              "w_ff_in": _f32(wi[:ff]), "b_ff_in": _f32(bi[:ff]), "w_ff_gate": _f32(wi[ff:]), "b_ff_gate": _f32(bi[ff:]),
              "w_ff2": get(p + "mlp.Wo.weight"), "b_ff2": get(p + "mlp.Wo.bias", dm)}
        want = {"w_qkv": (3 * dm, dm), "w_o": (dm, dm), "w_ff_in": (ff, dm), "w_ff_gate": (ff, dm), "w_ff2": (dm, ff)}
        for k, shp in want.items():
            if lw[k].shape != shp:
                raise ValueError(f"layer {i}: {k} has shape {lw[k].shape}, config says {shp}")
        w["layers"].append(lw)
    return cfg, w
