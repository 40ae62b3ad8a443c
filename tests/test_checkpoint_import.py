"""Local checkpoint import (grilly_amd/checkpoint.py) on synthetic BERT- and DistilBERT-named files."""
import json
import os

import numpy as np
import pytest
from dataclasses import replace as dataclasses_replace

from grilly_amd.checkpoint import load_encoder_checkpoint
from grilly_amd.encoder import EncoderConfig, random_bert_weights

CFG = EncoderConfig(layers=2, d_model=64, heads=2, d_ff=128, vocab=100, max_pos=32)


def bert_state(w, prefix="bert."):
    sd = {prefix + "embeddings.word_embeddings.weight": w["tok_emb"], prefix + "embeddings.position_embeddings.weight": w["pos_emb"],
          prefix + "embeddings.token_type_embeddings.weight": w["type_emb"],
          prefix + "embeddings.LayerNorm.weight": w["emb_ln_g"], prefix + "embeddings.LayerNorm.bias": w["emb_ln_b"]}
    d = CFG.d_model
    for i, lw in enumerate(w["layers"]):
        p = f"{prefix}encoder.layer.{i}."
        for j, t in enumerate(("query", "key", "value")):
            sd[p + f"attention.self.{t}.weight"] = lw["w_qkv"][j * d:(j + 1) * d]
            sd[p + f"attention.self.{t}.bias"] = lw["b_qkv"][j * d:(j + 1) * d]
        for name, (wk, bk) in {"attention.output.dense": ("w_o", "b_o"), "attention.output.LayerNorm": ("ln1_g", "ln1_b"),
                               "intermediate.dense": ("w_ff1", "b_ff1"), "output.dense": ("w_ff2", "b_ff2"),
                               "output.LayerNorm": ("ln2_g", "ln2_b")}.items():
            sd[p + name + ".weight"], sd[p + name + ".bias"] = lw[wk], lw[bk]
    return {k: np.ascontiguousarray(v) for k, v in sd.items()}


def noisy_weights(seed):
    w = random_bert_weights(CFG, seed=seed)
    rng = np.random.default_rng(seed + 1)
    for lw in w["layers"]:
        for k in lw:
            if lw[k].ndim == 1:
                lw[k] = (lw[k] + 0.1 * rng.standard_normal(lw[k].shape)).astype(np.float32)
    return w


def same(a, b):
    for k in ("tok_emb", "pos_emb", "type_emb", "emb_ln_g", "emb_ln_b"):
        np.testing.assert_array_equal(a[k], b[k])
    assert len(a["layers"]) == len(b["layers"])
    for la, lb in zip(a["layers"], b["layers"]):
        assert set(la) == set(lb)
        for k in la:
            np.testing.assert_array_equal(la[k], lb[k])


def write_config(d, distil=False):
    hf = ({"n_layers": 2, "dim": 64, "n_heads": 2, "hidden_dim": 128} if distil else
          {"num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 2, "intermediate_size": 128, "hidden_act": "gelu"})
    hf.update({"vocab_size": 100, "max_position_embeddings": 32, "layer_norm_eps": 1e-12})
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(hf, f)


def test_bert_safetensors_roundtrip(tmp_path):
    from safetensors.numpy import save_file
    w = noisy_weights(1)
    write_config(tmp_path)
    save_file(bert_state(w), str(tmp_path / "model.safetensors"))
    cfg, got = load_encoder_checkpoint(str(tmp_path))
    import dataclasses
    assert cfg == dataclasses.replace(CFG, emb_eps=1e-12)      # the embedding LayerNorm keeps the checkpoint's own eps
    assert cfg.embedding_eps == 1e-12 and cfg.eps == 1e-5 and CFG.embedding_eps == CFG.eps
    same(got, w)


def test_sentence_transformers_layout_and_torch_bin(tmp_path):
    torch = pytest.importorskip("torch")
    w = noisy_weights(2)
    sub = tmp_path / "0_Transformer"
    sub.mkdir()
    write_config(sub)
    torch.save({k: torch.from_numpy(v) for k, v in bert_state(w, prefix="").items()}, str(sub / "pytorch_model.bin"))
    cfg, got = load_encoder_checkpoint(str(tmp_path))
    import dataclasses
    assert cfg == dataclasses.replace(CFG, emb_eps=1e-12)      # the embedding LayerNorm keeps the checkpoint's own eps
    assert cfg.embedding_eps == 1e-12 and cfg.eps == 1e-5 and CFG.embedding_eps == CFG.eps
    same(got, w)


def test_distilbert_names(tmp_path):
    from safetensors.numpy import save_file
    w = noisy_weights(3)
    w["type_emb"] = np.zeros_like(w["type_emb"])
    d = CFG.d_model
    sd = {"distilbert.embeddings.word_embeddings.weight": w["tok_emb"], "distilbert.embeddings.position_embeddings.weight": w["pos_emb"],
          "distilbert.embeddings.LayerNorm.weight": w["emb_ln_g"], "distilbert.embeddings.LayerNorm.bias": w["emb_ln_b"]}
    for i, lw in enumerate(w["layers"]):
        p = f"distilbert.transformer.layer.{i}."
        for j, t in enumerate(("q_lin", "k_lin", "v_lin")):
            sd[p + f"attention.{t}.weight"] = lw["w_qkv"][j * d:(j + 1) * d]
            sd[p + f"attention.{t}.bias"] = lw["b_qkv"][j * d:(j + 1) * d]
        for name, (wk, bk) in {"attention.out_lin": ("w_o", "b_o"), "sa_layer_norm": ("ln1_g", "ln1_b"), "ffn.lin1": ("w_ff1", "b_ff1"),
                               "ffn.lin2": ("w_ff2", "b_ff2"), "output_layer_norm": ("ln2_g", "ln2_b")}.items():
            sd[p + name + ".weight"], sd[p + name + ".bias"] = lw[wk], lw[bk]
    write_config(tmp_path, distil=True)
    save_file({k: np.ascontiguousarray(v) for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    cfg, got = load_encoder_checkpoint(str(tmp_path))
    import dataclasses
    assert cfg == dataclasses.replace(CFG, emb_eps=1e-12)      # the embedding LayerNorm keeps the checkpoint's own eps
    assert cfg.embedding_eps == 1e-12 and cfg.eps == 1e-5 and CFG.embedding_eps == CFG.eps
    same(got, w)


def test_errors(tmp_path):
    from safetensors.numpy import save_file
    with pytest.raises(FileNotFoundError):
        load_encoder_checkpoint(str(tmp_path))
    write_config(tmp_path)
    with pytest.raises(FileNotFoundError):
        load_encoder_checkpoint(str(tmp_path))
    sd = bert_state(noisy_weights(4))
    del sd["bert.encoder.layer.1.output.dense.bias"]
    save_file(sd, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="output.dense.bias"):
        load_encoder_checkpoint(str(tmp_path))
    save_file({"x": np.zeros(3, np.float32)}, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="word_embeddings"):
        load_encoder_checkpoint(str(tmp_path))


@pytest.mark.gpu
def test_imported_checkpoint_runs_like_the_oracle(tmp_path, backend, corc):
    from safetensors.numpy import save_file
    from grilly_amd import BertEncoder
    from oracle import oracle_np as O
    w = noisy_weights(5)
    # small embeddings (variance ~1e-7 per row): the embedding LayerNorm's eps = 1e-12 of the checkpoint
    # (reference utils/vulkan_sentence_transformer.py:729-736) and the layers' 1e-5 give visibly different rows
    for k in ("tok_emb", "pos_emb", "type_emb"):
        w[k] = (w[k] * 1e-2).astype(np.float32)
    write_config(tmp_path)
    save_file(bert_state(w), str(tmp_path / "model.safetensors"))
    cfg, got = load_encoder_checkpoint(str(tmp_path))
    assert cfg.embedding_eps == 1e-12
    rng = np.random.default_rng(6)
    ids = rng.integers(0, cfg.vocab, (3, 20))
    mask = (np.arange(20)[None] < np.array([20, 9, 14])[:, None]).astype(np.float32)
    enc = BertEncoder(backend, cfg, got, dtype="fp32")
    pooled = enc.forward(ids, mask)
    emb = corc.embed(ids, w["tok_emb"], w["pos_emb"], w["type_emb"])
    x = corc.layernorm(emb, w["emb_ln_g"], w["emb_ln_b"], cfg.embedding_eps)
    wrong = corc.layernorm(emb, w["emb_ln_g"], w["emb_ln_b"], cfg.eps)
    assert O.max_rel(wrong, x) > 0.5                       # the two eps values are told apart by this input
    h0 = BertEncoder(backend, dataclasses_replace(cfg, layers=0), dict(got, layers=[]), dtype="fp32").forward(ids, mask, pool=False)
    assert O.max_rel(h0, x) < 1e-4
    for lw in w["layers"]:
        x = corc.bert_layer(x, lw, mask, cfg.heads, cfg.eps)
    assert O.max_rel(pooled, corc.mean_pool(x, mask)) < 1e-4


def test_modernbert_names(tmp_path):
    """tok_embeddings / Wqkv / Wi-Wo names give the pre-norm configuration; Wi is split first half =
    activated half, missing biases become zeros, rope base comes from local_rope_theta."""
    from safetensors.numpy import save_file
    from grilly_amd.encoder import PreNormEncoderConfig, random_prenorm_weights
    cfg = PreNormEncoderConfig(layers=2, d_model=64, heads=2, d_ff=48, vocab=90)
    w = random_prenorm_weights(cfg, seed=4)
    sd = {"model.embeddings.tok_embeddings.weight": w["tok_emb"], "model.embeddings.norm.weight": w["emb_ln_g"],
          "model.final_norm.weight": w["final_ln_g"]}
    for i, lw in enumerate(w["layers"]):
        p = f"model.layers.{i}."
        sd[p + "attn.Wqkv.weight"], sd[p + "attn.Wo.weight"] = lw["w_qkv"], lw["w_o"]
        sd[p + "mlp.Wi.weight"] = np.concatenate([lw["w_ff_in"], lw["w_ff_gate"]], 0)
        sd[p + "mlp.Wo.weight"], sd[p + "mlp_norm.weight"] = lw["w_ff2"], lw["ffn_ln_g"]
        if i > 0:
            sd[p + "attn_norm.weight"] = np.ones(64, np.float32)        # present in real files, unused by the recipe
    save_file({k: np.ascontiguousarray(v) for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    with open(tmp_path / "config.json", "w") as f:
        json.dump({"num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 2, "intermediate_size": 48,
                   "vocab_size": 90, "local_rope_theta": 160000.0, "global_rope_theta": 10000.0, "norm_eps": 1e-5}, f)
    got_cfg, got = load_encoder_checkpoint(str(tmp_path))
    assert isinstance(got_cfg, PreNormEncoderConfig)
    assert (got_cfg.layers, got_cfg.d_model, got_cfg.heads, got_cfg.d_ff, got_cfg.vocab) == (2, 64, 2, 48, 90)
    assert got_cfg.rope_base == 160000.0 and got_cfg.rope_scaling == 1.0
    np.testing.assert_array_equal(got["tok_emb"], w["tok_emb"])
    for la, lb in zip(got["layers"], w["layers"]):
        assert set(la) == set(lb)
        for k in la:
            np.testing.assert_array_equal(la[k], lb[k])           # biases: zeros on both sides
    # a wrong Wi height is reported with the layer and the name
    sd["model.layers.1.mlp.Wi.weight"] = sd["model.layers.1.mlp.Wi.weight"][:-2]
    save_file({k: np.ascontiguousarray(v) for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="layer 1: w_ff_gate"):
        load_encoder_checkpoint(str(tmp_path))
