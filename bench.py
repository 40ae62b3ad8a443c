#!/usr/bin/env python3
"""Headline benchmark: BERT-base-shaped encoder forward (12 post-LN layers, d=768, 12x64 heads,
FFN 3072 GELU, fused QKV) at batch 128 x seq 512, bf16 storage with fp32 accumulation, on ONE
MI355X.  A step = one full forward over one synthetic batch already resident in HBM.

Prints one JSON line: encoder tokens/s, plus
  roofline     -- the dominant kernel (the bf16 MFMA GEMM): algorithmic FLOPs per launch divided
                  by its average launch duration, measured here with HIP events on the library's
                  own stream, against the 2.5 PFLOP/s dense bf16 MFMA peak;
  kernels      -- the same measurement for every kernel of the layer (GEMMs and attention against
                  the MFMA peak, LayerNorm against 8 TB/s HBM);
  cpu_baseline -- the C restatement of the reference shaders (oracle/oracle.c) timed on the host
                  cores on a bounded sample (--cpu-sequences of the 128 sequences through all 12 layers).
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16 = 2.5e15      # MI355X dense bf16 MFMA, FLOP/s
PEAK_FP32 = 157.3e12
PEAK_HBM = 8.0e12       # B/s

# HBM bytes per launch of the plain bf16 GEMM kernel, mean over its three layer shapes at batch 128 x seq 512:
# rocprofv3 --pmc FETCH_SIZE (x2, the factor a 1 GiB copy kernel calibrates) + --pmc WRITE_SIZE (x1) on
# `bench.py --mode gemm`; summary in profiles/gemm_bf16_bert_shapes_hbm_traffic.md.  A profiler reading, not
# something this script can measure itself, so it is reported only for exactly that workload.
GEMM_TRAFFIC_BYTES = {("bf16", 128, 512): 617.2e6}


WARM = 5


def time_launches(core, fn, reps, warm=WARM):
    """average milliseconds of one call of fn() (which only enqueues), HIP events on the context stream"""
    for _ in range(warm):
        fn()
    core.sync()
    core.timer_start()
    for _ in range(reps):
        fn()
    return core.timer_stop() / reps


def kernel_table(backend, enc, B, S, reps, only=None):
    """per-kernel average duration of one encoder layer's launches at the benchmark shape"""
    from grilly_amd import _lib as L
    cfg, c, lib, code = enc.cfg, backend.core, backend.core.lib, enc.code
    M, d, ff, H, D = B * S, cfg.d_model, cfg.d_ff, cfg.heads, cfg.head_dim
    es = 2 if code == L.GRL_BF16 else 4
    s = enc.layer_structs[0]
    qkv, attn, ffb = c.alloc(M * 3 * d * es), c.alloc(M * d * es), c.alloc(M * ff * es)
    proj = c.alloc(M * d * es)
    x = enc.x
    peak = PEAK_BF16 if code == L.GRL_BF16 else PEAK_FP32
    scale = 1.0 / np.sqrt(D)
    runs = [
        ("gemm_qkv", "gemm_nt", lambda: lib.grl_gemm_nt(c.ctx, code, code, M, 3 * d, d, x.ptr, s.w_qkv, s.b_qkv, qkv.ptr, 0),
         2.0 * M * 3 * d * d, (M * d + 3 * d * d + M * 3 * d) * es),
        ("gemm_out", "gemm_nt", lambda: lib.grl_gemm_nt(c.ctx, code, code, M, d, d, attn.ptr, s.w_o, s.b_o, proj.ptr, 0),
         2.0 * M * d * d, (2 * M * d + d * d) * es),
        ("gemm_ffn2", "gemm_nt", lambda: lib.grl_gemm_nt(c.ctx, code, code, M, d, ff, ffb.ptr, s.w_ff2, s.b_ff2, proj.ptr, 0),
         2.0 * M * d * ff, (M * ff + d * ff + M * d) * es),
        ("gemm_ffn1_gelu", "gemm_nt_gelu", lambda: lib.grl_gemm_nt(c.ctx, code, code, M, ff, d, x.ptr, s.w_ff1, s.b_ff1, ffb.ptr, 1),
         2.0 * M * d * ff, (M * d + d * ff + M * ff) * es),
        ("fa2_fwd", "fa2", lambda: lib.grl_fa2_fwd_strided(c.ctx, code, B, S, H, D, qkv.ptr, qkv.ptr + d * es, qkv.ptr + 2 * d * es,
                                                           None, attn.ptr, 3 * d, 3 * d, 3 * d, d, scale, 0, 0, 1e4, 1.0),
         4.0 * B * H * S * S * D, 4 * M * d * es),
        ("layernorm_residual", "ln", lambda: lib.grl_layernorm(c.ctx, code, M, d, x.ptr, proj.ptr, s.ln1_g, s.ln1_b, cfg.eps, attn.ptr),
         0.0, 3 * M * d * es),
    ]
    out = {}
    for name, group, fn, flops, nbytes in runs:
        if only and name not in only:
            continue
        ms = time_launches(c, fn, reps)
        rec = {"ms": round(ms, 4), "group": group, "flops": flops, "bytes": nbytes}
        if flops:
            rec["tflops"] = round(flops / ms / 1e9, 1)
            rec["frac_mfma"] = round(flops / (ms * 1e-3) / peak, 4)
        rec["gbps"] = round(nbytes / ms / 1e6, 1)
        rec["frac_hbm"] = round(nbytes / (ms * 1e-3) / PEAK_HBM, 4)
        out[name] = rec
    for b in (qkv, attn, ffb, proj):
        b.free()
    return out


def fill_normal(core, nbytes_elems, rng, std, code):
    """device buffer of `nbytes_elems` elements ~N(0,std), tiled from a 4 Mi-element random block"""
    from grilly_amd import _lib as L
    es = 2 if code == L.GRL_BF16 else 4
    blk = (rng.standard_normal(1 << 22) * std).astype(np.float32)
    src = core.upload(blk, code)
    dst = core.alloc(nbytes_elems * es)
    off = 0
    while off < nbytes_elems * es:
        m = min(blk.size * es, nbytes_elems * es - off)
        L.check(core.lib.grl_d2d(core.ctx, dst.ptr + off, src.ptr, m))
        off += m
    core.sync()
    src.free()
    return dst


def side_workload(backend, mode, seed, reps):
    """the two single-operator configurations: long causal attention with RoPE, and the SwiGLU MLP"""
    from grilly_amd import _lib as L
    c, lib, code = backend.core, backend.core.lib, L.GRL_BF16
    rng = np.random.default_rng(seed)
    if mode == "prenorm_forward":
        from grilly_amd import PreNormEncoder, PreNormEncoderConfig, random_prenorm_weights
        cfg = PreNormEncoderConfig()            # ModernBERT-base shape: 22 layers, d 768, 12 heads, GeGLU halves of 1152
        B, S = 128, 512
        enc = PreNormEncoder(backend, cfg, random_prenorm_weights(cfg, seed=seed), dtype="bf16")
        enc.set_inputs(rng.integers(0, cfg.vocab, (B, S)), None)
        ms = time_launches(c, enc.launch, max(reps // 4, 3), warm=2)
        M, d, ff = B * S, cfg.d_model, cfg.d_ff
        flops = cfg.layers * (2.0 * M * d * 3 * d + 2.0 * M * d * d + 3 * 2.0 * M * d * ff + 4.0 * B * cfg.heads * S * S * cfg.head_dim)
        return {"mode": mode, "workload": "pre-norm / rotary / GeGLU encoder forward, ModernBERT-base shape (22 layers, d 768, 12x64 heads, "
                "GeGLU 2x1152), batch 128 x seq 512, bf16, random weights, first-token pooling",
                "ms": round(ms, 3), "tokens_per_s": round(M / ms * 1e3, 1), "tflops": round(flops / ms / 1e9, 1),
                "frac_mfma": round(flops / (ms * 1e-3) / PEAK_BF16, 4), "flops": flops}
    if mode == "fa2_long":
        B, H, S, D = 4, 32, 8192, 128
        n = B * S * H * D
        q, k, v = (fill_normal(c, n, rng, 1.0, code) for _ in range(3))
        o = c.alloc(n * 2)
        fn = lambda: L.check(lib.grl_fa2_fwd(c.ctx, code, B, S, H, D, q.ptr, k.ptr, v.ptr, None, o.ptr,
                                             1.0 / np.sqrt(D), 1, L.ROPE_INTERLEAVED, 1e4, 1.0, None))
        ms = time_launches(c, fn, reps)
        flops = 4.0 * B * H * S * S * D * 0.5    # causal: half of the score matrix
        return {"mode": mode, "workload": "BASELINE configs[4]: causal FA2 forward with RoPE, (B,S,H,D)=(4,8192,32,128), bf16",
                "ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1), "frac_mfma": round(flops / (ms * 1e-3) / PEAK_BF16, 4),
                "flops": flops, "includes": "cos/sin table kernel + K pre-rotation kernel + attention kernel (buffers from the caching pool)", "launches": reps + WARM}
    M, Kd, F = 16384, 4096, 11008
    x = fill_normal(c, M * Kd, rng, 1.0, code)
    wg, wu = fill_normal(c, F * Kd, rng, 0.02, code), fill_normal(c, F * Kd, rng, 0.02, code)
    wd = fill_normal(c, Kd * F, rng, 0.02, code)
    h, y = c.alloc(M * F * 2), c.alloc(M * Kd * 2)
    f1 = lambda: L.check(lib.grl_swiglu_nt(c.ctx, code, code, M, F, Kd, x.ptr, wg.ptr, wu.ptr, None, None, h.ptr, None, None))
    f2 = lambda: L.check(lib.grl_gemm_nt(c.ctx, code, code, M, Kd, F, h.ptr, wd.ptr, None, y.ptr, 0))
    ms1, ms2 = time_launches(c, f1, reps), time_launches(c, f2, reps)
    fl1, fl2 = 4.0 * M * F * Kd, 2.0 * M * F * Kd
    return {"mode": mode, "workload": "BASELINE configs[3]: X[16384,4096] . (W_g,W_u)[11008,4096]^T -> silu(up)*gate -> . W_d[4096,11008]^T, bf16",
            "gate_up_swiglu": {"ms": round(ms1, 4), "tflops": round(fl1 / ms1 / 1e9, 1), "frac_mfma": round(fl1 / (ms1 * 1e-3) / PEAK_BF16, 4)},
            "down": {"ms": round(ms2, 4), "tflops": round(fl2 / ms2 / 1e9, 1), "frac_mfma": round(fl2 / (ms2 * 1e-3) / PEAK_BF16, 4)},
            "total_ms": round(ms1 + ms2, 4), "tflops": round((fl1 + fl2) / (ms1 + ms2) / 1e9, 1),
            "frac_mfma": round((fl1 + fl2) / ((ms1 + ms2) * 1e-3) / PEAK_BF16, 4), "launches_each": reps + WARM}


def cpu_baseline(cfg, weights, seed, nseq):
    """C restatement of the reference shaders on the host cores: `nseq` sequences of the workload
    (S=512 each) through embeddings + all layers.  tokens/s = nseq*512 / elapsed."""
    from oracle import oracle_np as O
    O.build()
    C = O.COracle()
    rng = np.random.default_rng(seed)
    S = 512
    ids = rng.integers(0, cfg.vocab, (nseq, S))
    t0 = time.perf_counter()
    x = C.layernorm(C.embed(ids, weights["tok_emb"], weights["pos_emb"], weights["type_emb"]),
                    weights["emb_ln_g"], weights["emb_ln_b"], cfg.eps)
    for lw in weights["layers"]:
        x = C.bert_layer(x, lw, None, cfg.heads, cfg.eps)
    dt = time.perf_counter() - t0
    return {"value": round(nseq * S / dt, 2), "unit": "tokens/s", "cores": C.num_threads(), "kind": "port",
            "sample": f"{nseq} of the 128 sequences x {S} tokens through embeddings + {cfg.layers} layers, fp32, "
                      f"oracle/oracle.c (one-output-per-invocation shader loops, OpenMP over rows); {dt:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--batch", type=int, default=128)
    ap.add_argument("--seq", type=int, default=512)
    ap.add_argument("--kernel-reps", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--mode", default="forward", choices=["forward", "gemm", "kernels", "copy", "fa2_long", "swiglu_mlp", "prenorm_forward"],
                    help="forward: the benchmark; gemm / copy: only launch the dominant GEMM kernel at its three "
                         "layer shapes, or a plain 1 GiB copy kernel (for rocprofv3 counter runs); kernels: every kernel of "
                         "the layer at its layer shape, nothing else (counter runs); fa2_long: "
                         "causal attention with RoPE at batch 4, 32 heads, seq 8192, head dim 128, bf16; swiglu_mlp: "
                         "X[16384,4096] through gate/up [11008,4096] + silu*up + down [4096,11008], bf16; prenorm_forward: the "
                         "pre-norm / rotary / GeGLU encoder at the ModernBERT-base shape, batch 128 x seq 512, bf16")
    ap.add_argument("--cpu-sequences", type=int, default=12)
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one MI355X: this path has no multi-GPU leg (data-parallel sharding over "
                 "batch needs no exchange between GPUs).  Run with --gpus 1.")

    import grilly_amd
    from grilly_amd import BertEncoder, random_bert_weights
    from grilly_amd.encoder import BERT_BASE as cfg

    seed = 20260131 + 3
    backend = grilly_amd.Compute(0)
    info = backend.device_info()
    if a.mode == "copy":
        # calibration for the HBM counters: a copy kernel that reads 1 GiB and writes 1 GiB per launch
        c, nbytes = backend.core, 1 << 30
        src, dst = c.alloc(nbytes), c.alloc(nbytes)
        c.lib.grl_memset(c.ctx, src.ptr, 1, nbytes)
        ms = time_launches(c, lambda: c.lib.grl_d2d(c.ctx, dst.ptr, src.ptr, nbytes), a.kernel_reps)
        print(json.dumps({"mode": "copy", "kernel": "copy_kernel", "bytes_read": nbytes, "bytes_written": nbytes,
                          "ms": round(ms, 4), "gbps": round(2 * nbytes / ms / 1e6, 1), "launches": a.kernel_reps + WARM}))
        backend.cleanup()
        return
    if a.mode in ("fa2_long", "swiglu_mlp", "prenorm_forward"):
        print(json.dumps(side_workload(backend, a.mode, seed, a.kernel_reps)))
        backend.cleanup()
        return
    weights = random_bert_weights(cfg, seed=seed)
    enc = BertEncoder(backend, cfg, weights, dtype=a.dtype)
    rng = np.random.default_rng(seed)
    B, S = a.batch, a.seq
    ids = rng.integers(0, cfg.vocab, (B, S))
    enc.set_inputs(ids, None)                 # no padding in this configuration

    if a.mode in ("gemm", "kernels"):
        only = ("gemm_qkv", "gemm_out", "gemm_ffn2") if a.mode == "gemm" else None
        kt = kernel_table(backend, enc, B, S, a.kernel_reps, only=only)
        print(json.dumps({"mode": a.mode, "kernels": kt, "launches_each": a.kernel_reps + WARM}))
        backend.cleanup()
        return

    for _ in range(a.warmup):
        enc.launch(pool=True)
    backend.core.sync()
    t0 = time.perf_counter()
    backend.core.timer_start()
    for _ in range(a.steps):
        enc.launch(pool=True)
    ev_ms = backend.core.timer_stop()         # records the stop event and waits for it
    backend.core.sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / a.steps
    tokens_per_s = B * S * a.steps / wall
    flops = enc.flops_per_forward(B, S)

    out = {
        "metric": "encoder tokens/s (BERT-base, L=512)", "value": round(tokens_per_s, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": a.dtype, "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: BERT-base-shaped encoder forward, 12 post-LN layers, d=768, "
                               "12x64 heads, FFN 3072 GELU, fused QKV, no padding, random init N(0,0.02)",
                   "batch": B, "seq_len": S, "tokens_per_step": B * S, "flops_per_step": flops},
        "event_ms_per_step": round(ev_ms / a.steps, 3),
        "model_tflops": round(flops / (ms_per_step * 1e-3) / 1e12, 1),
        "device": info,
    }
    peak = PEAK_BF16 if a.dtype == "bf16" else PEAK_FP32
    if not a.no_kernels:
        kt = kernel_table(backend, enc, B, S, a.kernel_reps)
        out["kernels"] = kt
        # dominant kernel = the plain (no activation) GEMM instantiation, launched three times per layer
        # (QKV, out-proj, FFN2): average FLOPs per launch over average duration per launch
        g = [kt[k] for k in ("gemm_qkv", "gemm_out", "gemm_ffn2")]
        avg_flops = sum(r["flops"] for r in g) / 3
        avg_ms = sum(r["ms"] for r in g) / 3
        ach = avg_flops / (avg_ms * 1e-3) / 1e12
        out["roofline"] = {"kernel": "gemm_nt_dma_kernel<bf16,bf16,256,256,2,4,EPI_NONE>" if a.dtype == "bf16" else "gemm_nt_dma_kernel<f32,f32,256,256,2,4,EPI_NONE>",
                           "bound": "mfma", "achieved": round(ach, 1), "peak": peak / 1e12, "unit": "TFLOP/s",
                           "frac": round(ach * 1e12 / peak, 4),
                           "traffic": GEMM_TRAFFIC_BYTES.get((a.dtype, B, S)),
                           "algorithmic_bytes": sum(r["bytes"] for r in g) / 3,
                           "avg_launch_ms": round(avg_ms, 4), "flops_per_launch": avg_flops,
                           "launches_per_step": 3 * cfg.layers}
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, weights, seed, a.cpu_sequences)
    backend.cleanup()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
