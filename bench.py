#!/usr/bin/env python3
"""Headline benchmark: BERT-base-shaped encoder forward (12 post-LN layers, d=768, 12x64 heads,
FFN 3072 GELU, fused QKV) at batch 128 x seq 512, bf16 storage with fp32 accumulation, on ONE
MI355X.  A step = one full forward over one synthetic batch already resident in HBM.

Prints one JSON line: encoder tokens/s, plus
  roofline     -- the dominant kernel (the bf16 MFMA GEMM instantiation with the largest share of the forward):
                  algorithmic FLOPs per launch divided by its average launch duration, measured here with HIP
                  events on the library's own stream, against the 2.5 PFLOP/s dense bf16 MFMA peak;
  kernels      -- the same measurement for every kernel of the layer (GEMMs and attention against
                  the MFMA peak, LayerNorm against 8 TB/s HBM), each launched on the data the layer really
                  hands it, each with a sampled check of the timed output buffer against the float64 closed form;
  extra        -- outside the timed region: the fp32 forward of the same configuration, BASELINE configs[3]
                  (SwiGLU MLP) and configs[4] (long causal attention with RoPE), each with flops, ms,
                  fraction of the matrix peak and a sampled check of its own output buffers;
  cpu_baseline -- the C restatement of the reference shaders (oracle/oracle.c) timed on the host
                  cores on a bounded sample (--cpu-sequences of the 128 sequences through all 12 layers);
                  the GPU's hidden states of the same sequences are compared with its result;
  cpu_baseline_blas -- what the reference's gemm() really executes on the host: numpy `@` (OpenBLAS) on the
                  layer's four GEMM shapes, a bounded number of rows.
"""
import argparse
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
NOMINAL_GHZ = 2.4        # engine clock the MFMA peaks are quoted at (256 CUs x 4 SIMDs x 1024 bf16 FLOP/cycle x 2.4 GHz = 2.5 PFLOP/s)
TOL = {"bf16": 2e-2, "fp32": 1e-4}

WARM = 10


def gemm_traffic(dtype, B, S, kernel):
    """HBM bytes per launch of the dominant kernel: a profiler reading (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE),
    not something this script can measure itself, so it comes from the tracked record next to the profile
    summary and is reported only for exactly the workload it was taken on."""
    path = os.path.join(ROOT, "profiles", "gemm_bf16_bert_shapes_hbm_traffic.json")
    try:
        rec = json.load(open(path))
    except (OSError, ValueError):
        return None, None
    k = rec.get("key", {})
    if (k.get("dtype"), k.get("batch"), k.get("seq"), k.get("kernel")) != (dtype, B, S, kernel):
        return None, None
    return rec.get("traffic_bytes_per_launch"), rec.get("measured_at_commit")


def time_launches(core, fn, reps, warm=WARM):
    """average milliseconds of one call of fn() (which only enqueues), HIP events on the context stream"""
    for _ in range(warm):
        fn()
    core.sync()
    core.timer_start()
    for _ in range(reps):
        fn()
    return core.timer_stop() / reps


def lap_times(core, fn, reps, warm=WARM):
    """per-launch milliseconds of `reps` back-to-back calls of fn() (which only enqueues): one event between every two
    launches on the context stream, no host synchronisation inside the sequence"""
    from grilly_amd import _lib as L
    import ctypes
    reps = min(reps, 255)
    for _ in range(warm):
        fn()
    core.sync()
    for i in range(reps):
        L.check(core.lib.grl_timer_lap(core.ctx, i))
        fn()
    L.check(core.lib.grl_timer_lap(core.ctx, reps))
    ms = ctypes.c_float()
    out = []
    for i in range(reps):
        L.check(core.lib.grl_timer_lap_ms(core.ctx, i, i + 1, ctypes.byref(ms)))
        out.append(float(ms.value))
    return out


def median(v):
    return float(np.median(np.asarray(v, np.float64)))


def forward_kernel_times(backend, enc, cfg, forwards=8):
    """Durations of the layer's launches INSIDE whole forwards: the layer entry points record a lap event at entry and after
    each of their kernels (grl_timer_lap_trace), `forwards` forwards run back to back behind two untimed ones, and every
    interval is attributed to the launch it follows (a residual-type GEMM's interval includes its 3-5 us moment merge).
    Returns {launch name: {ms (mean), median_ms, n}} and "layer_ms": what the kernels do under the forward's sustained
    load, next to the back-to-back table of kernel_table()."""
    from grilly_amd import _lib as L
    import ctypes
    core = backend.core
    fused = getattr(enc, "fused_now", False)
    names = ["gemm_qkv_ln", "fa2_fwd", "gemm_out_resln", "gemm_ffn1_ln_gelu", "gemm_ffn2_resln"] if fused else \
            ["gemm_qkv", "fa2_fwd", "gemm_out", "layernorm_residual", "gemm_ffn1_gelu", "gemm_ffn2", "layernorm_residual"]
    per_layer = len(names) + 1                         # the mark at layer entry
    assert 1 + per_layer * cfg.layers <= 256
    acc = {}
    for _ in range(2):
        enc.launch(pool=True)
    nxt, ms = ctypes.c_int(), ctypes.c_float()
    for _ in range(forwards):
        L.check(core.lib.grl_timer_lap_trace(core.ctx, 0, None))
        enc.launch(pool=True)
        L.check(core.lib.grl_timer_lap_trace(core.ctx, -1, ctypes.byref(nxt)))
        assert nxt.value == 1 + per_layer * cfg.layers, (nxt.value, per_layer, cfg.layers)
        for layer in range(cfg.layers):
            base = 1 + layer * per_layer               # index of the layer's entry mark
            for j, nm in enumerate(names):
                L.check(core.lib.grl_timer_lap_ms(core.ctx, base + j, base + j + 1, ctypes.byref(ms)))
                acc.setdefault(nm, []).append(float(ms.value))
    out = {nm: {"ms": round(float(np.mean(v)), 4), "median_ms": round(median(v), 4), "n": len(v)} for nm, v in acc.items()}
    out["layer_ms"] = round(sum(sum(v) for v in acc.values()) / (forwards * cfg.layers), 4)
    return out


def download_rows(core, buf, row0, nrows, ncols, code):
    """rows [row0, row0+nrows) of a device matrix with `ncols` columns -> float32 numpy"""
    from grilly_amd import _lib as L
    es = 2 if code == L.GRL_BF16 else 4
    out = np.empty((nrows, ncols), np.float32)
    n = nrows * ncols
    src = buf.ptr + row0 * ncols * es
    if code == L.GRL_BF16:
        with core.alloc(n * 4) as tmp:
            L.check(core.lib.grl_cast(core.ctx, L.GRL_BF16, L.GRL_F32, n, src, tmp.ptr), "cast")
            L.check(core.lib.grl_d2h(core.ctx, out.ctypes.data, tmp.ptr, n * 4), "download")
    else:
        L.check(core.lib.grl_d2h(core.ctx, out.ctypes.data, src, n * 4), "download")
    return out


class _Ptr:
    """a raw device address with the .ptr attribute of a DeviceBuffer (weights held in the layer structs)"""

    def __init__(self, ptr):
        self.ptr = ptr


def gather_rows(core, buf, rows, ncols, code):
    return np.concatenate([download_rows(core, buf, int(r), 1, ncols, code) for r in rows])


def max_rel(y, ref):
    ref = np.asarray(ref, np.float64)
    return float(np.abs(np.asarray(y, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))


def kernel_table(backend, enc, B, S, reps, only=None, check=True):
    """per-kernel average duration of one encoder layer's launches at the benchmark shape.  The buffers are
    first filled by one untimed pass in data-flow order (QKV -> attention -> out-proj -> LayerNorm -> FFN1 -> FFN2),
    so every timed launch reads what the layer really hands it; after timing, sampled rows of every output
    buffer are compared with the float64 closed form of the same inputs (CPU leg, checker only)."""
    from grilly_amd import _lib as L
    cfg, c, lib, code = enc.cfg, backend.core, backend.core.lib, enc.code
    M, d, ff, H, D = B * S, cfg.d_model, cfg.d_ff, cfg.heads, cfg.head_dim
    es = 2 if code == L.GRL_BF16 else 4
    dt = "bf16" if code == L.GRL_BF16 else "fp32"
    s = enc.layer_structs[0]
    qkv, attn, ffb = c.alloc(M * 3 * d * es), c.alloc(M * d * es), c.alloc(M * ff * es)
    proj, x1, y2 = c.alloc(M * d * es), c.alloc(M * d * es), c.alloc(M * d * es)
    x = enc.x
    peak = PEAK_BF16 if code == L.GRL_BF16 else PEAK_FP32
    scale = 1.0 / np.sqrt(D)
    f_qkv = lambda: lib.grl_gemm_nt(c.ctx, code, code, M, 3 * d, d, x.ptr, s.w_qkv, s.b_qkv, qkv.ptr, 0)
    f_fa = lambda: lib.grl_fa2_fwd_strided(c.ctx, code, B, S, H, D, qkv.ptr, qkv.ptr + d * es, qkv.ptr + 2 * d * es,
                                           None, attn.ptr, 3 * d, 3 * d, 3 * d, d, scale, 0, 0, 1e4, 1.0)
    # the same attention launch under a key mask of right-padded sequences (lengths uniform in [S/2, S])
    lens = np.random.default_rng(11).integers(S // 2, S + 1, B)
    mask_h = (np.arange(S)[None] < lens[:, None]).astype(np.float32)
    mask_d, attn_m = c.upload(mask_h), c.alloc(M * d * es)
    f_fam = lambda: lib.grl_fa2_fwd_strided(c.ctx, code, B, S, H, D, qkv.ptr, qkv.ptr + d * es, qkv.ptr + 2 * d * es,
                                            mask_d.ptr, attn_m.ptr, 3 * d, 3 * d, 3 * d, d, scale, 0, 0, 1e4, 1.0)
    f_out = lambda: lib.grl_gemm_nt(c.ctx, code, code, M, d, d, attn.ptr, s.w_o, s.b_o, proj.ptr, 0)
    f_ln = lambda: lib.grl_layernorm(c.ctx, code, M, d, x.ptr, proj.ptr, s.ln1_g, s.ln1_b, cfg.eps, x1.ptr)
    f_ff1 = lambda: lib.grl_gemm_nt(c.ctx, code, code, M, ff, d, x1.ptr, s.w_ff1, s.b_ff1, ffb.ptr, 1)
    f_ff2 = lambda: lib.grl_gemm_nt(c.ctx, code, code, M, d, ff, ffb.ptr, s.w_ff2, s.b_ff2, y2.ptr, 0)
    for f in (f_qkv, f_fa, f_out, f_ln, f_ff1, f_ff2):       # data-flow order, untimed
        L.check(f())
    c.sync()
    fused_runs = []
    if getattr(enc, "fused_now", False):
        # the four GEMMs of the layer in the form the forward launches them (LayerNorms folded in): the raw residual
        # stream r0 = x (its "LayerNorm" statistics are those of x itself), r1 = out-proj + LN(r0), ff, r2 = FFN2 + LN(r1)
        fs = enc.fused_structs[0]
        r1, r2, ffl = c.alloc(M * d * es), c.alloc(M * d * es), c.alloc(M * ff * es)
        qkvl = c.alloc(M * 3 * d * es)
        st0, st1, st2 = c.alloc(M * 8), c.alloc(M * 8), c.alloc(M * 8)
        part = c.alloc(lib.grl_gemm_nt_resln_workspace(M, d))
        f_st = lambda: lib.grl_ln_stats(c.ctx, code, M, d, x.ptr, cfg.eps, st0.ptr)
        f_qkvl = lambda: lib.grl_ln_gemm_nt_stats(c.ctx, code, code, M, 3 * d, d, x.ptr, fs.ws_qkv, fs.c_qkv, fs.bf_qkv, st0.ptr, qkvl.ptr, 0)
        f_outl = lambda: lib.grl_gemm_nt_resln(c.ctx, code, M, d, d, attn.ptr, fs.w_o, fs.b_o, x.ptr, st0.ptr, fs.in_g, fs.in_b, r1.ptr,
                                               cfg.eps, st1.ptr, part.ptr)
        f_ff1l = lambda: lib.grl_ln_gemm_nt_stats(c.ctx, code, code, M, ff, d, r1.ptr, fs.ws_ff1, fs.c_ff1, fs.bf_ff1, st1.ptr, ffl.ptr, 1)
        f_ff2l = lambda: lib.grl_gemm_nt_resln(c.ctx, code, M, d, ff, ffl.ptr, fs.w_ff2, fs.b_ff2, r1.ptr, st1.ptr, fs.ln1_g, fs.ln1_b, r2.ptr,
                                               cfg.eps, st2.ptr, part.ptr)
        for f in (f_st, f_qkvl, f_outl, f_ff1l, f_ff2l):
            L.check(f())
        c.sync()
        fused_runs = [
            ("gemm_qkv_ln", "gemm_nt_ln", f_qkvl, 2.0 * M * 3 * d * d, (M * d + 3 * d * d + M * 3 * d) * es),
            ("gemm_out_resln", "gemm_nt_resln", f_outl, 2.0 * M * d * d, (3 * M * d + d * d) * es),
            ("gemm_ffn1_ln_gelu", "gemm_nt_ln_gelu", f_ff1l, 2.0 * M * d * ff, (M * d + d * ff + M * ff) * es),
            ("gemm_ffn2_resln", "gemm_nt_resln", f_ff2l, 2.0 * M * d * ff, (M * ff + d * ff + 2 * M * d) * es),
            ("ln_stats", "ln", f_st, 0.0, M * d * es + M * 8),
        ]
    runs = [
        ("gemm_qkv", "gemm_nt", f_qkv, 2.0 * M * 3 * d * d, (M * d + 3 * d * d + M * 3 * d) * es),
        ("gemm_out", "gemm_nt", f_out, 2.0 * M * d * d, (2 * M * d + d * d) * es),
        ("gemm_ffn2", "gemm_nt", f_ff2, 2.0 * M * d * ff, (M * ff + d * ff + M * d) * es),
        ("gemm_ffn1_gelu", "gemm_nt_gelu", f_ff1, 2.0 * M * d * ff, (M * d + d * ff + M * ff) * es),
        ("fa2_fwd", "fa2", f_fa, 4.0 * B * H * S * S * D, 4 * M * d * es),
        ("fa2_fwd_key_mask", "fa2", f_fam, 4.0 * B * H * S * S * D, 4 * M * d * es),     # nominal FLOPs: padding counted
        ("layernorm_residual", "ln", f_ln, 0.0, 3 * M * d * es),
    ] + fused_runs
    out = {}
    for name, group, fn, flops, nbytes in runs:
        if only and name not in only:
            continue
        ms = time_launches(c, fn, reps)
        rec = {"ms": round(ms, 4), "median_ms": round(median(lap_times(c, fn, reps)), 4), "group": group, "flops": flops, "bytes": nbytes}
        # the shader clock these launches run at: a one-wave probe on a second stream lives for 70 % of a repeat of the
        # same launch sequence (the clock is one domain for the whole GPU)
        c.sync()
        c.clock_probe_begin(max(0.7 * ms * reps, 0.05))
        for _ in range(reps):
            fn()
        rec["shader_clock_ghz"] = round(c.clock_probe_end(), 3)
        c.sync()
        if flops:
            rec["tflops"] = round(flops / ms / 1e9, 1)
            rec["frac_mfma"] = round(flops / (ms * 1e-3) / peak, 4)
        rec["gbps"] = round(nbytes / ms / 1e6, 1)
        rec["frac_hbm"] = round(nbytes / (ms * 1e-3) / PEAK_HBM, 4)
        out[name] = rec
    if check:
        from oracle import oracle_np as O          # checker only: the timed buffers against the float64 closed form
        rng = np.random.default_rng(7)
        rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 30)]))
        dl = lambda ptr, n: download_rows(c, _Ptr(ptr), 0, 1, n, L.GRL_F32)[0]
        wt = lambda ptr, r, k: download_rows(c, _Ptr(ptr), 0, r, k, code)

        def gemm_err(a_buf, K, w_ptr, b_ptr, N, c_buf, epi):
            a = gather_rows(c, a_buf, rows, K, code)
            ref = O.truth_linear(a, wt(w_ptr, N, K), dl(b_ptr, N), epi)
            return max_rel(gather_rows(c, c_buf, rows, N, code), ref)
        errs = {"gemm_qkv": gemm_err(x, d, s.w_qkv, s.b_qkv, 3 * d, qkv, "none"),
                "gemm_out": gemm_err(attn, d, s.w_o, s.b_o, d, proj, "none"),
                "gemm_ffn1_gelu": gemm_err(x1, d, s.w_ff1, s.b_ff1, ff, ffb, "gelu"),
                "gemm_ffn2": gemm_err(ffb, ff, s.w_ff2, s.b_ff2, d, y2, "none")}
        b0 = int(rng.integers(0, B))
        q3 = download_rows(c, qkv, b0 * S, S, 3 * d, code).reshape(1, S, 3, H, D)
        at = download_rows(c, attn, b0 * S, S, d, code).reshape(1, S, H, D)
        hs = [0, H - 1]
        errs["fa2_fwd"] = max_rel(at[:, :, hs], O.truth_attention(q3[:, :, 0][:, :, hs], q3[:, :, 1][:, :, hs], q3[:, :, 2][:, :, hs]))
        atm = download_rows(c, attn_m, b0 * S, S, d, code).reshape(1, S, H, D)
        errs["fa2_fwd_key_mask"] = max_rel(atm[:, :, hs], O.truth_attention(q3[:, :, 0][:, :, hs], q3[:, :, 1][:, :, hs], q3[:, :, 2][:, :, hs],
                                                                            mask=mask_h[b0:b0 + 1]))
        errs["layernorm_residual"] = max_rel(gather_rows(c, x1, rows, d, code),
                                            O.truth_layernorm(gather_rows(c, x, rows, d, code), dl(s.ln1_g, d), dl(s.ln1_b, d), cfg.eps,
                                                              residual=gather_rows(c, proj, rows, d, code)))
        for k, e in errs.items():
            if k in out:
                out[k]["max_rel_vs_float64"] = float(f"{e:.3g}")
                out[k]["within_tolerance"] = bool(e < TOL[dt])
    if fused_runs and check:
        from oracle import oracle_np as O
        rng = np.random.default_rng(8)
        rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, 30)]))
        dl = lambda ptr, n: download_rows(c, _Ptr(ptr), 0, 1, n, L.GRL_F32)[0]
        wt = lambda ptr, r, k: download_rows(c, _Ptr(ptr), 0, r, k, code)
        s0 = enc.layer_structs[0]
        xs = gather_rows(c, x, rows, d, code)
        xn = O.truth_layernorm(xs, dl(fs.in_g, d), dl(fs.in_b, d), cfg.eps)
        e = {"gemm_qkv_ln": max_rel(gather_rows(c, qkvl, rows, 3 * d, code), O.truth_linear(xn, wt(s0.w_qkv, 3 * d, d), dl(s0.b_qkv, 3 * d)))}
        r1s = gather_rows(c, r1, rows, d, code)
        e["gemm_out_resln"] = max_rel(r1s, O.truth_linear(gather_rows(c, attn, rows, d, code), wt(s0.w_o, d, d), dl(s0.b_o, d)) + xn)
        x1n = O.truth_layernorm(r1s, dl(s0.ln1_g, d), dl(s0.ln1_b, d), cfg.eps)
        ffs = gather_rows(c, ffl, rows, ff, code)
        e["gemm_ffn1_ln_gelu"] = max_rel(ffs, O.truth_linear(x1n, wt(s0.w_ff1, ff, d), dl(s0.b_ff1, ff), "gelu"))
        e["gemm_ffn2_resln"] = max_rel(gather_rows(c, r2, rows, d, code), O.truth_linear(ffs, wt(s0.w_ff2, d, ff), dl(s0.b_ff2, d)) + x1n)
        st = download_rows(c, st1, 0, M, 2, L.GRL_F32)[rows]
        r64 = r1s.astype(np.float64)
        sd = np.sqrt(r64.var(-1) + cfg.eps)
        # 1/sd relative, mean/sd absolute (it is a number of spreads, near zero for these rows)
        e["row_statistics_out"] = max(max_rel(st[:, 0], 1 / sd), float(np.abs(st[:, 1] - r64.mean(-1) / sd).max()))
        for k, v in e.items():
            if k == "row_statistics_out":
                out["gemm_out_resln"]["row_statistics_max_err"] = float(f"{v:.3g}")
            else:
                out[k]["max_rel_vs_float64"] = float(f"{v:.3g}")
                out[k]["within_tolerance"] = bool(v < TOL[dt])
    if fused_runs:
        for b in (r1, r2, ffl, qkvl, st0, st1, st2, part):
            b.free()
    for b in (qkv, attn, ffb, proj, x1, y2, mask_d, attn_m):
        b.free()
    return out


def fill_normal(core, n_elems, rng, std, code):
    """device buffer of `n_elems` elements ~N(0,std), tiled from a 4 Mi-element random block; returns the
    buffer and the host copy of the block (element i of the buffer is block[i % block.size], rounded to `code`)"""
    from grilly_amd import _lib as L
    es = 2 if code == L.GRL_BF16 else 4
    blk = (rng.standard_normal(1 << 22) * std).astype(np.float32)
    src = core.upload(blk, code)
    dst = core.alloc(n_elems * es)
    off = 0
    while off < n_elems * es:
        m = min(blk.size * es, n_elems * es - off)
        L.check(core.lib.grl_d2d(core.ctx, dst.ptr + off, src.ptr, m))
        off += m
    core.sync()
    src.free()
    return dst, blk


def tiled(blk, start, n):
    """elements [start, start+n) of the tiled buffer fill_normal made from blk"""
    idx = (np.int64(start) + np.arange(n, dtype=np.int64)) % blk.size
    return blk[idx]


def side_workload(backend, mode, seed, reps, check=True):
    """the single-operator configurations: long causal attention with RoPE, the SwiGLU MLP, and the pre-norm encoder"""
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
        (q, qb), (k, kb), (v, vb) = (fill_normal(c, n, rng, 1.0, code) for _ in range(3))
        o = c.alloc(n * 2)
        fn = lambda: L.check(lib.grl_fa2_fwd(c.ctx, code, B, S, H, D, q.ptr, k.ptr, v.ptr, None, o.ptr,
                                             1.0 / np.sqrt(D), 1, L.ROPE_INTERLEAVED, 1e4, 1.0, None))
        ms = time_launches(c, fn, reps)
        flops = 4.0 * B * H * S * S * D * 0.5    # causal: half of the score matrix
        res = {"mode": mode, "workload": "BASELINE configs[4]: causal FA2 forward with RoPE, (B,S,H,D)=(4,8192,32,128), bf16",
               "ms": round(ms, 4), "tflops": round(flops / ms / 1e9, 1), "frac_mfma": round(flops / (ms * 1e-3) / PEAK_BF16, 4),
               "flops": flops, "includes": "every kernel the entry point launches for this call (cos/sin table, rotation, attention)", "launches": reps + WARM}
        if check:
            from oracle import oracle_np as O      # checker only
            worst = 0.0
            for (b, h, i) in [(0, 0, 0), (1, 5, 127), (2, 17, 128), (3, 31, 4097), (0, 9, 8191), (1, 30, 2049)]:
                row = lambda blk, s0, cnt: O.bf16_round(np.stack([tiled(blk, ((b * S + s) * H + h) * D, D) for s in range(s0, s0 + cnt)]))
                qr = O.truth_rope(row(qb, i, 1).reshape(1, 1, 1, D), style="interleaved", position_ids=np.array([[i]]))[0, 0, 0]
                kr = O.truth_rope(row(kb, 0, i + 1).reshape(1, i + 1, 1, D), style="interleaved")[0, :, 0]
                sc = kr @ qr / np.sqrt(D)
                pw = np.exp(sc - sc.max()); pw /= pw.sum()
                ref = pw @ row(vb, 0, i + 1).astype(np.float64)
                got = download_rows(c, o, (b * S + i) * H + h, 1, D, code)[0]
                worst = max(worst, max_rel(got, ref))
            res["max_rel_vs_float64"] = float(f"{worst:.3g}"); res["within_tolerance"] = bool(worst < TOL["bf16"])
        for t in (q, k, v, o):
            t.free()
        return res
    M, Kd, F = 16384, 4096, 11008
    x, xb = fill_normal(c, M * Kd, rng, 1.0, code)
    (wg, wgb), (wu, wub) = fill_normal(c, F * Kd, rng, 0.02, code), fill_normal(c, F * Kd, rng, 0.02, code)
    wd, wdb = fill_normal(c, Kd * F, rng, 0.02, code)
    h, y = c.alloc(M * F * 2), c.alloc(M * Kd * 2)
    f1 = lambda: L.check(lib.grl_swiglu_nt(c.ctx, code, code, M, F, Kd, x.ptr, wg.ptr, wu.ptr, None, None, h.ptr, None, None))
    f2 = lambda: L.check(lib.grl_gemm_nt(c.ctx, code, code, M, Kd, F, h.ptr, wd.ptr, None, y.ptr, 0))
    ms1, ms2 = time_launches(c, f1, reps), time_launches(c, f2, reps)
    fl1, fl2 = 4.0 * M * F * Kd, 2.0 * M * F * Kd
    res = {"mode": mode, "workload": "BASELINE configs[3]: X[16384,4096] . (W_g,W_u)[11008,4096]^T -> silu(up)*gate -> . W_d[4096,11008]^T, bf16",
           "gate_up_swiglu": {"ms": round(ms1, 4), "tflops": round(fl1 / ms1 / 1e9, 1), "frac_mfma": round(fl1 / (ms1 * 1e-3) / PEAK_BF16, 4)},
           "down": {"ms": round(ms2, 4), "tflops": round(fl2 / ms2 / 1e9, 1), "frac_mfma": round(fl2 / (ms2 * 1e-3) / PEAK_BF16, 4)},
           "total_ms": round(ms1 + ms2, 4), "tflops": round((fl1 + fl2) / (ms1 + ms2) / 1e9, 1), "flops": fl1 + fl2,
           "frac_mfma": round((fl1 + fl2) / ((ms1 + ms2) * 1e-3) / PEAK_BF16, 4), "launches_each": reps + WARM}
    if check:
        from oracle import oracle_np as O          # checker only
        r2 = np.random.default_rng(11)
        rows = np.unique(np.concatenate([[0, M - 1], r2.integers(0, M, 10)]))
        cols = np.unique(np.concatenate([[0, F - 1], r2.integers(0, F, 254)]))
        xs = O.bf16_round(np.stack([tiled(xb, int(r) * Kd, Kd) for r in rows])).astype(np.float64)
        wgs = O.bf16_round(np.stack([tiled(wgb, int(n) * Kd, Kd) for n in cols])).astype(np.float64)
        wus = O.bf16_round(np.stack([tiled(wub, int(n) * Kd, Kd) for n in cols])).astype(np.float64)
        hrows = gather_rows(c, h, rows, F, code)
        e1 = max_rel(hrows[:, cols], (xs @ wgs.T) * O.truth_silu(xs @ wus.T))
        ocols = np.unique(np.concatenate([[0, Kd - 1], r2.integers(0, Kd, 126)]))
        wds = O.bf16_round(np.stack([tiled(wdb, int(n) * F, F) for n in ocols])).astype(np.float64)
        e2 = max_rel(gather_rows(c, y, rows, Kd, code)[:, ocols], hrows.astype(np.float64) @ wds.T)
        res["gate_up_swiglu"]["max_rel_vs_float64"] = float(f"{e1:.3g}"); res["down"]["max_rel_vs_float64"] = float(f"{e2:.3g}")
        res["within_tolerance"] = bool(e1 < TOL["bf16"] and e2 < TOL["bf16"])
    for t in (x, wg, wu, wd, h, y):
        t.free()
    return res


def small_configs(backend, reps, check=True):
    """BASELINE configs[0] (the README quick-start operators, fp32: linear x[32,384].W[384,128] + 0 -> swiglu, and
    attention on (32,8,64,64) Q/K/V, no mask, scale 1/8) in microseconds, device-resident (per-launch events, median
    and mean) and numpy -> numpy through the facade (host clock around the whole call, uploads and downloads
    included, like the reference's API), and configs[1] (MiniLM-L6-shaped fp32 encoder, batch 64 x seq 256, padding
    mask with lengths uniform in [32,256]) as a device-resident forward.  Each result is checked: the operators
    against the float64 closed forms, two sequences of the encoder against the C restatement of the shaders."""
    from grilly_amd import _lib as L
    from grilly_amd import BertEncoder, random_bert_weights
    from grilly_amd.encoder import MINILM_L6
    c, lib = backend.core, backend.core.lib
    rng = np.random.default_rng(20260131 + 1)
    x = rng.standard_normal((32, 384)).astype(np.float32)
    Wt = np.ascontiguousarray(rng.standard_normal((384, 128)).astype(np.float32).T)
    b0 = np.zeros(128, np.float32)
    q, k, v = (np.ascontiguousarray(rng.standard_normal((32, 8, 64, 64)).astype(np.float32).transpose(0, 2, 1, 3)) for _ in range(3))
    dx, dw, db = c.upload(x), c.upload(Wt), c.upload(b0)
    dy, dg = c.alloc(32 * 128 * 4), c.alloc(32 * 64 * 4)
    dq, dk, dv, do = c.upload(q), c.upload(k), c.upload(v), c.alloc(q.size * 4)
    f_lin = lambda: lib.grl_gemm_nt(c.ctx, L.GRL_F32, L.GRL_F32, 32, 128, 384, dx.ptr, dw.ptr, db.ptr, dy.ptr, 0)
    f_act = lambda: lib.grl_swiglu_act(c.ctx, L.GRL_F32, 32, 64, dy.ptr, dg.ptr)
    f_fa = lambda: lib.grl_fa2_fwd(c.ctx, L.GRL_F32, 32, 64, 8, 64, dq.ptr, dk.ptr, dv.ptr, None, do.ptr, 0.125, 0, 0, 1e4, 1.0, None)
    us = lambda v: {"median_us": round(median(v) * 1e3, 2), "mean_us": round(float(np.mean(v)) * 1e3, 2), "launches": len(v)}

    def host_us(fn, n=20):
        fn(); t = []
        for _ in range(n):
            t0 = time.perf_counter(); fn(); t.append((time.perf_counter() - t0) * 1e3)
        return us(t)
    r0 = {"workload": "BASELINE configs[0]: linear x[32,384].W[384,128]+0 -> swiglu; attention Q/K/V (32,8,64,64), no mask, fp32",
          "linear": {"device_resident": us(lap_times(c, f_lin, 50)), "numpy_to_numpy": host_us(lambda: backend.fnn.linear(x, Wt, b0))},
          "activation_swiglu": {"device_resident": us(lap_times(c, f_act, 50)),
                                "numpy_to_numpy": host_us(lambda: backend.fnn.activation_swiglu(np.zeros((32, 128), np.float32)))},
          "flash_attention2": {"device_resident": us(lap_times(c, f_fa, 50)),
                               "numpy_to_numpy": host_us(lambda: backend.attention.flash_attention2(q, k, v, 8, 64, scale=0.125))}}
    if check:
        from oracle import oracle_np as O
        y = c.download(dy, (32, 128)); g = c.download(dg, (32, 64)); o = c.download(do, q.shape)
        yd = y.astype(np.float64)
        e = [max_rel(y, O.truth_linear(x, Wt, b0)), max_rel(g, yd[:, :64] * (yd[:, 64:] / (1 + np.exp(-yd[:, 64:])))),
             max_rel(o, O.truth_attention(q, k, v, scale=0.125))]
        r0["max_rel_vs_float64"] = {"linear": float(f"{e[0]:.3g}"), "activation_swiglu": float(f"{e[1]:.3g}"), "flash_attention2": float(f"{e[2]:.3g}")}
        r0["within_tolerance"] = bool(max(e) < TOL["fp32"])
    for t in (dx, dw, db, dy, dg, dq, dk, dv, do):
        t.free()
    # configs[1]
    cfg = MINILM_L6
    w = random_bert_weights(cfg, seed=20260131 + 2)
    rng = np.random.default_rng(20260131 + 2)
    B, S = 64, 256
    ids = rng.integers(0, cfg.vocab, (B, S))
    lens = rng.integers(32, 257, B)
    mask = (np.arange(S)[None] < lens[:, None]).astype(np.float32)
    enc = BertEncoder(backend, cfg, w, dtype="fp32")
    enc.set_inputs(ids, mask)
    t = lap_times(c, lambda: enc.launch(pool=True), reps, warm=3)
    flops = enc.flops_per_forward(B, S)
    r1 = {"workload": "BASELINE configs[1]: MiniLM-L6-shaped encoder forward, 6 post-LN layers, d=384, 12x32 heads, FFN 1536 GELU, fp32, "
                      "batch 64 x seq 256, lengths uniform in [32,256], embeddings + layers + masked mean pooling",
          "median_ms": round(median(t), 4), "mean_ms": round(float(np.mean(t)), 4), "steps": len(t),
          "tokens_per_s": round(B * S / median(t) * 1e3, 1), "real_tokens_per_s": round(float(lens.sum()) / median(t) * 1e3, 1),
          "flops": flops, "tflops": round(flops / median(t) / 1e9, 1), "frac_mfma": round(flops / (median(t) * 1e-3) / PEAK_FP32, 4),
          "peak": "fp32 MFMA 157.3 TFLOP/s (nominal FLOPs: padding counted)"}
    if check:
        from oracle import oracle_np as O
        O.build()
        C = O.COracle()
        h = c.download(enc.x, (B, S, cfg.d_model))
        worst = 0.0
        for bi in (int(np.argmin(lens)), 17):
            xr = C.layernorm(C.embed(ids[bi:bi + 1], w["tok_emb"], w["pos_emb"], w["type_emb"]), w["emb_ln_g"], w["emb_ln_b"], cfg.eps)
            for lw in w["layers"]:
                xr = C.bert_layer(xr, lw, mask[bi:bi + 1], cfg.heads, cfg.eps)
            worst = max(worst, max_rel(h[bi:bi + 1], xr))
        r1["max_rel_vs_cpu_port"] = float(f"{worst:.3g}"); r1["within_tolerance"] = bool(worst < TOL["fp32"])
    enc.release_activations()
    return r0, r1


def small_batch_latency(backend, weights, cfg, reps):
    """The benchmark's encoder at the other end of the batch range: one sentence and eight sentences of 128 tokens, both
    storage types, median milliseconds per forward (device-resident, no host synchronisation between forwards).  The
    launcher's small-tile choice and the encoder's choice of layer form by batch size are what these figures show."""
    from grilly_amd import BertEncoder
    rng = np.random.default_rng(11)
    out = {"workload": "BERT-base-shaped encoder forward at batch 1 and batch 8, seq 128, no padding, embeddings + layers + mean pooling"}
    for dtype in ("bf16", "fp32"):
        enc = BertEncoder(backend, cfg, weights, dtype=dtype)
        for B in (1, 8):
            ids = rng.integers(0, cfg.vocab, (B, 128))
            enc.set_inputs(ids, None)
            t = lap_times(backend.core, lambda: enc.launch(pool=True), reps, warm=5)
            out[f"{dtype}_batch{B}_median_ms"] = round(median(t), 4)
        enc.release_activations()
        del enc
    return out


def mfma_ceiling(backend, iters=20000):
    """What the matrix cores deliver under the board's power limit with nothing else going on: a register-resident loop
    of MFMAs (grl_mfma_probe: eight waves per CU, the GEMM's 128 x 64 wave tile, no memory access in the loop) for both
    bf16 instruction shapes, on all-zero operands and on N(0,1) x N(0,0.02) random ones, with the shader clock read
    beside each run.  The fractions are of the published 2.5 PFLOP/s."""
    import ctypes
    from grilly_amd import _lib as L
    c = backend.core
    rng = np.random.default_rng(3)
    blk = np.concatenate([rng.standard_normal(16384), rng.standard_normal(16384) * 0.02]).astype(np.float32)   # 32768 bf16 = 64 KiB
    rnd = c.upload(rng.permutation(blk), L.GRL_BF16)
    out = {}
    for kind, name in ((0, "v_mfma_f32_32x32x16_bf16"), (1, "v_mfma_f32_16x16x32_bf16")):
        for label, ptr in (("zero_operands", None), ("random_operands", rnd.ptr)):
            ms, fl = ctypes.c_float(), ctypes.c_double()
            L.check(c.lib.grl_mfma_probe(c.ctx, kind, ptr, iters, ctypes.byref(ms), ctypes.byref(fl)), "mfma_probe")
            c.clock_probe_begin(max(0.7 * ms.value, 0.05))
            ms2, fl2 = ctypes.c_float(), ctypes.c_double()
            L.check(c.lib.grl_mfma_probe(c.ctx, kind, ptr, iters, ctypes.byref(ms2), ctypes.byref(fl2)), "mfma_probe")
            ghz = c.clock_probe_end()
            out.setdefault(name, {})[label] = {"ms": round(ms.value, 3), "tflops": round(fl.value / ms.value / 1e9, 1),
                                               "frac_of_peak": round(fl.value / (ms.value * 1e-3) / PEAK_BF16, 4), "shader_clock_ghz": round(ghz, 3)}
    # the 32x32x16 loop again with its fragments paired in other orders (random operands): does the order matter?
    for kind, label in ((2, "one_operand_held_for_four"), (3, "serpentine_walk"), (4, "same_operand_pair_always")):
        ms, fl = ctypes.c_float(), ctypes.c_double()
        L.check(c.lib.grl_mfma_probe(c.ctx, kind, rnd.ptr, iters, ctypes.byref(ms), ctypes.byref(fl)), "mfma_probe")
        out.setdefault("v_mfma_f32_32x32x16_bf16_operand_order", {})[label] = {"ms": round(ms.value, 3), "frac_of_peak": round(fl.value / (ms.value * 1e-3) / PEAK_BF16, 4)}
    rnd.free()
    return out


def cpu_baseline(cfg, weights, ids, nseq):
    """C restatement of the reference shaders on the host cores: the first `nseq` sequences of the workload
    (S=512 each) through embeddings + all layers.  tokens/s = nseq*512 / elapsed.  Returns the record and the
    hidden states it computed (the checker for the GPU's hidden states of the same sequences)."""
    from oracle import oracle_np as O
    O.build()
    C = O.COracle()
    S = ids.shape[1]
    t0 = time.perf_counter()
    x = C.layernorm(C.embed(ids[:nseq], weights["tok_emb"], weights["pos_emb"], weights["type_emb"]),
                    weights["emb_ln_g"], weights["emb_ln_b"], cfg.eps)
    for lw in weights["layers"]:
        x = C.bert_layer(x, lw, None, cfg.heads, cfg.eps)
    dt = time.perf_counter() - t0
    rec = {"value": round(nseq * S / dt, 2), "unit": "tokens/s", "cores": C.num_threads(), "kind": "port",
           "sample": f"{nseq} of the 128 sequences x {S} tokens through embeddings + {cfg.layers} layers, fp32, "
                     f"oracle/oracle.c (one-output-per-invocation shader loops, OpenMP over rows); {dt:.1f} s"}
    return rec, x


def cpu_baseline_blas(cfg, S, rows=4096, budget_s=8.0):
    """What the reference's gemm() executes on the host (backend/fnn.py:110-124): numpy `@`, fp32, on the four
    GEMM shapes of one layer at `rows` rows; the encoder's other operators are not included, so the figure is
    an upper bound for a numpy-backed reference forward."""
    rng = np.random.default_rng(5)
    d, ff = cfg.d_model, cfg.d_ff
    shapes = [(d, 3 * d), (d, d), (d, ff), (ff, d)]
    try:
        import threadpoolctl
        threads = max((p.get("num_threads", 1) for p in threadpoolctl.threadpool_info()), default=os.cpu_count())
    except Exception:
        threads = os.cpu_count()
    per_layer = 0.0
    t_all = time.perf_counter()
    for K, N in shapes:
        a = rng.standard_normal((rows, K)).astype(np.float32)
        w = rng.standard_normal((K, N)).astype(np.float32)
        a @ w
        t0 = time.perf_counter(); reps = 0
        while reps < 3 or (time.perf_counter() - t0 < budget_s / 8 and reps < 50):
            a @ w; reps += 1
        per_layer += (time.perf_counter() - t0) / reps
    tok = rows / (per_layer * cfg.layers)
    return {"value": round(tok, 1), "unit": "tokens/s", "cores": int(threads), "kind": "reference-blas",
            "sample": f"numpy @ (OpenBLAS, fp32) on the four GEMMs of one layer at {rows} rows, x{cfg.layers} layers; attention, "
                      f"LayerNorm and GELU excluded; {time.perf_counter() - t_all:.1f} s"}


def timed_forward(backend, enc, steps, warmup):
    for _ in range(warmup):
        enc.launch(pool=True)
    backend.core.sync()
    t0 = time.perf_counter()
    backend.core.timer_start()
    for _ in range(steps):
        enc.launch(pool=True)
    ev_ms = backend.core.timer_stop()         # records the stop event and waits for it
    backend.core.sync()
    return time.perf_counter() - t0, ev_ms


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
    ap.add_argument("--no-extra", action="store_true", help="skip the fp32 forward and the two single-operator configurations")
    ap.add_argument("--mode", default="forward", choices=["forward", "gemm", "kernels", "copy", "fa2_long", "swiglu_mlp", "prenorm_forward", "small", "mfma_ceiling", "gemm_shapes"],
                    help="forward: the benchmark; gemm / copy: only launch the dominant GEMM kernel at its three "
                         "layer shapes, or a plain 1 GiB copy kernel (for rocprofv3 counter runs); kernels: every kernel of "
                         "the layer at its layer shape, nothing else (counter runs); fa2_long: "
                         "causal attention with RoPE at batch 4, 32 heads, seq 8192, head dim 128, bf16; swiglu_mlp: "
                         "X[16384,4096] through gate/up [11008,4096] + silu*up + down [4096,11008], bf16; prenorm_forward: the "
                         "pre-norm / rotary / GeGLU encoder at the ModernBERT-base shape, batch 128 x seq 512, bf16; small: the README "
                         "operators (configs[0]) in microseconds and the MiniLM-shaped fp32 encoder (configs[1]); mfma_ceiling: "
                         "register-resident MFMA loops, zero and random operands (what the power limit leaves of the matrix peak); gemm_shapes: "
                         "fused GELU linear at mid-size shapes either side of the tile choice (GRL_GEMM_VARIANT=3 / 4 forces a tile size)")
    ap.add_argument("--cpu-sequences", type=int, default=12)
    ap.add_argument("--unfused", action="store_true", help="run the seven-launch layer (two LayerNorm passes per layer) instead of the "
                    "layer with both LayerNorms folded into its GEMMs")
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
    if a.mode == "small":
        r0, r1 = small_configs(backend, a.kernel_reps, check=not a.no_cpu_baseline)
        lat = small_batch_latency(backend, random_bert_weights(cfg, seed=seed), cfg, a.kernel_reps)
        print(json.dumps({"mode": "small", "readme_ops": r0, "minilm_forward": r1, "small_batch_latency": lat}))
        backend.cleanup()
        return
    if a.mode == "gemm_shapes":
        # fused GELU linear at mid-size shapes either side of the launcher's tile choice, both storage types: median launch in
        # microseconds.  GRL_GEMM_VARIANT=3 / 4 in the environment forces 256 x 256 / 128 x 128 tiles for comparison.
        from grilly_amd import _lib as L
        c = backend.core
        rng = np.random.default_rng(0)
        shapes = [(16384, 1152, 384), (16384, 384, 384), (16384, 1536, 384), (16384, 384, 1536), (8192, 2304, 768), (8192, 768, 768),
                  (8192, 3072, 768), (8192, 768, 3072), (4096, 2304, 768), (4096, 3072, 768), (4096, 768, 3072), (2048, 3072, 768),
                  (2048, 768, 3072), (32768, 768, 768), (32768, 3072, 768), (20000, 1024, 1024), (12000, 4096, 1024)]
        res = {}
        for dt, code, es in (("fp32", L.GRL_F32, 4), ("bf16", L.GRL_BF16, 2)):
            for (M, N, K) in shapes:
                x = c.upload(rng.standard_normal((M, K)).astype(np.float32), code)
                w = c.upload((rng.standard_normal((N, K)) * 0.02).astype(np.float32), code)
                bias = c.upload(rng.standard_normal(N).astype(np.float32))
                y = c.alloc(M * N * es)
                fn = lambda: L.check(c.lib.grl_gemm_nt(c.ctx, code, code, M, N, K, x.ptr, w.ptr, bias.ptr, y.ptr, L.EPI_GELU))
                res[f"{dt} {M}x{N}x{K}"] = round(median(lap_times(c, fn, 30)) * 1e3, 1)
                for t in (x, w, bias, y):
                    t.free()
        print(json.dumps({"mode": "gemm_shapes", "forced_variant": os.environ.get("GRL_GEMM_VARIANT"), "median_us": res}))
        backend.cleanup()
        return
    if a.mode == "mfma_ceiling":
        print(json.dumps({"mode": "mfma_ceiling", "device": info, "peak_tflops": PEAK_BF16 / 1e12, "mfma_ceiling": mfma_ceiling(backend)}))
        backend.cleanup()
        return
    if a.mode in ("fa2_long", "swiglu_mlp", "prenorm_forward"):
        print(json.dumps(side_workload(backend, a.mode, seed, a.kernel_reps, check=not a.no_cpu_baseline)))
        backend.cleanup()
        return
    weights = random_bert_weights(cfg, seed=seed)
    enc = BertEncoder(backend, cfg, weights, dtype=a.dtype, fused=False if a.unfused else None)
    rng = np.random.default_rng(seed)
    B, S = a.batch, a.seq
    ids = rng.integers(0, cfg.vocab, (B, S))
    enc.set_inputs(ids, None)                 # no padding in this configuration

    if a.mode in ("gemm", "kernels"):
        only = None
        if a.mode == "gemm":        # the launches of the dominant GEMM instantiation only (counter runs)
            only = ("gemm_out_resln", "gemm_ffn2_resln") if enc.fused_now else ("gemm_qkv", "gemm_out", "gemm_ffn2")
        kt = kernel_table(backend, enc, B, S, a.kernel_reps, only=only, check=False)
        print(json.dumps({"mode": a.mode, "kernels": kt, "launches_each": a.kernel_reps + WARM}))
        backend.cleanup()
        return

    wall, ev_ms = timed_forward(backend, enc, a.steps, a.warmup)
    ms_per_step = wall * 1e3 / a.steps
    # the same steps once more with an event between every two of them: the median step next to the mean
    step_ms = lap_times(backend.core, lambda: enc.launch(pool=True), a.steps, warm=0)
    # shader clock during the forward: probe beside three more (untimed) steps
    backend.core.clock_probe_begin(max(2.0 * ms_per_step, 0.05))
    for _ in range(3):
        enc.launch(pool=True)
    fwd_clock = backend.core.clock_probe_end()
    backend.core.sync()
    tokens_per_s = B * S * a.steps / wall
    flops = enc.flops_per_forward(B, S)
    peak = PEAK_BF16 if a.dtype == "bf16" else PEAK_FP32

    out = {
        "metric": "encoder tokens/s (BERT-base, L=512)", "value": round(tokens_per_s, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": a.dtype, "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: BERT-base-shaped encoder forward, 12 post-LN layers, d=768, "
                               "12x64 heads, FFN 3072 GELU, fused QKV, no padding, random init N(0,0.02)",
                   "batch": B, "seq_len": S, "tokens_per_step": B * S, "flops_per_step": flops},
        "event_ms_per_step": round(ev_ms / a.steps, 3),
        "median_ms_per_step": round(median(step_ms), 3), "median_steps": len(step_ms),
        "model_tflops": round(flops / (ms_per_step * 1e-3) / 1e12, 1),
        "model_frac_mfma": round(flops / (ms_per_step * 1e-3) / peak, 4),
        "shader_clock_ghz_during_forward": round(fwd_clock, 3),
        "device": info,
    }
    nseq = min(a.cpu_sequences, B)
    # hidden states of the first sequences after the timed steps (the pooled output is computed from them)
    gpu_hidden = download_rows(backend.core, enc.x, 0, nseq * S, cfg.d_model, enc.code).reshape(nseq, S, cfg.d_model)
    if not a.no_kernels:
        # the layer's launches timed inside whole forwards first (the GPU is in the forward's power state), then back to back
        fk = forward_kernel_times(backend, enc, cfg)
        kt = kernel_table(backend, enc, B, S, a.kernel_reps, check=not a.no_cpu_baseline)
        out["kernels"] = kt
        for nm, r in fk.items():
            if nm in kt and kt[nm].get("flops"):
                r["frac_mfma"] = round(kt[nm]["flops"] / (r["ms"] * 1e-3) / peak, 4)
            elif nm in kt:
                r["frac_hbm"] = round(kt[nm]["bytes"] / (r["ms"] * 1e-3) / 8e12, 4)
        out["forward_kernels"] = fk
        # dominant kernel = the GEMM instantiation with the largest share of the forward.  With the LayerNorms folded
        # into the GEMMs that is the one whose epilogue adds the re-formed LayerNorm residual and reduces the row
        # statistics (out-proj and FFN2: two launches per layer); in the seven-launch layer the plain instantiation
        # (QKV, out-proj, FFN2: three launches per layer).  Average FLOPs per launch over average duration per launch,
        # the durations being those INSIDE the forward (lap events between the layer's launches); the same launches
        # timed back to back in a table of their own are reported next to it.
        fused = getattr(enc, "fused_now", False)
        names = ("gemm_out_resln", "gemm_ffn2_resln") if fused else ("gemm_qkv", "gemm_out", "gemm_ffn2")
        tname = "float" if a.dtype == "fp32" else "bf16"
        kname = f"gemm_nt_dma_kernel<{tname},{tname},256,256,2,4,{'EPI_RESLN' if fused else 'EPI_NONE'}>"
        g = [kt[k] for k in names]
        avg_flops = sum(r["flops"] for r in g) / len(g)
        fwd_ms = sum(fk[k]["ms"] for k in names) / len(names)
        fwd_med = sum(fk[k]["median_ms"] for k in names) / len(names)
        ach = avg_flops / (fwd_ms * 1e-3) / 1e12
        tab_ms = sum(r["ms"] for r in g) / len(g)
        tab_clk = sum(r["shader_clock_ghz"] for r in g) / len(g)
        tab = avg_flops / (tab_ms * 1e-3) / 1e12
        traffic, at_commit = gemm_traffic(a.dtype, B, S, kname)
        out["roofline"] = {"kernel": kname, "launches": list(names),
                           "bound": "mfma", "achieved": round(ach, 1), "peak": peak / 1e12, "unit": "TFLOP/s",
                           "frac": round(ach * 1e12 / peak, 4),
                           "traffic": traffic, "traffic_measured_at_commit": at_commit,
                           "algorithmic_bytes": sum(r["bytes"] for r in g) / len(g),
                           "avg_launch_ms": round(fwd_ms, 4), "median_launch_ms": round(fwd_med, 4),
                           "launches_timed": sum(fk[k]["n"] for k in names),
                           "flops_per_launch": avg_flops,
                           "shader_clock_ghz": round(fwd_clock, 3), "nominal_clock_ghz": NOMINAL_GHZ,
                           "frac_at_measured_clock": round(ach * 1e12 / (peak * fwd_clock / NOMINAL_GHZ), 4),
                           "launches_per_step": len(names) * cfg.layers,
                           "back_to_back": {"avg_launch_ms": round(tab_ms, 4), "median_launch_ms": round(sum(r["median_ms"] for r in g) / len(g), 4),
                                            "achieved": round(tab, 1), "frac": round(tab * 1e12 / peak, 4), "shader_clock_ghz": round(tab_clk, 3),
                                            "frac_at_measured_clock": round(tab * 1e12 / (peak * tab_clk / NOMINAL_GHZ), 4)},
                           "clock_note": "peak = 256 CUs x 4 SIMDs x 1024 bf16 FLOP per cycle (fp32: 64) x the nominal 2.4 GHz; under the board's "
                                         "power limit the launches run at shader_clock_ghz (probe kernel beside the forward, or beside the "
                                         "back-to-back launches), and frac_at_measured_clock is the same achieved rate against the peak at that clock",
                           "note": "achieved / frac / avg_launch_ms: the kernel's launches inside whole forwards (lap events between the "
                                   "layer's launches; a launch's interval includes its 3-5 us moment-merge kernel), i.e. under the sustained "
                                   "load of the timed region; back_to_back: the same launches in a table of their own (`kernels`), where "
                                   "the board often holds a higher clock because the load comes in bursts of a few milliseconds between "
                                   "host-side checks.  Both move with the box (up to 20 % between boxes)."}
        if fused:
            # the plain instantiation (what linear / fused_qkv_projection launch; the dominant kernel of the seven-launch
            # layer and of earlier measurements of this benchmark), same definition: mean FLOPs over mean duration
            gp = [kt[k] for k in ("gemm_qkv", "gemm_out", "gemm_ffn2")]
            fl, ms3 = sum(r["flops"] for r in gp) / 3, sum(r["ms"] for r in gp) / 3
            out["roofline_plain_gemm"] = {"kernel": f"gemm_nt_dma_kernel<{tname},{tname},256,256,2,4,EPI_NONE>", "launches": ["gemm_qkv", "gemm_out", "gemm_ffn2"],
                                          "achieved": round(fl / (ms3 * 1e-3) / 1e12, 1), "peak": peak / 1e12, "unit": "TFLOP/s",
                                          "frac": round(fl / (ms3 * 1e-3) / peak, 4), "avg_launch_ms": round(ms3, 4),
                                          "shader_clock_ghz": round(sum(r["shader_clock_ghz"] for r in gp) / 3, 3),
                                          "note": "not launched by the default forward (its GEMMs carry the folded LayerNorms); bench.py --unfused times the forward built from it"}
    extra = {}
    hidden32 = None
    if not a.no_extra and a.dtype == "bf16":
        enc.release_activations()
        # fp32 leg of the same configuration (BASELINE configs[2], fp32 storage and true-fp32 matrix instructions)
        enc32 = BertEncoder(backend, cfg, weights, dtype="fp32")
        enc32.set_inputs(ids, None)
        w32, _ = timed_forward(backend, enc32, 3, 1)
        ms32 = w32 * 1e3 / 3
        extra["fp32_forward"] = {"workload": "BASELINE configs[2] in fp32", "ms": round(ms32, 3), "tokens_per_s": round(B * S / ms32 * 1e3, 1),
                                 "flops": flops, "tflops": round(flops / ms32 / 1e9, 1), "frac_mfma": round(flops / (ms32 * 1e-3) / PEAK_FP32, 4),
                                 "peak": "fp32 MFMA 157.3 TFLOP/s", "steps": 3}
        hidden32 = download_rows(backend.core, enc32.x, 0, nseq * S, cfg.d_model, enc32.code).reshape(nseq, S, cfg.d_model)
        enc32.release_activations()
        del enc32
        backend.core.lib.grl_pool_trim(backend.core.ctx)
        for mode in ("swiglu_mlp", "fa2_long"):
            r = side_workload(backend, mode, seed, 10, check=not a.no_cpu_baseline)
            r.pop("mode")
            extra[mode] = r
            backend.core.lib.grl_pool_trim(backend.core.ctx)
        r0, r1 = small_configs(backend, 20, check=not a.no_cpu_baseline)
        extra["readme_ops"], extra["minilm_forward"] = r0, r1
        extra["small_batch_latency"] = small_batch_latency(backend, weights, cfg, 20)
        extra["mfma_ceiling"] = mfma_ceiling(backend)
        out["extra"] = extra
    if not a.no_cpu_baseline:
        rec, cpu_hidden = cpu_baseline(cfg, weights, ids, nseq)
        # the CPU leg's result is also the checker for the forwards timed above (same token ids, same weights)
        e16 = max_rel(gpu_hidden, cpu_hidden)
        rec["gpu_forward_max_rel_vs_cpu"] = {a.dtype: float(f"{e16:.3g}")}
        ok = e16 < (TOL[a.dtype] if a.dtype == "fp32" else 5e-2)      # bf16 storage against an unquantised fp32 run
        if hidden32 is not None:
            e32 = max_rel(hidden32, cpu_hidden)
            rec["gpu_forward_max_rel_vs_cpu"]["fp32"] = float(f"{e32:.3g}")
            ok = ok and e32 < TOL["fp32"]
            extra["fp32_forward"]["max_rel_vs_cpu_port"] = float(f"{e32:.3g}")
            extra["fp32_forward"]["within_tolerance"] = bool(e32 < TOL["fp32"])
        rec["gpu_forward_within_tolerance"] = bool(ok)
        out["cpu_baseline"] = rec
        out["cpu_baseline_blas"] = cpu_baseline_blas(cfg, S)
    backend.cleanup()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
