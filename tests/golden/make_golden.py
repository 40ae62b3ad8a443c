#!/usr/bin/env python3
"""Writes tests/golden/hotpath_golden.npz: seeded inputs and expected outputs for every op of the
hot path, small enough to commit.  Expected values come from the float64 closed forms of
oracle/oracle_np.py (pinned by tests/test_oracle.py), rounded to float32; nothing of the reference
is imported or executed.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle_np as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hotpath_golden.npz")


def build():
    rng = np.random.default_rng(20260131)
    g = {}
    f32 = lambda a: np.asarray(a, np.float32)
    n = lambda *s: rng.standard_normal(s).astype(np.float32)

    # GEMM family: ragged sizes so every edge path is exercised
    x, W, b = n(37, 72), n(45, 72) * 0.2, n(45)
    g.update(lin_x=x, lin_W=W, lin_b=b, lin_y=f32(O.truth_linear(x, W, b)),
             lin_gelu=f32(O.truth_linear(x, W, b, "gelu")), lin_silu=f32(O.truth_linear(x, W, b, "silu")))
    Wg, Wu, bg, bu = n(40, 72) * 0.2, n(40, 72) * 0.2, n(40), n(40)
    out, gate, up = O.truth_fused_swiglu(x, Wg, Wu, bg, bu)
    g.update(sw_Wg=Wg, sw_Wu=Wu, sw_bg=bg, sw_bu=bu, sw_out=f32(out), sw_gate=f32(gate), sw_up=f32(up))
    B_ = n(72, 29)
    g.update(gemm_B=B_, gemm_C=f32(O.truth_gemm(x, B_)))

    # attention: (B,S,H,D) with a key-padding mask, causal, and both RoPE styles
    q, k, v = n(2, 70, 2, 32), n(2, 70, 2, 32), n(2, 70, 2, 32)
    m = (np.arange(70)[None] < np.array([70, 41])[:, None]).astype(np.float32)
    g.update(att_q=q, att_k=k, att_v=v, att_mask=m,
             att_plain=f32(O.truth_attention(q, k, v)), att_masked=f32(O.truth_attention(q, k, v, mask=m)),
             att_causal=f32(O.truth_attention(q, k, v, causal=True)),
             att_rope_i=f32(O.truth_attention(q, k, v, causal=True, rope="interleaved")),
             att_rope_h=f32(O.truth_attention(q, k, v, rope="half")),
             rope_half=f32(O.truth_rope(q, style="half")), rope_inter=f32(O.truth_rope(q, style="interleaved")))

    # row / element kernels
    xr, res, gam, bet = n(9, 384) * 2 + 0.5, n(9, 384), 1 + 0.1 * n(384), 0.1 * n(384)
    e = (n(300) * 20).astype(np.float32)
    g.update(ln_x=xr, ln_res=res, ln_g=gam, ln_b=bet, ln_y=f32(O.truth_layernorm(xr, gam, bet)),
             ln_res_y=f32(O.truth_layernorm(xr, gam, bet, residual=res)),
             ew_x=e, ew_gelu=f32(O.truth_gelu(e)), ew_silu=f32(O.truth_silu(e)),
             ew_swiglu=f32(O.truth_swiglu_act(xr)))

    # one post-LN encoder layer (d=64, 2 heads x 32, FFN 128)
    d, ff, H = 64, 128, 2
    w = {"w_qkv": n(3 * d, d) * 0.1, "b_qkv": n(3 * d) * 0.1, "w_o": n(d, d) * 0.1, "b_o": n(d) * 0.1,
         "ln1_g": 1 + 0.1 * n(d), "ln1_b": 0.1 * n(d), "w_ff1": n(ff, d) * 0.1, "b_ff1": n(ff) * 0.1,
         "w_ff2": n(d, ff) * 0.1, "b_ff2": n(d) * 0.1, "ln2_g": 1 + 0.1 * n(d), "ln2_b": 0.1 * n(d)}
    xl = n(2, 24, d)
    ml = (np.arange(24)[None] < np.array([24, 13])[:, None]).astype(np.float32)
    g.update({f"layer_{k_}": v_ for k_, v_ in w.items()})
    g.update(layer_x=xl, layer_mask=ml, layer_y=f32(O.truth_bert_layer(xl, w, ml, H)))

    # further epilogues on the same inputs (appended last so that the arrays above keep their values)
    g.update(lin_relu=f32(O.truth_linear(x, W, b, "relu")), lin_gcu=f32(O.truth_linear(x, W, b, "gcu")),
             lin_roswish=f32(O.truth_linear(x, W, b, "roswish", 0.7, 1.3)),
             glu_relu=f32(O.truth_fused_glu(x, Wg, Wu, bg, bu, "relu")[0]),
             glu_gelu=f32(O.truth_fused_glu(x, Wg, Wu, bg, bu, "gelu")[0]),
             ew_relu=f32(np.maximum(e, 0)))
    Wl, bl = n(20, 384) * 0.1, n(20)
    g.update(lnlin_W=Wl, lnlin_b=bl, lnlin_y=f32(O.truth_linear(O.truth_layernorm(xr, gam, bet), Wl, bl)))
    return g


if __name__ == "__main__":
    g = build()
    np.savez_compressed(OUT, **g)
    print(f"wrote {OUT}: {len(g)} arrays, {os.path.getsize(OUT)} bytes")
