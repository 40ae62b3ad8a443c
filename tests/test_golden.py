"""Committed golden vectors (tests/golden/hotpath_golden.npz, written by tests/golden/make_golden.py).
CPU: the generator is reproducible and the C oracle (fp32, shader order) agrees with the stored float64-derived
values.  GPU: the HIP path, through the numpy facade and the C ABI, matches the stored values."""
import os

import numpy as np
import pytest

from conftest import TOL_F32
from oracle import oracle_np as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hotpath_golden.npz"))


def layer_weights():
    return {k[len("layer_"):]: G[k] for k in G.files if k.startswith("layer_") and k not in ("layer_x", "layer_mask", "layer_y")}


def test_generator_is_reproducible():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(os.path.dirname(__file__), "golden", "make_golden.py"))
    mod = importlib.util.module_from_spec(spec); spec.loader.exec_module(mod)
    fresh = mod.build()
    assert sorted(fresh) == sorted(G.files)
    for k in G.files:
        np.testing.assert_allclose(fresh[k], G[k], rtol=1e-6, atol=1e-7, err_msg=k)


def test_c_oracle_matches_golden(corc):
    x = G["lin_x"]
    assert O.max_rel(corc.linear(x, G["lin_W"], G["lin_b"]), G["lin_y"]) < 1e-5
    assert O.max_rel(corc.linear(x, G["lin_W"], G["lin_b"], "gelu"), G["lin_gelu"]) < 1e-5
    assert O.max_rel(corc.linear(x, G["lin_W"], G["lin_b"], "silu"), G["lin_silu"]) < 1e-5
    out, g, u = corc.fused_swiglu(x, G["sw_Wg"], G["sw_Wu"], G["sw_bg"], G["sw_bu"])
    assert O.max_rel(out, G["sw_out"]) < 1e-5 and O.max_rel(g, G["sw_gate"]) < 1e-5 and O.max_rel(u, G["sw_up"]) < 1e-5
    assert O.max_rel(corc.gemm(x, G["gemm_B"]), G["gemm_C"]) < 1e-5
    q, k, v, m = G["att_q"], G["att_k"], G["att_v"], G["att_mask"]
    assert O.max_rel(corc.attention(q, k, v), G["att_plain"]) < 1e-5
    assert O.max_rel(corc.attention(q, k, v, mask=m), G["att_masked"]) < 1e-5
    assert O.max_rel(corc.attention(q, k, v, causal=True), G["att_causal"]) < 1e-5
    assert O.max_rel(corc.attention(q, k, v, causal=True, rope="interleaved"), G["att_rope_i"]) < 1e-5
    assert O.max_rel(corc.attention(q, k, v, rope="half"), G["att_rope_h"]) < 1e-5
    assert O.max_rel(corc.rope(q, "half"), G["rope_half"]) < 1e-5
    assert O.max_rel(corc.layernorm(G["ln_x"], G["ln_g"], G["ln_b"]), G["ln_y"]) < 1e-5
    assert O.max_rel(corc.layernorm(G["ln_x"], G["ln_g"], G["ln_b"], residual=G["ln_res"]), G["ln_res_y"]) < 1e-5
    assert O.max_rel(corc.gelu(G["ew_x"]), G["ew_gelu"]) < 1e-5
    assert O.max_rel(corc.silu(G["ew_x"]), G["ew_silu"]) < 1e-5
    assert O.max_rel(corc.swiglu_act(G["ln_x"]), G["ew_swiglu"]) < 1e-5
    assert O.max_rel(corc.bert_layer(G["layer_x"], layer_weights(), G["layer_mask"], 2), G["layer_y"]) < 1e-5
    assert O.max_rel(corc.linear(x, G["lin_W"], G["lin_b"], "relu"), G["lin_relu"]) < 1e-5
    assert O.max_rel(corc.linear(x, G["lin_W"], G["lin_b"], "gcu"), G["lin_gcu"]) < 1e-5
    assert O.max_rel(corc.linear(x, G["lin_W"], G["lin_b"], "roswish", 0.7, 1.3), G["lin_roswish"]) < 1e-5
    assert O.max_rel(corc.fused_glu(x, G["sw_Wg"], G["sw_Wu"], G["sw_bg"], G["sw_bu"], "relu")[0], G["glu_relu"]) < 1e-5
    assert O.max_rel(corc.fused_glu(x, G["sw_Wg"], G["sw_Wu"], G["sw_bg"], G["sw_bu"], "gelu")[0], G["glu_gelu"]) < 1e-5
    assert O.max_rel(corc.linear(corc.layernorm(G["ln_x"], G["ln_g"], G["ln_b"]), G["lnlin_W"], G["lnlin_b"]), G["lnlin_y"]) < 1e-5


@pytest.mark.gpu
def test_hip_path_matches_golden(backend):
    f, a = backend.fnn, backend.attention
    x = G["lin_x"]
    assert O.max_rel(f.linear(x, G["lin_W"], G["lin_b"]), G["lin_y"]) < TOL_F32
    assert O.max_rel(f.fused_linear_gelu(x, G["lin_W"], G["lin_b"]), G["lin_gelu"]) < TOL_F32
    assert O.max_rel(f.fused_linear_silu(x, G["lin_W"], G["lin_b"]), G["lin_silu"]) < TOL_F32
    out, g, u = f.fused_swiglu(x, G["sw_Wg"], G["sw_Wu"], G["sw_bg"], G["sw_bu"], return_cache=True)
    assert O.max_rel(out, G["sw_out"]) < TOL_F32 and O.max_rel(g, G["sw_gate"]) < TOL_F32 and O.max_rel(u, G["sw_up"]) < TOL_F32
    assert O.max_rel(f.gemm(x, G["gemm_B"]), G["gemm_C"]) < TOL_F32
    q, k, v, m = G["att_q"], G["att_k"], G["att_v"], G["att_mask"]
    assert O.max_rel(a.flash_attention2(q, k, v, 2, 32), G["att_plain"]) < TOL_F32
    assert O.max_rel(a.flash_attention2(q, k, v, 2, 32, mask=m), G["att_masked"]) < TOL_F32
    assert O.max_rel(a.flash_attention2(q, k, v, 2, 32, causal=True), G["att_causal"]) < TOL_F32
    assert O.max_rel(a.flash_attention2_rope(q, k, v, 2, 32, causal=True), G["att_rope_i"]) < TOL_F32
    assert O.max_rel(a.flash_attention2_rope(q, k, v, 2, 32, rope_style="half"), G["att_rope_h"]) < TOL_F32
    assert O.max_rel(a.apply_rope(q), G["rope_half"]) < TOL_F32
    assert O.max_rel(a.apply_rope(q, rope_style="interleaved"), G["rope_inter"]) < TOL_F32
    assert O.max_rel(f.layernorm(G["ln_x"], G["ln_g"], G["ln_b"]), G["ln_y"]) < TOL_F32
    assert O.max_rel(f.activation_gelu(G["ew_x"]), G["ew_gelu"]) < TOL_F32
    assert O.max_rel(f.activation_silu(G["ew_x"]), G["ew_silu"]) < TOL_F32
    assert O.max_rel(f.activation_swiglu(G["ln_x"]), G["ew_swiglu"]) < TOL_F32
    assert O.max_rel(f.fused_linear_relu(x, G["lin_W"], G["lin_b"]), G["lin_relu"]) < TOL_F32
    assert O.max_rel(f.fused_linear_gcu(x, G["lin_W"], G["lin_b"]), G["lin_gcu"]) < TOL_F32
    assert O.max_rel(f.fused_linear_roswish(x, G["lin_W"], G["lin_b"], alpha=0.7, beta=1.3), G["lin_roswish"]) < TOL_F32
    assert O.max_rel(f.fused_reglu(x, G["sw_Wg"], G["sw_Wu"], G["sw_bg"], G["sw_bu"]), G["glu_relu"]) < TOL_F32
    assert O.max_rel(f.fused_geglu(x, G["sw_Wg"], G["sw_Wu"], G["sw_bg"], G["sw_bu"]), G["glu_gelu"]) < TOL_F32
    np.testing.assert_array_equal(f.activation_relu(G["ew_x"]), G["ew_relu"])
    assert O.max_rel(f.fused_layernorm_linear(G["ln_x"], G["ln_g"], G["ln_b"], G["lnlin_W"], G["lnlin_b"]), G["lnlin_y"]) < TOL_F32
    # the encoder layer through the device-pointer entry point
    import ctypes
    from grilly_amd import _lib as L
    c = backend.core
    w = layer_weights()
    keep, s = [], L.BertLayer()
    for kk, vv in w.items():
        buf = c.upload(vv.reshape(-1) if vv.ndim == 1 else vv); keep.append(buf); setattr(s, kk, buf.ptr)
    xl, ml = G["layer_x"], G["layer_mask"]
    B, S, d = xl.shape
    dx, dm = c.upload(xl), c.upload(ml)
    ws = c.alloc(c.lib.grl_bert_layer_workspace(L.GRL_F32, B, S, 2, 32, 128))
    L.check(c.lib.grl_bert_layer_fwd(c.ctx, L.GRL_F32, B, S, 2, 32, 128, ctypes.byref(s), dm.ptr, 1e-5, dx.ptr, ws.ptr))
    assert O.max_rel(c.download(dx, xl.shape), G["layer_y"]) < TOL_F32
    for t in keep + [dx, dm, ws]:
        t.free()
