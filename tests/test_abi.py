"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, the ctypes table covers exactly those symbols, and without a GPU the entry points
fail loudly (no fallback)."""
import ctypes
import os
import re

import numpy as np
import pytest

from grilly_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "grilly_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(grl_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = L.load()
    syms = header_symbols()
    assert len(syms) >= 30
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in include/grilly_hip.h but not exported"


def test_ctypes_table_matches_header():
    assert sorted(L.SIGNATURES) == header_symbols()


def test_struct_layouts():
    assert ctypes.sizeof(L.BertLayer) == 12 * ctypes.sizeof(ctypes.c_void_p)
    assert ctypes.sizeof(L.PoolStats) == 6 * 8
    assert ctypes.sizeof(L.DevInfo) == 128 + 64 + 4 * 4 + 8


def test_workspace_size_is_pure_host_arithmetic():
    lib = L.load()
    B, S, H, D, ff = 4, 128, 12, 64, 3072
    M, d = B * S, H * D
    got = lib.grl_bert_layer_workspace(L.GRL_BF16, B, S, H, D, ff)
    assert got >= M * (3 * d + 2 * d + ff) * 2 and got % 256 == 0
    assert lib.grl_bert_layer_workspace(7, B, S, H, D, ff) == -1


def test_null_context_is_rejected_not_crashed():
    lib = L.load()
    rc = lib.grl_gemm_nt(None, 0, 0, 4, 4, 4, None, None, None, None, 0)
    assert rc == L.ERR_ARG and "null context" in L.last_error()
    with pytest.raises(ValueError):
        L.check(rc, "gemm")
    assert lib.grl_sync(None) == L.ERR_ARG
    assert lib.grl_malloc(None, 16) is None


def _has_gpu():
    lib = L.load()
    ctx = lib.grl_create(0)
    if ctx:
        lib.grl_destroy(ctx)
        return True
    return False


def test_no_device_fails_loudly():
    if _has_gpu():
        pytest.skip("a device is present")
    import grilly_amd
    with pytest.raises(RuntimeError, match="HIP device not available"):
        grilly_amd.Compute()


def test_product_does_not_import_oracle():
    # the shipped package must never reach into oracle/
    for dirpath, _, files in os.walk(os.path.join(ROOT, "grilly_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", "Makefile")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.lower(), f"{f} mentions the oracle"


def test_dtype_codes_and_encoder_config():
    from grilly_amd.backend.core import dtype_code
    from grilly_amd.encoder import EncoderConfig, random_bert_weights, MINILM_L6
    assert dtype_code("fp32") == 0 and dtype_code("bf16") == 1
    with pytest.raises(ValueError):
        dtype_code("fp16")
    cfg = EncoderConfig(layers=2, d_model=64, heads=2, d_ff=128, vocab=100, max_pos=32)
    w = random_bert_weights(cfg, seed=1)
    assert len(w["layers"]) == 2 and w["layers"][0]["w_qkv"].shape == (192, 64) and w["layers"][0]["w_ff2"].shape == (64, 128)
    assert abs(float(w["tok_emb"].std()) - 0.02) < 2e-3
    assert MINILM_L6.head_dim == 32


def test_gemm_tile_choice_for_the_benchmark_shapes():
    """grl_gemm_plan is the launcher's tile choice as host arithmetic: the benchmark's shapes (65536 rows: whole passes
    of 256 x 256 tiles over 256 CUs) and the SwiGLU MLP stay on the persistent big-tile kernel, the MiniLM-shaped
    GEMMs whose big tiles would leave the last pass mostly empty get 128 x 128 tiles, README-sized problems 64 x 64
    tiles, and a K that is not a whole number of 128-byte slabs the register-staged kernels."""
    lib = L.load()
    plan = lambda dt, M, N, K, dual=0, cus=256: lib.grl_gemm_plan(dt, M, N, K, dual, cus)
    for dt in (L.GRL_BF16, L.GRL_F32):
        for (N, K) in [(2304, 768), (768, 768), (3072, 768), (768, 3072)]:
            assert plan(dt, 65536, N, K) == 3, (dt, N, K)
    assert plan(L.GRL_BF16, 16384, 11008, 4096, dual=1) == 3 and plan(L.GRL_BF16, 16384, 4096, 11008) == 3
    assert plan(L.GRL_BF16, 65536, 1152, 768, dual=1) == 3                  # the pre-norm encoder's gated GEMM
    # 16384 x 1152: 320 big tiles = two passes, the second a quarter full; 1152 small tiles = two full passes and a bit
    assert plan(L.GRL_F32, 16384, 1152, 384) == 4 and plan(L.GRL_F32, 16384, 1536, 384) == 4
    assert plan(L.GRL_F32, 16384, 384, 384) == 4                             # below 192 big tiles: always small
    assert plan(L.GRL_BF16, 8192, 2304, 768) == 4 and plan(L.GRL_BF16, 32768, 3072, 768) == 3
    # small batches: 64 x 64 tiles up to one per CU in bf16, four per CU in fp32
    assert plan(L.GRL_F32, 32, 128, 384) == 5 and plan(L.GRL_BF16, 128, 2304, 768) == 5 and plan(L.GRL_BF16, 128, 768, 768) == 5
    assert plan(L.GRL_BF16, 1024, 768, 3072) == 5 and plan(L.GRL_BF16, 1024, 2304, 768) == 4
    assert plan(L.GRL_F32, 1024, 3072, 768) == 5 and plan(L.GRL_F32, 2048, 3072, 768) == 4
    assert plan(L.GRL_F32, 4096, 4096, 1000) == 1 and plan(L.GRL_F32, 4096, 2048, 1000) == 2      # K tail: register-staged
    assert plan(L.GRL_F32, 0, 8, 8) == L.ERR_ARG and plan(7, 8, 8, 8) == L.ERR_ARG and plan(L.GRL_F32, 8, 8, 8, cus=0) == L.ERR_ARG
