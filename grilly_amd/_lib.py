"""ctypes binding of libgrilly_hip.so (the C ABI declared in include/grilly_hip.h).

This is the stub a grilly maintainer would add in place of the Vulkan layer
(backend/core.py + backend/pipelines.py of the reference): it loads the shared library,
declares every entry point, and turns negative status codes into Python exceptions.
There is no fallback: if the library is missing or no gfx950 device is visible, loading or
context creation raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# GRILLY_HIP_LIB points at another build of the same library (comparing two builds on one machine)
LIB_PATH = os.environ.get("GRILLY_HIP_LIB") or os.path.join(_HERE, "lib", "libgrilly_hip.so")

GRL_F32, GRL_BF16 = 0, 1
EPI_NONE, EPI_GELU, EPI_SILU, EPI_RELU, EPI_GCU, EPI_ROSWISH = 0, 1, 2, 3, 4, 5
ROPE_NONE, ROPE_INTERLEAVED, ROPE_HALF = 0, 1, 2
ERR_ARG, ERR_SHAPE, ERR_HIP, ERR_OOM = -1, -2, -3, -4

c_void_p, c_int, c_i64, c_float, c_size_t = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t


class DevInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 64), ("compute_units", ctypes.c_int32),
                ("clock_khz", ctypes.c_int32), ("lds_bytes_per_block", ctypes.c_int32), ("wavefront", ctypes.c_int32),
                ("hbm_bytes", ctypes.c_int64)]


class PoolStats(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in ("allocations", "hits", "misses", "bytes_in_use", "bytes_cached", "bytes_peak")]


class BertLayer(ctypes.Structure):
    _fields_ = [(n, c_void_p) for n in ("w_qkv", "b_qkv", "w_o", "b_o", "ln1_g", "ln1_b", "w_ff1", "b_ff1",
                                        "w_ff2", "b_ff2", "ln2_g", "ln2_b")]


class BertLayerFused(ctypes.Structure):
    _fields_ = [(n, c_void_p) for n in ("ws_qkv", "c_qkv", "bf_qkv", "in_g", "in_b", "w_o", "b_o", "ln1_g", "ln1_b",
                                        "ws_ff1", "c_ff1", "bf_ff1", "w_ff2", "b_ff2")]


# name -> (restype, argtypes); every symbol include/grilly_hip.h declares
SIGNATURES = {
    "grl_create": (c_void_p, [c_int]),
    "grl_destroy": (None, [c_void_p]),
    "grl_last_error": (ctypes.c_char_p, []),
    "grl_device_info": (c_int, [c_void_p, ctypes.POINTER(DevInfo)]),
    "grl_stream": (c_void_p, [c_void_p]),
    "grl_malloc": (c_void_p, [c_void_p, c_size_t]),
    "grl_free": (c_int, [c_void_p, c_void_p]),
    "grl_pool_get_stats": (c_int, [c_void_p, ctypes.POINTER(PoolStats)]),
    "grl_pool_trim": (c_int, [c_void_p]),
    "grl_h2d": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "grl_d2h": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "grl_d2d": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "grl_memset": (c_int, [c_void_p, c_void_p, c_int, c_size_t]),
    "grl_sync": (c_int, [c_void_p]),
    "grl_timer_start": (c_int, [c_void_p]),
    "grl_timer_stop": (c_int, [c_void_p, ctypes.POINTER(c_float)]),
    "grl_timer_lap": (c_int, [c_void_p, c_int]),
    "grl_timer_lap_ms": (c_int, [c_void_p, c_int, c_int, ctypes.POINTER(c_float)]),
    "grl_timer_lap_trace": (c_int, [c_void_p, c_int, ctypes.POINTER(c_int)]),
    "grl_mfma_probe": (c_int, [c_void_p, c_int, c_void_p, c_int, ctypes.POINTER(c_float), ctypes.POINTER(ctypes.c_double)]),
    "grl_clock_probe_begin": (c_int, [c_void_p, c_float]),
    "grl_clock_probe_end": (c_int, [c_void_p, ctypes.POINTER(c_float)]),
    "grl_cast": (c_int, [c_void_p, c_int, c_int, c_i64, c_void_p, c_void_p]),
    "grl_gemm_plan": (c_int, [c_int, c_i64, c_i64, c_i64, c_int, c_int]),
    "grl_gemm_nt": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_void_p, c_void_p, c_int]),
    "grl_gemm_nn": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "grl_gemm_nn_noalloc": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_void_p]),
    "grl_gemm_nn_noalloc_max_bytes": (c_i64, []),
    "grl_swiglu_nt": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 8),
    "grl_glu_nt": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 8 + [c_int]),
    "grl_gemm_nt_res": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 5),
    "grl_gemm_nt_act": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 4 + [c_int, c_float, c_float]),
    "grl_fa2_fwd": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64, c_i64] + [c_void_p] * 5 + [c_float, c_int, c_int, c_float, c_float, c_void_p]),
    "grl_fa2_fwd_strided": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64, c_i64] + [c_void_p] * 5 + [c_i64] * 4 + [c_float, c_int, c_int, c_float, c_float]),
    "grl_rope": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_void_p, c_int, c_float, c_float]),
    "grl_ln_fold": (c_int, [c_void_p, c_int, c_i64, c_i64] + [c_void_p] * 7),
    "grl_ln_stats": (c_int, [c_void_p, c_int, c_i64, c_i64, c_void_p, c_float, c_void_p]),
    "grl_ln_gemm_nt": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 4 + [c_float, c_void_p, c_void_p]),
    "grl_ln_glu_nt": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 7 + [c_float, c_void_p, c_void_p, c_int]),
    "grl_ln_glu_nt_stats": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 7 + [c_void_p, c_void_p, c_int]),
    "grl_ln_gemm_nt_stats": (c_int, [c_void_p, c_int, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 6 + [c_int]),
    "grl_gemm_nt_resln_workspace": (c_i64, [c_i64, c_i64]),
    "grl_gemm_nt_resln": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64] + [c_void_p] * 8 + [c_float, c_void_p, c_void_p]),
    "grl_layernorm": (c_int, [c_void_p, c_int, c_i64, c_i64, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p]),
    "grl_add": (c_int, [c_void_p, c_int, c_i64, c_void_p, c_void_p, c_void_p]),
    "grl_gelu": (c_int, [c_void_p, c_int, c_i64, c_void_p, c_void_p]),
    "grl_silu": (c_int, [c_void_p, c_int, c_i64, c_void_p, c_void_p]),
    "grl_relu": (c_int, [c_void_p, c_int, c_i64, c_void_p, c_void_p]),
    "grl_gcu": (c_int, [c_void_p, c_int, c_i64, c_void_p, c_void_p]),
    "grl_roswish": (c_int, [c_void_p, c_int, c_i64, c_void_p, c_void_p, c_float, c_float]),
    "grl_softmax": (c_int, [c_void_p, c_int, c_i64, c_i64, c_void_p, c_void_p]),
    "grl_swiglu_act": (c_int, [c_void_p, c_int, c_i64, c_i64, c_void_p, c_void_p]),
    "grl_embed": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "grl_embed_layernorm": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_float, c_void_p]),
    "grl_mean_pool": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_void_p, c_int]),
    "grl_bert_layer_workspace": (c_i64, [c_int, c_i64, c_i64, c_i64, c_i64, c_i64]),
    "grl_bert_layer_fused_workspace": (c_i64, [c_int, c_i64, c_i64, c_i64, c_i64, c_i64]),
    "grl_bert_layer_fwd_fused": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64, c_i64, c_i64, ctypes.POINTER(BertLayerFused), c_void_p, c_float,
                                 c_void_p, c_void_p, c_void_p]),
    "grl_bert_layer_fwd": (c_int, [c_void_p, c_int, c_i64, c_i64, c_i64, c_i64, c_i64, ctypes.POINTER(BertLayer), c_void_p, c_float, c_void_p, c_void_p]),
}

_lib = None


def load():
    """Load libgrilly_hip.so and declare its entry points.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C grilly_amd/csrc` (hipcc, --offload-arch=gfx950). "
            "There is no CPU fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError here = header and library disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error():
    return load().grl_last_error().decode("utf-8", "replace")


def check(rc, what=""):
    """0 -> None; ERR_ARG/ERR_SHAPE -> ValueError; ERR_HIP -> RuntimeError; ERR_OOM -> MemoryError."""
    if rc == 0:
        return
    msg = f"{what}: {last_error()}" if what else last_error()
    if rc in (ERR_ARG, ERR_SHAPE):
        raise ValueError(msg)
    if rc == ERR_OOM:
        raise MemoryError(msg)
    raise RuntimeError(msg)
