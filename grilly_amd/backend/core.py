"""Device context and buffers: the part of the reference's VulkanCore that the hot path uses
(backend/core.py:304-421: create / upload / download buffer, dispatch + wait), on HIP.

One HipCore = one gfx950 device + one HIP stream + one caching buffer pool, all inside
libgrilly_hip.so.  numpy arrays are copied in and out; nothing here computes.
"""
import ctypes
import numpy as np

from .. import _lib as L

_DT = {"fp32": L.GRL_F32, "float32": L.GRL_F32, "f32": L.GRL_F32, "bf16": L.GRL_BF16, "bfloat16": L.GRL_BF16}


def dtype_code(dtype):
    try:
        return _DT[dtype]
    except KeyError:
        raise ValueError(f"dtype must be 'fp32' or 'bf16', got {dtype!r}") from None


def dtype_size(code):
    return 2 if code == L.GRL_BF16 else 4


class DeviceBuffer:
    """A pool-owned device allocation; returned to the pool by free() or when collected."""
    __slots__ = ("core", "ptr", "nbytes", "__weakref__")

    def __init__(self, core, nbytes):
        self.core = core
        self.nbytes = int(nbytes)
        self.ptr = core.lib.grl_malloc(core.ctx, max(self.nbytes, 1))
        if not self.ptr:
            raise MemoryError(L.last_error())

    def free(self):
        if self.ptr and self.core.ctx:
            self.core.lib.grl_free(self.core.ctx, self.ptr)
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.free()


class HipCore:
    def __init__(self, device=0):
        self.lib = L.load()
        self.ctx = self.lib.grl_create(int(device))
        if not self.ctx:
            # same exception type as the reference when its device layer is absent (backend/core.py:18-19)
            raise RuntimeError(f"HIP device not available: {L.last_error()}")
        self.device = int(device)

    # ---- lifetime
    def cleanup(self):
        if self.ctx:
            self.lib.grl_destroy(self.ctx)
            self.ctx = None

    def __del__(self):
        try:
            self.cleanup()
        except Exception:
            pass

    # ---- info
    def device_info(self):
        d = L.DevInfo()
        L.check(self.lib.grl_device_info(self.ctx, ctypes.byref(d)), "device_info")
        return {"name": d.name.decode(), "arch": d.arch.decode(), "compute_units": d.compute_units,
                "clock_khz": d.clock_khz, "lds_bytes_per_block": d.lds_bytes_per_block,
                "wavefront": d.wavefront, "hbm_bytes": d.hbm_bytes}

    def pool_stats(self):
        s = L.PoolStats()
        L.check(self.lib.grl_pool_get_stats(self.ctx, ctypes.byref(s)), "pool_stats")
        total = s.hits + s.misses
        return {"allocations": s.allocations, "hits": s.hits, "misses": s.misses, "bytes_in_use": s.bytes_in_use,
                "bytes_cached": s.bytes_cached, "bytes_peak": s.bytes_peak,
                "hit_rate": (s.hits / total) if total else 0.0}

    # ---- buffers
    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def upload(self, arr, code=L.GRL_F32):
        """numpy (any dtype, any strides) -> fresh device buffer holding fp32 or bf16 values.
        bf16 is produced on the device from the fp32 upload (round to nearest even)."""
        a = np.ascontiguousarray(arr, dtype=np.float32)
        buf = self.alloc(a.nbytes)
        L.check(self.lib.grl_h2d(self.ctx, buf.ptr, a.ctypes.data, a.nbytes), "upload")
        if code == L.GRL_BF16:
            half = self.alloc(a.size * 2)
            L.check(self.lib.grl_cast(self.ctx, L.GRL_F32, L.GRL_BF16, a.size, buf.ptr, half.ptr), "cast")
            buf.free()
            return half
        return buf

    def upload_raw(self, arr):
        """numpy array copied byte-for-byte (int32 ids, fp32 vectors, pre-packed bf16 bits)."""
        a = np.ascontiguousarray(arr)
        buf = self.alloc(a.nbytes)
        L.check(self.lib.grl_h2d(self.ctx, buf.ptr, a.ctypes.data, a.nbytes), "upload")
        return buf

    def download(self, buf, shape, code=L.GRL_F32):
        """device buffer of fp32 or bf16 values -> fresh C-contiguous float32 numpy array."""
        n = int(np.prod(shape)) if len(shape) else 1
        out = np.empty(shape, dtype=np.float32)
        if n == 0:
            return out
        if code == L.GRL_BF16:
            with self.alloc(n * 4) as full:
                L.check(self.lib.grl_cast(self.ctx, L.GRL_BF16, L.GRL_F32, n, buf.ptr, full.ptr), "cast")
                L.check(self.lib.grl_d2h(self.ctx, out.ctypes.data, full.ptr, n * 4), "download")
        else:
            L.check(self.lib.grl_d2h(self.ctx, out.ctypes.data, buf.ptr, n * 4), "download")
        return out

    def sync(self):
        L.check(self.lib.grl_sync(self.ctx), "sync")

    def timer_start(self):
        L.check(self.lib.grl_timer_start(self.ctx), "timer_start")

    def timer_stop(self):
        ms = ctypes.c_float()
        L.check(self.lib.grl_timer_stop(self.ctx, ctypes.byref(ms)), "timer_stop")
        return float(ms.value)

    def clock_probe_begin(self, millis):
        """start the shader-clock probe: it runs for `millis` (held within the library's (0, 500] ms range) beside
        whatever is enqueued next"""
        L.check(self.lib.grl_clock_probe_begin(self.ctx, min(max(float(millis), 0.05), 500.0)), "clock_probe_begin")

    def clock_probe_end(self):
        """wait for the probe; average shader clock in GHz while it ran"""
        ghz = ctypes.c_float()
        L.check(self.lib.grl_clock_probe_end(self.ctx, ctypes.byref(ghz)), "clock_probe_end")
        return float(ghz.value)
