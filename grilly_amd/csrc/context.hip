// Context, caching device-buffer pool, copies and the event stopwatch.
#include "common.hpp"
#include <cstring>

static thread_local char g_err[512] = "";

int grl_gemm_scratch_init(grl_ctx* c);    // gemm.hip: device address of the static scratch of grl_gemm_nn_noalloc

void grl_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char* grl_last_error(void) { return g_err; }

extern "C" grl_ctx* grl_create(int device) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        grl_set_error("no HIP device visible (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
        return nullptr;
    }
    if (device < 0 || device >= n) {
        grl_set_error("device %d out of range (0..%d)", device, n - 1);
        return nullptr;
    }
    grl_ctx* c = new grl_ctx();
    c->device = device;
    if ((e = hipSetDevice(device)) != hipSuccess ||
        (e = hipGetDeviceProperties(&c->prop, device)) != hipSuccess ||
        (e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking)) != hipSuccess ||
        (e = hipEventCreate(&c->ev0)) != hipSuccess ||
        (e = hipEventCreate(&c->ev1)) != hipSuccess) {
        grl_set_error("context creation failed: %s", hipGetErrorString(e));
        delete c;
        return nullptr;
    }
    if (strncmp(c->prop.gcnArchName, "gfx950", 6) != 0) {
        grl_set_error("device %d is %s; this library carries gfx950 code only", device, c->prop.gcnArchName);
        hipStreamDestroy(c->stream);
        delete c;
        return nullptr;
    }
    if (grl_gemm_scratch_init(c) != GRL_OK) {      // message already set
        hipStreamDestroy(c->stream);
        delete c;
        return nullptr;
    }
    return c;
}

extern "C" void grl_destroy(grl_ctx* c) {
    if (!c) return;
    hipSetDevice(c->device);
    hipStreamSynchronize(c->stream);
    for (auto& kv : c->free_blocks)
        for (void* p : kv.second) hipFree(p);
    for (auto& kv : c->live) hipFree(kv.first);
    hipEventDestroy(c->ev0);
    hipEventDestroy(c->ev1);
    for (auto& e : c->laps) if (e) hipEventDestroy(e);
    if (c->probe_stream) { hipStreamSynchronize(c->probe_stream); hipStreamDestroy(c->probe_stream); }
    if (c->probe_out) hipFree(c->probe_out);
    if (c->stage) hipHostFree(c->stage);
    hipStreamDestroy(c->stream);
    delete c;
}

extern "C" void* grl_stream(grl_ctx* c) { return c ? (void*)c->stream : nullptr; }

extern "C" int grl_device_info(grl_ctx* c, grl_devinfo* out) {
    GRL_REQUIRE(c && out, GRL_ERR_ARG, "grl_device_info: null argument");
    memset(out, 0, sizeof(*out));
    strncpy(out->name, c->prop.name, sizeof(out->name) - 1);
    strncpy(out->arch, c->prop.gcnArchName, sizeof(out->arch) - 1);
    out->compute_units = c->prop.multiProcessorCount;
    out->clock_khz = c->prop.clockRate;
    out->lds_bytes_per_block = (int32_t)c->prop.sharedMemPerBlock;
    out->wavefront = c->prop.warpSize;
    out->hbm_bytes = (int64_t)c->prop.totalGlobalMem;
    return GRL_OK;
}

// ---------------------------------------------------------------- pool
// Buckets are powers of two from 256 B; blocks above 1 GiB round to a multiple of
// 256 MiB instead so a 3 GiB activation does not pin 4 GiB.
static size_t bucket_of(size_t bytes) {
    if (bytes <= 256) return 256;
    const size_t big = (size_t)1 << 30, step = (size_t)256 << 20;
    if (bytes > big) return (bytes + step - 1) / step * step;
    size_t b = 256;
    while (b < bytes) b <<= 1;
    return b;
}

extern "C" void* grl_malloc(grl_ctx* c, size_t bytes) {
    if (!c) { grl_set_error("grl_malloc: null context"); return nullptr; }
    if (bytes == 0) bytes = 1;
    size_t b = bucket_of(bytes);
    std::lock_guard<std::mutex> lk(c->mu);
    void* p = nullptr;
    auto it = c->free_blocks.find(b);
    if (it != c->free_blocks.end() && !it->second.empty()) {
        p = it->second.back();
        it->second.pop_back();
        c->stats.hits++;
        c->stats.bytes_cached -= (int64_t)b;
    } else {
        hipSetDevice(c->device);
        hipError_t e = hipMalloc(&p, b);
        if (e != hipSuccess) {
            // drop the cache and retry once before reporting out-of-memory
            (void)hipGetLastError();
            hipStreamSynchronize(c->stream);
            for (auto& kv : c->free_blocks) {
                for (void* q : kv.second) hipFree(q);
                kv.second.clear();
            }
            c->stats.bytes_cached = 0;
            e = hipMalloc(&p, b);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                grl_set_error("grl_malloc: hipMalloc(%zu) failed: %s", b, hipGetErrorString(e));
                return nullptr;
            }
        }
        c->stats.misses++;
        c->stats.allocations++;
    }
    c->live[p] = b;
    c->stats.bytes_in_use += (int64_t)b;
    if (c->stats.bytes_in_use > c->stats.bytes_peak) c->stats.bytes_peak = c->stats.bytes_in_use;
    return p;
}

extern "C" int grl_free(grl_ctx* c, void* p) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_free: null context");
    if (!p) return GRL_OK;
    std::lock_guard<std::mutex> lk(c->mu);
    auto it = c->live.find(p);
    GRL_REQUIRE(it != c->live.end(), GRL_ERR_ARG, "grl_free: pointer %p was not allocated by this context", p);
    size_t b = it->second;
    c->live.erase(it);
    c->free_blocks[b].push_back(p);
    c->stats.bytes_in_use -= (int64_t)b;
    c->stats.bytes_cached += (int64_t)b;
    return GRL_OK;
}

extern "C" int grl_pool_get_stats(grl_ctx* c, grl_pool_stats* out) {
    GRL_REQUIRE(c && out, GRL_ERR_ARG, "grl_pool_get_stats: null argument");
    std::lock_guard<std::mutex> lk(c->mu);
    *out = c->stats;
    return GRL_OK;
}

extern "C" int grl_pool_trim(grl_ctx* c) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_pool_trim: null context");
    GRL_CHECK_HIP(hipStreamSynchronize(c->stream));
    std::lock_guard<std::mutex> lk(c->mu);
    for (auto& kv : c->free_blocks) {
        for (void* q : kv.second) hipFree(q);
        kv.second.clear();
    }
    c->stats.bytes_cached = 0;
    return GRL_OK;
}

// ---------------------------------------------------------------- copies
// Host -> device.  Returns when the caller's buffer has been consumed; the transfer is ordered on the context stream like
// a kernel launch (work enqueued later on this context sees the data, grl_sync / grl_d2h wait for it).  Copies of up to
// 4 MiB go through a pinned staging ring (one memcpy, then a truly asynchronous transfer: no wait per upload, which is
// most of the cost of a small numpy -> numpy operator call); larger ones are handed to the runtime and waited for.
static constexpr size_t GRL_STAGE_MAX = 4u << 20, GRL_STAGE_RING = 32u << 20;
extern "C" int grl_h2d(grl_ctx* c, void* dst, const void* src, size_t bytes) {
    GRL_REQUIRE(c && (bytes == 0 || (dst && src)), GRL_ERR_ARG, "grl_h2d: null argument");
    if (!bytes) return GRL_OK;
    if (bytes <= GRL_STAGE_MAX) {
        std::lock_guard<std::mutex> lk(c->stage_mu);
        if (!c->stage && !c->stage_failed) {
            GRL_CHECK_HIP(hipSetDevice(c->device));
            void* p = nullptr;
            if (hipHostMalloc(&p, GRL_STAGE_RING, hipHostMallocDefault) == hipSuccess) { c->stage = (char*)p; c->stage_cap = GRL_STAGE_RING; }
            else { (void)hipGetLastError(); c->stage_failed = true; }
        }
        if (c->stage) {
            if (c->stage_off + bytes > c->stage_cap) {
                GRL_CHECK_HIP(hipStreamSynchronize(c->stream));      // every earlier transfer has left the ring
                c->stage_off = 0;
            }
            char* slot = c->stage + c->stage_off;
            memcpy(slot, src, bytes);
            GRL_CHECK_HIP(hipMemcpyAsync(dst, slot, bytes, hipMemcpyHostToDevice, c->stream));
            c->stage_off += (bytes + 255) & ~(size_t)255;
            return GRL_OK;
        }
    }
    GRL_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, c->stream));
    GRL_CHECK_HIP(hipStreamSynchronize(c->stream));
    return GRL_OK;
}
extern "C" int grl_d2h(grl_ctx* c, void* dst, const void* src, size_t bytes) {
    GRL_REQUIRE(c && (bytes == 0 || (dst && src)), GRL_ERR_ARG, "grl_d2h: null argument");
    if (!bytes) return GRL_OK;
    GRL_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, c->stream));
    GRL_CHECK_HIP(hipStreamSynchronize(c->stream));
    return GRL_OK;
}
int grl_copy_kernel_launch(grl_ctx* c, void* dst, const void* src, size_t bytes);

extern "C" int grl_d2d(grl_ctx* c, void* dst, const void* src, size_t bytes) {
    GRL_REQUIRE(c && (bytes == 0 || (dst && src)), GRL_ERR_ARG, "grl_d2d: null argument");
    if (!bytes) return GRL_OK;
    // a plain copy kernel when everything is 16-byte granular (ordinary kernel launch on the
    // context stream), else the runtime's copy
    if ((((uintptr_t)dst | (uintptr_t)src | bytes) & 15u) == 0) return grl_copy_kernel_launch(c, dst, src, bytes);
    GRL_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, c->stream));
    return GRL_OK;
}
extern "C" int grl_memset(grl_ctx* c, void* dst, int byte, size_t bytes) {
    GRL_REQUIRE(c && (bytes == 0 || dst), GRL_ERR_ARG, "grl_memset: null argument");
    if (!bytes) return GRL_OK;
    GRL_CHECK_HIP(hipMemsetAsync(dst, byte, bytes, c->stream));
    return GRL_OK;
}
extern "C" int grl_sync(grl_ctx* c) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_sync: null context");
    GRL_CHECK_HIP(hipStreamSynchronize(c->stream));
    return GRL_OK;
}

extern "C" int grl_timer_start(grl_ctx* c) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_timer_start: null context");
    std::lock_guard<std::mutex> lk(c->timer_mu);      // one event pair per context: calls are serialised, timings are not nestable
    GRL_CHECK_HIP(hipEventRecord(c->ev0, c->stream));
    return GRL_OK;
}
extern "C" int grl_timer_stop(grl_ctx* c, float* ms) {
    GRL_REQUIRE(c && ms, GRL_ERR_ARG, "grl_timer_stop: null argument");
    std::lock_guard<std::mutex> lk(c->timer_mu);
    GRL_CHECK_HIP(hipEventRecord(c->ev1, c->stream));
    GRL_CHECK_HIP(hipEventSynchronize(c->ev1));
    GRL_CHECK_HIP(hipEventElapsedTime(ms, c->ev0, c->ev1));
    return GRL_OK;
}

// ---- lap events: per-launch durations of a back-to-back sequence without a host synchronisation in between -----
extern "C" int grl_timer_lap(grl_ctx* c, int index) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_timer_lap: null context");
    GRL_REQUIRE(index >= 0 && index < GRL_MAX_LAPS, GRL_ERR_ARG, "grl_timer_lap: index %d outside 0..%d", index, GRL_MAX_LAPS - 1);
    std::lock_guard<std::mutex> lk(c->timer_mu);
    if (!c->laps[index]) {
        GRL_CHECK_HIP(hipSetDevice(c->device));
        GRL_CHECK_HIP(hipEventCreate(&c->laps[index]));
    }
    GRL_CHECK_HIP(hipEventRecord(c->laps[index], c->stream));
    return GRL_OK;
}
extern "C" int grl_timer_lap_ms(grl_ctx* c, int from, int to, float* ms) {
    GRL_REQUIRE(c && ms, GRL_ERR_ARG, "grl_timer_lap_ms: null argument");
    GRL_REQUIRE(from >= 0 && from < GRL_MAX_LAPS && to >= 0 && to < GRL_MAX_LAPS, GRL_ERR_ARG, "grl_timer_lap_ms: index outside 0..%d", GRL_MAX_LAPS - 1);
    std::lock_guard<std::mutex> lk(c->timer_mu);
    GRL_REQUIRE(c->laps[from] && c->laps[to], GRL_ERR_ARG, "grl_timer_lap_ms: lap %d or %d was never recorded", from, to);
    GRL_CHECK_HIP(hipEventSynchronize(c->laps[to]));
    GRL_CHECK_HIP(hipEventElapsedTime(ms, c->laps[from], c->laps[to]));
    return GRL_OK;
}

// lap trace: the multi-launch entry points (the encoder layers) record lap first, first+1, ... after each of their launches
extern "C" int grl_timer_lap_trace(grl_ctx* c, int first, int* next) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_timer_lap_trace: null context");
    GRL_REQUIRE(first >= -1 && first < GRL_MAX_LAPS, GRL_ERR_ARG, "grl_timer_lap_trace: first index %d outside -1..%d", first, GRL_MAX_LAPS - 1);
    int old;
    {
        std::lock_guard<std::mutex> lk(c->timer_mu);
        old = c->lap_next;
        c->lap_next = -1;
    }
    if (next) *next = old;
    if (first < 0) return GRL_OK;
    int rc = grl_timer_lap(c, first);          // the trace starts with a lap of its own: index `first`
    if (rc) return rc;
    std::lock_guard<std::mutex> lk(c->timer_mu);
    c->lap_next = first + 1;
    return GRL_OK;
}
void grl_lap_mark(grl_ctx* c) {
    int idx;
    {
        std::lock_guard<std::mutex> lk(c->timer_mu);
        if (c->lap_next < 0 || c->lap_next >= GRL_MAX_LAPS) return;
        idx = c->lap_next++;
    }
    grl_timer_lap(c, idx);
}

// ---- matrix-core ceiling probe ---------------------------------------------------------------------------------
// Nothing but MFMAs on register-resident operands: eight waves per CU (two per SIMD, as in the GEMM kernels), each
// with the GEMM wave tile's accumulators (128 registers) and two alternating sets of operand fragments, no memory
// access inside the loop.  What this reaches is what the matrix cores deliver under the board's power limit for the
// given operand bits (zeros, or the caller's data), i.e. the ceiling the GEMM and attention kernels work under.
template <int KIND, int ORDER = 0>
__global__ __launch_bounds__(512) void mfma_probe_kernel(const u32x4* __restrict__ operands, float* __restrict__ sink, int iters) {
    const int lane = threadIdx.x & 63;
    constexpr int NA = KIND == 0 ? 4 : 8, NB = KIND == 0 ? 2 : 4;       // fragments of a 128 x 64 wave tile
    u32x4 fa[2][NA], fb[2][NB];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int i = 0; i < NA; ++i) fa[s][i] = operands ? operands[((s * 12 + i) * 64 + lane) % 4096] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < NB; ++i) fb[s][i] = operands ? operands[((s * 12 + 8 + i) * 64 + lane) % 4096] : u32x4{0u, 0u, 0u, 0u};
    }
    if constexpr (KIND == 0) {
        f32x16 acc[NA][NB];
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
        // ORDER 0: the four activation-side fragments outermost (an operand pair shares one fragment with the pair before it
        // every second instruction); 1: the two weight-side fragments outermost (one operand unchanged for four instructions
        // in a row); 2: the same with the inner walk reversed on every second pass (the turn shares both); 3: one operand pair
        // for every instruction (what operand reuse could save at most)
        auto one = [&](int s, int a, int b) __attribute__((always_inline)) {
            const int so = ORDER == 3 ? 0 : s, ao = ORDER == 3 ? 0 : a, bo = ORDER == 3 ? 0 : b;
            acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fb[so][bo]), __builtin_bit_cast(bf16x8, fa[so][ao]), acc[a][b], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        };
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                if constexpr (ORDER == 0 || ORDER == 3) {
#pragma unroll
                    for (int a = 0; a < NA; ++a)
#pragma unroll
                        for (int b = 0; b < NB; ++b) one(s, a, b);
                } else {
#pragma unroll
                    for (int b = 0; b < NB; ++b)
#pragma unroll
                        for (int a = 0; a < NA; ++a) one(s, (ORDER == 2 && ((b + s * NB) & 1)) ? NA - 1 - a : a, b);
                }
            }
        }
        float t = 0.f;
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) t += acc[a][b][r];
        if (t == 12345.678f) sink[0] = t;          // keeps the accumulators alive; practically never true
    } else {
        f32x4 acc[NA][NB];
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
            for (int b = 0; b < NB; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int a = 0; a < NA; ++a)
#pragma unroll
                    for (int b = 0; b < NB; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, fb[s][b]), __builtin_bit_cast(bf16x8, fa[s][a]), acc[a][b], 0, 0, 0);
        }
        float t = 0.f;
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int r = 0; r < 4; ++r) t += acc[a][b][r];
        if (t == 12345.678f) sink[0] = t;
    }
}

extern "C" int grl_mfma_probe(grl_ctx* c, int kind, const void* operands, int iters, float* ms, double* flops) {
    GRL_REQUIRE(c && ms && flops, GRL_ERR_ARG, "grl_mfma_probe: null argument");
    GRL_REQUIRE(kind >= 0 && kind <= 4, GRL_ERR_ARG, "grl_mfma_probe: kind must be 0 (32x32x16 bf16), 1 (16x16x32 bf16) or 2..4 (32x32x16 in another operand order)");
    GRL_REQUIRE(iters > 0 && iters <= (1 << 20), GRL_ERR_ARG, "grl_mfma_probe: iters must be in 1..2^20");
    GRL_REQUIRE((((uintptr_t)operands) & 15u) == 0, GRL_ERR_ARG, "grl_mfma_probe: operands must be 16-byte aligned (64 KiB of them, or NULL for zeros)");
    float* sink = (float*)grl_malloc(c, 256);
    if (!sink) return GRL_ERR_OOM;
    const int cus = c->prop.multiProcessorCount;
    auto launch = [&](int n) {
        if (kind == 0) hipLaunchKernelGGL(mfma_probe_kernel<0>, dim3(cus), dim3(512), 0, c->stream, (const u32x4*)operands, sink, n);
        else if (kind == 2) hipLaunchKernelGGL((mfma_probe_kernel<0, 1>), dim3(cus), dim3(512), 0, c->stream, (const u32x4*)operands, sink, n);
        else if (kind == 3) hipLaunchKernelGGL((mfma_probe_kernel<0, 2>), dim3(cus), dim3(512), 0, c->stream, (const u32x4*)operands, sink, n);
        else if (kind == 4) hipLaunchKernelGGL((mfma_probe_kernel<0, 3>), dim3(cus), dim3(512), 0, c->stream, (const u32x4*)operands, sink, n);
        else hipLaunchKernelGGL(mfma_probe_kernel<1>, dim3(cus), dim3(512), 0, c->stream, (const u32x4*)operands, sink, n);
    };
    launch(iters);                                   // warm-up: clocks and power settle
    int rc = GRL_OK;
    if (hipGetLastError() != hipSuccess) rc = GRL_ERR_HIP;
    if (!rc) rc = grl_timer_start(c);
    if (!rc) { launch(iters); if (hipGetLastError() != hipSuccess) rc = GRL_ERR_HIP; }
    if (!rc) rc = grl_timer_stop(c, ms);
    grl_free(c, sink);
    if (rc == GRL_ERR_HIP) grl_set_error("grl_mfma_probe: launch failed");
    // per iteration and wave: 2 fragment sets x a 128 x 64 wave tile x 16 (32) deep = 2 x 128*64*2*16 flops (kind 0), x 32 (kind 1)
    *flops = (double)iters * 2.0 * 128.0 * 64.0 * 2.0 * (kind == 1 ? 32.0 : 16.0) * 8.0 * cus;
    return rc;
}

// ---- shader-clock probe ---------------------------------------------------------------------------------------
// One wave that sleeps in short naps until `ticks` of the 100 MHz reference counter have passed and reports how many
// shader-clock cycles went by meanwhile.  The shader clock is one domain for the whole GPU, so a probe that runs
// beside a kernel (on its own stream) reads the clock that kernel runs at: under a power limit that is well below
// the nominal frequency the peak figures are quoted for.
__global__ __launch_bounds__(64) void clock_probe_kernel(uint64_t* out, uint64_t ticks) {
    const uint64_t r0 = __builtin_amdgcn_s_memrealtime();
    const uint64_t c0 = __builtin_amdgcn_s_memtime();
    uint64_t r;
    do {
        __builtin_amdgcn_s_sleep(32);
        r = __builtin_amdgcn_s_memrealtime();
    } while (r - r0 < ticks);             // the reference counter only moves forward: the loop ends
    const uint64_t c1 = __builtin_amdgcn_s_memtime();
    if (threadIdx.x == 0) { out[0] = c1 - c0; out[1] = r - r0; }
}

extern "C" int grl_clock_probe_begin(grl_ctx* c, float millis) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_clock_probe_begin: null context");
    GRL_REQUIRE(millis > 0.f && millis <= 500.f, GRL_ERR_ARG, "grl_clock_probe_begin: duration must be in (0, 500] ms");
    std::lock_guard<std::mutex> lk(c->timer_mu);
    GRL_CHECK_HIP(hipSetDevice(c->device));
    if (!c->probe_stream) GRL_CHECK_HIP(hipStreamCreateWithFlags(&c->probe_stream, hipStreamNonBlocking));
    if (!c->probe_out) GRL_CHECK_HIP(hipMalloc((void**)&c->probe_out, 2 * sizeof(uint64_t)));
    c->probe_pending = false;
    GRL_CHECK_HIP(hipStreamSynchronize(c->probe_stream));        // an earlier probe that nobody read has ended by now
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, c->probe_stream, c->probe_out, (uint64_t)((double)millis * 1e5));
    GRL_CHECK_LAUNCH();
    c->probe_pending = true;
    return GRL_OK;
}

extern "C" int grl_clock_probe_end(grl_ctx* c, float* ghz) {
    GRL_REQUIRE(c && ghz, GRL_ERR_ARG, "grl_clock_probe_end: null argument");
    std::lock_guard<std::mutex> lk(c->timer_mu);
    GRL_REQUIRE(c->probe_stream && c->probe_out && c->probe_pending, GRL_ERR_ARG,
                "grl_clock_probe_end: no probe was started since the last reading");
    c->probe_pending = false;       // one reading per probe, also when the copy below fails
    uint64_t h[2] = {0, 0};
    // copied on the probe's own stream: a copy on the null stream would serialise with the work being observed
    GRL_CHECK_HIP(hipMemcpyAsync(h, c->probe_out, sizeof(h), hipMemcpyDeviceToHost, c->probe_stream));
    GRL_CHECK_HIP(hipStreamSynchronize(c->probe_stream));
    *ghz = h[1] ? (float)((double)h[0] / (double)h[1] * 0.1) : 0.f;
    return GRL_OK;
}
