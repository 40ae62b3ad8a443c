// HBM-bound kernels: LayerNorm(+residual), elementwise add / GELU / SiLU / SwiGLU,
// dtype casts, RoPE, embedding gather, masked mean pooling, 2-D transpose.
// Each moves every input byte once and every output byte once; wave64 reductions only.
#include "common.hpp"
#include <cmath>

static inline bool aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }

// ------------------------------------------------------------------ 4-element vectors
template <typename T> struct vec4;
template <> struct vec4<float> {
    f32x4 v;
    __device__ __forceinline__ void load(const float* p) { v = *(const f32x4*)p; }
    __device__ __forceinline__ void store(float* p) const { *(f32x4*)p = v; }
    // streaming variants: data that is touched once should not displace what other kernels keep in L2
    __device__ __forceinline__ void load_stream(const float* p) { v = __builtin_nontemporal_load((const f32x4*)p); }
    __device__ __forceinline__ void store_stream(float* p) const { __builtin_nontemporal_store(v, (f32x4*)p); }
    __device__ __forceinline__ float get(int i) const { return v[i]; }
    __device__ __forceinline__ void set(int i, float f) { v[i] = f; }
};
template <> struct vec4<uint16_t> {
    u32x2 w;
    __device__ __forceinline__ void load(const uint16_t* p) { w = *(const u32x2*)p; }
    __device__ __forceinline__ void store(uint16_t* p) const { *(u32x2*)p = w; }
    __device__ __forceinline__ void load_stream(const uint16_t* p) { w = __builtin_nontemporal_load((const u32x2*)p); }
    __device__ __forceinline__ void store_stream(uint16_t* p) const { __builtin_nontemporal_store(w, (u32x2*)p); }
    __device__ __forceinline__ float get(int i) const {
        uint32_t x = w[i >> 1];
        return (i & 1) ? bf16hi(x) : bf16lo(x);
    }
    __device__ __forceinline__ void set(int i, float f) {
        uint32_t b = f32_to_bf16_bits(f);
        uint32_t x = w[i >> 1];
        w[i >> 1] = (i & 1) ? ((x & 0x0000ffffu) | (b << 16)) : ((x & 0xffff0000u) | b);
    }
};

__device__ __forceinline__ float wave_sum(float v) { return group_sum<64>(v); }   // whole wave active

// ------------------------------------------------------------------ LayerNorm
// One wave per row.  Rows of up to 64*4*MAXC elements (F % 4 == 0) stay in registers
// between the mean pass, the variance pass and the normalise pass, so the row is read
// from HBM exactly once (the reference makes three dispatches over it,
// shaders/fnn-layernorm.glsl:44-103).
// STATS: instead of the normalised row, {1/sd, mean/sd} goes to ((float*)y)[2*row ..] (what the LayerNorm-folded GEMM reads).
template <typename T, int MAXC, bool HAS_RES, bool STATS = false>
__global__ __launch_bounds__(256) void layernorm_rows_kernel(
    const T* x, const T* res, const float* __restrict__ gamma,
    const float* __restrict__ beta, T* y, int64_t rows, int F, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int nch = F >> 2;
    const T* xr = x + row * (int64_t)F;
    const T* rr = HAS_RES ? res + row * (int64_t)F : nullptr;
    float t[MAXC][4];
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        int ch = lane + c * 64;
        if (ch < nch) {
            vec4<T> a; a.load_stream(xr + ch * 4);
            if (HAS_RES) {
                vec4<T> b; b.load_stream(rr + ch * 4);
#pragma unroll
                for (int i = 0; i < 4; ++i) t[c][i] = a.get(i) + b.get(i);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) t[c][i] = a.get(i);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) s += t[c][i];
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) t[c][i] = 0.f;
        }
    }
    const float mean = wave_sum(s) / (float)F;
    float q = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        if (lane + c * 64 < nch) {
#pragma unroll
            for (int i = 0; i < 4; ++i) { float d = t[c][i] - mean; q += d * d; }
        }
    }
    const float var = wave_sum(q) / (float)F;
    const float sd = sqrtf(var + eps);
    if constexpr (STATS) {
        if (lane == 0) { float2 o = {1.0f / sd, mean / sd}; ((float2*)y)[row] = o; }
        return;
    }
    T* yr = y + row * (int64_t)F;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        int ch = lane + c * 64;
        if (ch < nch) {
            f32x4 g = *(const f32x4*)(gamma + ch * 4);
            f32x4 b = *(const f32x4*)(beta + ch * 4);
            vec4<T> o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o.set(i, g[i] * ((t[c][i] - mean) / sd) + b[i]);
            o.store(yr + ch * 4);      // plain: the next kernel reads these rows at once
        }
    }
}

// bf16 rows with F % 8 == 0: 16-byte streaming accesses (8 values), LPR lanes per row, i.e. 64/LPR rows per
// wave (two rows per wave for F <= 1024 keeps 96 B of loads in flight per lane at F = 768 instead of 48).
template <int MAXC, bool HAS_RES, int LPR, bool STATS = false>
__global__ __launch_bounds__(256) void layernorm_bf16x8_kernel(
    const uint16_t* x, const uint16_t* res, const float* __restrict__ gamma,
    const float* __restrict__ beta, uint16_t* y, int64_t rows, int F, float eps) {
    constexpr int RPW = 64 / LPR;
    const int lane = threadIdx.x & 63, sub = lane % LPR;
    const int64_t row = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * RPW + lane / LPR;
    if (row >= rows) return;                       // whole LPR-lane groups leave together; shuffles stay inside a group
    const int nch = F >> 3;
    const uint16_t* xr = x + row * (int64_t)F;
    const uint16_t* rr = HAS_RES ? res + row * (int64_t)F : nullptr;
    float t[MAXC][8];
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int ch = sub + c * LPR;
        if (ch < nch) {
            const u32x4 a = __builtin_nontemporal_load((const u32x4*)(xr + ch * 8));
            u32x4 b = {0u, 0u, 0u, 0u};
            if (HAS_RES) b = __builtin_nontemporal_load((const u32x4*)(rr + ch * 8));
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                t[c][2 * i] = bf16lo(a[i]) + (HAS_RES ? bf16lo(b[i]) : 0.f);
                t[c][2 * i + 1] = bf16hi(a[i]) + (HAS_RES ? bf16hi(b[i]) : 0.f);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) s += t[c][i];
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) t[c][i] = 0.f;
        }
    }
    s = group_sum<LPR>(s);
    const float mean = s / (float)F;
    float q = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        if (sub + c * LPR < nch) {
#pragma unroll
            for (int i = 0; i < 8; ++i) { float d = t[c][i] - mean; q += d * d; }
        }
    }
    q = group_sum<LPR>(q);
    const float sd = sqrtf(q / (float)F + eps);
    if constexpr (STATS) {
        if (sub == 0) { float2 o = {1.0f / sd, mean / sd}; ((float2*)y)[row] = o; }
        return;
    }
    uint16_t* yr = y + row * (int64_t)F;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int ch = sub + c * LPR;
        if (ch < nch) {
            const f32x4 g0 = *(const f32x4*)(gamma + ch * 8), g1 = *(const f32x4*)(gamma + ch * 8 + 4);
            const f32x4 b0 = *(const f32x4*)(beta + ch * 8), b1 = *(const f32x4*)(beta + ch * 8 + 4);
            float o[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                o[i] = g0[i] * ((t[c][i] - mean) / sd) + b0[i];
                o[4 + i] = g1[i] * ((t[c][4 + i] - mean) / sd) + b1[i];
            }
            const u32x4 w = {pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7])};
            // plain store: the next kernel (a GEMM) reads these rows at once, and leaving them in the
            // cache hierarchy is worth more there than the streaming hint is here
            *(u32x4*)(yr + ch * 8) = w;
        }
    }
}

// Any F: three passes over the row from global memory (the second and third hit L2).
template <typename T, bool HAS_RES, bool STATS = false>
__global__ __launch_bounds__(256) void layernorm_rows_generic_kernel(
    const T* x, const T* res, const float* __restrict__ gamma,
    const float* __restrict__ beta, T* y, int64_t rows, int F, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * (int64_t)F;
    const T* rr = HAS_RES ? res + row * (int64_t)F : nullptr;
    float s = 0.f;
    for (int f = lane; f < F; f += 64) s += elem<T>::ld(xr + f) + (HAS_RES ? elem<T>::ld(rr + f) : 0.f);
    const float mean = wave_sum(s) / (float)F;
    float q = 0.f;
    for (int f = lane; f < F; f += 64) {
        float d = elem<T>::ld(xr + f) + (HAS_RES ? elem<T>::ld(rr + f) : 0.f) - mean;
        q += d * d;
    }
    const float sd = sqrtf(wave_sum(q) / (float)F + eps);
    if constexpr (STATS) {
        if (lane == 0) { float2 o = {1.0f / sd, mean / sd}; ((float2*)y)[row] = o; }
        return;
    }
    T* yr = y + row * (int64_t)F;
    for (int f = lane; f < F; f += 64) {
        float v = elem<T>::ld(xr + f) + (HAS_RES ? elem<T>::ld(rr + f) : 0.f);
        elem<T>::st(yr + f, gamma[f] * ((v - mean) / sd) + beta[f]);
    }
}

template <typename T>
static int launch_layernorm(grl_ctx* c, int64_t rows, int64_t F, const void* x, const void* res,
                            const float* g, const float* b, float eps, void* y) {
    dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    const T* X = (const T*)x; const T* R = (const T*)res; T* Y = (T*)y;
    bool fast = (F % 4 == 0) && F <= 64 * 4 * 8 && aligned16(x) && aligned16(y) && aligned16(g) &&
                aligned16(b) && (!res || aligned16(res)) && ((F * sizeof(T)) % 8 == 0);
    // bf16 rows need 8-byte alignment of every row start: F*2 % 8 == 0 <=> F % 4 == 0 (checked)
#define LN_LAUNCH(MAXC)                                                                             \
    do {                                                                                            \
        if (res) hipLaunchKernelGGL((layernorm_rows_kernel<T, MAXC, true>), grid, block, 0, c->stream, X, R, g, b, Y, rows, (int)F, eps); \
        else     hipLaunchKernelGGL((layernorm_rows_kernel<T, MAXC, false>), grid, block, 0, c->stream, X, R, g, b, Y, rows, (int)F, eps); \
    } while (0)
    if constexpr (sizeof(T) == 2) {
        // bf16, F % 8 == 0 (rows and vectors 16-byte aligned): the 16-byte kernel
        if (fast && F % 8 == 0 && F <= 4096) {
            const int nch8 = (int)(F / 8);
#define LN16_LAUNCH(MAXC, LPR)                                                                               \
    do {                                                                                                     \
        dim3 g16((unsigned)((rows + 4 * (64 / LPR) - 1) / (4 * (64 / LPR))));                                \
        if (res) hipLaunchKernelGGL((layernorm_bf16x8_kernel<MAXC, true, LPR>), g16, block, 0, c->stream, X, R, g, b, Y, rows, (int)F, eps); \
        else     hipLaunchKernelGGL((layernorm_bf16x8_kernel<MAXC, false, LPR>), g16, block, 0, c->stream, X, R, g, b, Y, rows, (int)F, eps); \
    } while (0)
            if (nch8 <= 32 * 2) LN16_LAUNCH(2, 32);
            else if (nch8 <= 32 * 4) LN16_LAUNCH(4, 32);
            else if (nch8 <= 64 * 4) LN16_LAUNCH(4, 64);
            else LN16_LAUNCH(8, 64);
#undef LN16_LAUNCH
            GRL_CHECK_LAUNCH();
            return GRL_OK;
        }
    }
    if (fast) {
        int nch = (int)(F / 4), maxc = (nch + 63) / 64;
        if (maxc <= 2) LN_LAUNCH(2);
        else if (maxc <= 3) LN_LAUNCH(3);
        else if (maxc <= 4) LN_LAUNCH(4);
        else LN_LAUNCH(8);
    } else {
        if (res) hipLaunchKernelGGL((layernorm_rows_generic_kernel<T, true>), grid, block, 0, c->stream, X, R, g, b, Y, rows, (int)F, eps);
        else     hipLaunchKernelGGL((layernorm_rows_generic_kernel<T, false>), grid, block, 0, c->stream, X, R, g, b, Y, rows, (int)F, eps);
    }
#undef LN_LAUNCH
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

extern "C" int grl_layernorm(grl_ctx* c, int dtype, int64_t rows, int64_t F, const void* x,
                             const void* residual, const float* gamma, const float* beta, float eps, void* y) {
    GRL_REQUIRE(c && x && gamma && beta && y, GRL_ERR_ARG, "grl_layernorm: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_layernorm: bad dtype %d", dtype);
    GRL_REQUIRE(rows >= 0 && F > 0 && F < (1 << 30), GRL_ERR_SHAPE, "grl_layernorm: bad shape rows=%lld F=%lld", (long long)rows, (long long)F);
    GRL_REQUIRE(rows < ((int64_t)1 << 33), GRL_ERR_SHAPE, "grl_layernorm: too many rows");
    if (rows == 0) return GRL_OK;
    return dtype == GRL_F32 ? launch_layernorm<float>(c, rows, F, x, residual, gamma, beta, eps, y)
                            : launch_layernorm<uint16_t>(c, rows, F, x, residual, gamma, beta, eps, y);
}

// Row statistics for the LayerNorm-folded GEMM: stats[2*row] = 1/sd, stats[2*row+1] = mean/sd with the same two-pass
// mean / variance as grl_layernorm (one read of x, 8 bytes per row written).
template <typename T>
static int launch_ln_stats(grl_ctx* c, int64_t rows, int64_t F, const void* x, float eps, float* stats) {
    dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    const T* X = (const T*)x; T* Y = (T*)stats;
    const float* nil = nullptr;
    const bool fast = (F % 4 == 0) && F <= 64 * 4 * 8 && aligned16(x) && ((F * sizeof(T)) % 8 == 0);
    if constexpr (sizeof(T) == 2) {
        if (fast && F % 8 == 0 && F <= 4096) {
            const int nch8 = (int)(F / 8);
#define LNS16_LAUNCH(MAXC, LPR)                                                                              \
    do {                                                                                                     \
        dim3 g16((unsigned)((rows + 4 * (64 / LPR) - 1) / (4 * (64 / LPR))));                                \
        hipLaunchKernelGGL((layernorm_bf16x8_kernel<MAXC, false, LPR, true>), g16, block, 0, c->stream, X, X, nil, nil, Y, rows, (int)F, eps); \
    } while (0)
            if (nch8 <= 32 * 2) LNS16_LAUNCH(2, 32);
            else if (nch8 <= 32 * 4) LNS16_LAUNCH(4, 32);
            else if (nch8 <= 64 * 4) LNS16_LAUNCH(4, 64);
            else LNS16_LAUNCH(8, 64);
#undef LNS16_LAUNCH
            GRL_CHECK_LAUNCH();
            return GRL_OK;
        }
    }
    if (fast) {
        const int nch = (int)(F / 4), maxc = (nch + 63) / 64;
        if (maxc <= 2) hipLaunchKernelGGL((layernorm_rows_kernel<T, 2, false, true>), grid, block, 0, c->stream, X, X, nil, nil, Y, rows, (int)F, eps);
        else if (maxc <= 3) hipLaunchKernelGGL((layernorm_rows_kernel<T, 3, false, true>), grid, block, 0, c->stream, X, X, nil, nil, Y, rows, (int)F, eps);
        else if (maxc <= 4) hipLaunchKernelGGL((layernorm_rows_kernel<T, 4, false, true>), grid, block, 0, c->stream, X, X, nil, nil, Y, rows, (int)F, eps);
        else hipLaunchKernelGGL((layernorm_rows_kernel<T, 8, false, true>), grid, block, 0, c->stream, X, X, nil, nil, Y, rows, (int)F, eps);
    } else {
        hipLaunchKernelGGL((layernorm_rows_generic_kernel<T, false, true>), grid, block, 0, c->stream, X, X, nil, nil, Y, rows, (int)F, eps);
    }
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

extern "C" int grl_ln_stats(grl_ctx* c, int dtype, int64_t rows, int64_t F, const void* x, float eps, float* stats) {
    GRL_REQUIRE(c && x && stats, GRL_ERR_ARG, "grl_ln_stats: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_ln_stats: bad dtype %d", dtype);
    GRL_REQUIRE(rows >= 0 && F > 0 && F < (1 << 30), GRL_ERR_SHAPE, "grl_ln_stats: bad shape rows=%lld F=%lld", (long long)rows, (long long)F);
    GRL_REQUIRE(rows < ((int64_t)1 << 33), GRL_ERR_SHAPE, "grl_ln_stats: too many rows");
    GRL_REQUIRE((((uintptr_t)stats) & 15u) == 0, GRL_ERR_ARG, "grl_ln_stats: stats must be 16-byte aligned");
    if (rows == 0) return GRL_OK;
    return dtype == GRL_F32 ? launch_ln_stats<float>(c, rows, F, x, eps, stats) : launch_ln_stats<uint16_t>(c, rows, F, x, eps, stats);
}

// Weight side of the LayerNorm-folded GEMM, once per weight: W_scaled[n,k] = gamma[k]*W[n,k] (rounded to the storage
// type), colsum[n] = sum_k W_scaled[n,k] (of the rounded values, which is what the GEMM multiplies), bias_folded[n] =
// bias[n] + sum_k beta[k]*W[n,k].  One wave per weight row.
template <typename T>
__global__ __launch_bounds__(256) void ln_fold_kernel(const T* W, const float* gamma, const float* beta, const float* bias,
                                                      T* Ws, float* colsum, float* bias_folded, int64_t N, int K) {
    const int lane = threadIdx.x & 63;
    const int64_t n = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const T* w = W + n * (int64_t)K;
    T* ws = Ws + n * (int64_t)K;
    float cs = 0.f, ds = 0.f;
    for (int k = lane; k < K; k += 64) {
        const float wv = elem<T>::ld(w + k);
        elem<T>::st(ws + k, gamma[k] * wv);
        cs += elem<T>::ld(ws + k);          // the value as stored
        ds += beta[k] * wv;
    }
    cs = wave_sum(cs); ds = wave_sum(ds);
    if (lane == 0) { colsum[n] = cs; bias_folded[n] = ds + (bias ? bias[n] : 0.f); }
}

extern "C" int grl_ln_fold(grl_ctx* c, int dtype, int64_t N, int64_t K, const void* W, const float* gamma, const float* beta,
                           const float* bias, void* W_scaled, float* colsum, float* bias_folded) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_ln_fold: null context");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_ln_fold: bad dtype %d", dtype);
    GRL_REQUIRE(N >= 0 && K > 0 && K < (1LL << 31) && N < (1LL << 31), GRL_ERR_SHAPE, "grl_ln_fold: bad shape N=%lld K=%lld", (long long)N, (long long)K);
    if (N == 0) return GRL_OK;
    GRL_REQUIRE(W && gamma && beta && W_scaled && colsum && bias_folded, GRL_ERR_ARG, "grl_ln_fold: null argument");
    dim3 grid((unsigned)((N + 3) / 4)), block(256);
    if (dtype == GRL_F32) hipLaunchKernelGGL(ln_fold_kernel<float>, grid, block, 0, c->stream, (const float*)W, gamma, beta, bias, (float*)W_scaled, colsum, bias_folded, N, (int)K);
    else hipLaunchKernelGGL(ln_fold_kernel<uint16_t>, grid, block, 0, c->stream, (const uint16_t*)W, gamma, beta, bias, (uint16_t*)W_scaled, colsum, bias_folded, N, (int)K);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// ------------------------------------------------------------------ elementwise
enum { OP_ADD = 0, OP_GELU = 1, OP_SILU = 2, OP_RELU = 3, OP_GCU = 4, OP_ROSWISH = 5 };

// shaders/activation-swiglu.glsl:40-49: sign-split stable sigmoid
__device__ __forceinline__ float sigmoid_stable(float v) {
    if (v >= 0.f) return 1.0f / (1.0f + __expf(-v));
    float e = __expf(v);
    return e / (1.0f + e);
}

// p0, p1: alpha and beta of RoSwish, unused otherwise
template <int OP> __device__ __forceinline__ float ew_apply(float a, float b, float p0, float p1) {
    if (OP == OP_ADD) return a + b;
    if (OP == OP_GELU) return gelu_ref(a);
    if (OP == OP_RELU) return fmaxf(a, 0.0f);   // shaders/activation-relu.glsl (backend/fnn.py:232-283)
    if (OP == OP_GCU) return a * cosf(a);       // shaders/activation-gcu.glsl:29-31 (backend/fnn.py:393-440)
    if (OP == OP_ROSWISH) return (a + p0) * sigmoid_stable(p1 * a) - 0.5f * p0;   // shaders/activation-roswish.glsl:30-46
    return a * sigmoid_stable(a);   // backend/fnn.py:344-391 (activation_silu): x*sigmoid(x)
}

template <typename T, int OP, bool VEC>
__global__ __launch_bounds__(256) void elementwise_kernel(const T* a, const T* b, T* out, int64_t n, float p0, float p1) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (VEC) {
        const int64_t nv = n >> 2;
        for (int64_t v = i; v < nv; v += stride) {
            vec4<T> x, y, o;
            x.load(a + v * 4);
            if (OP == OP_ADD) y.load(b + v * 4);
#pragma unroll
            for (int k = 0; k < 4; ++k) o.set(k, ew_apply<OP>(x.get(k), OP == OP_ADD ? y.get(k) : 0.f, p0, p1));
            o.store(out + v * 4);
        }
        for (int64_t t = (nv << 2) + i; t < n; t += stride)
            elem<T>::st(out + t, ew_apply<OP>(elem<T>::ld(a + t), OP == OP_ADD ? elem<T>::ld(b + t) : 0.f, p0, p1));
    } else {
        for (int64_t t = i; t < n; t += stride)
            elem<T>::st(out + t, ew_apply<OP>(elem<T>::ld(a + t), OP == OP_ADD ? elem<T>::ld(b + t) : 0.f, p0, p1));
    }
}

static inline unsigned ew_grid(int64_t work_items) {
    int64_t g = (work_items + 255) / 256;
    const int64_t cap = 256 * 32;   // 256 CUs x enough waves to cover HBM latency; grid-stride beyond
    if (g > cap) g = cap;
    if (g < 1) g = 1;
    return (unsigned)g;
}

template <typename T, int OP>
static int launch_ew(grl_ctx* c, int64_t n, const void* a, const void* b, void* out, float p0 = 0.f, float p1 = 0.f) {
    bool vec = aligned16(a) && aligned16(out) && (!b || aligned16(b));
    if (vec) hipLaunchKernelGGL((elementwise_kernel<T, OP, true>), dim3(ew_grid(n / 4 + 1)), dim3(256), 0, c->stream, (const T*)a, (const T*)b, (T*)out, n, p0, p1);
    else     hipLaunchKernelGGL((elementwise_kernel<T, OP, false>), dim3(ew_grid(n)), dim3(256), 0, c->stream, (const T*)a, (const T*)b, (T*)out, n, p0, p1);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

#define EW_ENTRY(NAME, OP, NEEDS_B)                                                                   \
    GRL_REQUIRE(c && a && out && (!(NEEDS_B) || b), GRL_ERR_ARG, NAME ": null argument");             \
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, NAME ": bad dtype %d", dtype);                   \
    GRL_REQUIRE(n >= 0, GRL_ERR_SHAPE, NAME ": negative size");                                       \
    if (n == 0) return GRL_OK;                                                                        \
    return dtype == GRL_F32 ? launch_ew<float, OP>(c, n, a, b, out) : launch_ew<uint16_t, OP>(c, n, a, b, out);

extern "C" int grl_add(grl_ctx* c, int dtype, int64_t n, const void* a, const void* b, void* out) { EW_ENTRY("grl_add", OP_ADD, true) }
extern "C" int grl_gelu(grl_ctx* c, int dtype, int64_t n, const void* a, void* out) { const void* b = nullptr; EW_ENTRY("grl_gelu", OP_GELU, false) }
extern "C" int grl_silu(grl_ctx* c, int dtype, int64_t n, const void* a, void* out) { const void* b = nullptr; EW_ENTRY("grl_silu", OP_SILU, false) }
extern "C" int grl_relu(grl_ctx* c, int dtype, int64_t n, const void* a, void* out) { const void* b = nullptr; EW_ENTRY("grl_relu", OP_RELU, false) }
extern "C" int grl_gcu(grl_ctx* c, int dtype, int64_t n, const void* a, void* out) { const void* b = nullptr; EW_ENTRY("grl_gcu", OP_GCU, false) }
extern "C" int grl_roswish(grl_ctx* c, int dtype, int64_t n, const void* a, void* out, float alpha, float beta) {
    GRL_REQUIRE(c && a && out, GRL_ERR_ARG, "grl_roswish: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_roswish: bad dtype %d", dtype);
    GRL_REQUIRE(n >= 0, GRL_ERR_SHAPE, "grl_roswish: negative size");
    if (n == 0) return GRL_OK;
    return dtype == GRL_F32 ? launch_ew<float, OP_ROSWISH>(c, n, a, nullptr, out, alpha, beta) : launch_ew<uint16_t, OP_ROSWISH>(c, n, a, nullptr, out, alpha, beta);
}

// softmax over the last dimension, one wave per row: maximum (starting from -1e10 like the shader's first pass),
// sum of exp(x - max), quotient; the second and third pass read the row again (from cache for rows of usual length)
template <typename T>
__global__ __launch_bounds__(256) void softmax_rows_kernel(const T* x, T* y, int64_t rows, int F) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const T* xr = x + row * (int64_t)F;
    T* yr = y + row * (int64_t)F;
    float m = -1e10f;
    for (int i = lane; i < F; i += 64) m = fmaxf(m, elem<T>::ld(xr + i));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    float sum = 0.f;
    for (int i = lane; i < F; i += 64) sum += __expf(elem<T>::ld(xr + i) - m);
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    for (int i = lane; i < F; i += 64) elem<T>::st(yr + i, __expf(elem<T>::ld(xr + i) - m) * inv);
}

extern "C" int grl_softmax(grl_ctx* c, int dtype, int64_t rows, int64_t F, const void* x, void* y) {
    GRL_REQUIRE(c && x && y, GRL_ERR_ARG, "grl_softmax: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_softmax: bad dtype %d", dtype);
    GRL_REQUIRE(rows >= 0 && F > 0 && F < (1 << 30) && rows < ((int64_t)1 << 33), GRL_ERR_SHAPE, "grl_softmax: bad shape rows=%lld F=%lld", (long long)rows, (long long)F);
    if (rows == 0) return GRL_OK;
    const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    if (dtype == GRL_F32) hipLaunchKernelGGL(softmax_rows_kernel<float>, grid, block, 0, c->stream, (const float*)x, (float*)y, rows, (int)F);
    else hipLaunchKernelGGL(softmax_rows_kernel<uint16_t>, grid, block, 0, c->stream, (const uint16_t*)x, (uint16_t*)y, rows, (int)F);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// x (rows, 2h) -> y (rows, h)
template <typename T>
__global__ __launch_bounds__(256) void swiglu_act_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t h) {
    const int64_t n = rows * h, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        int64_t r = i / h, p = i - r * h;
        float x1 = elem<T>::ld(x + r * 2 * h + p);
        float x2 = elem<T>::ld(x + r * 2 * h + h + p);
        elem<T>::st(y + i, x1 * (x2 * sigmoid_stable(x2)));
    }
}

extern "C" int grl_swiglu_act(grl_ctx* c, int dtype, int64_t rows, int64_t h, const void* x, void* y) {
    GRL_REQUIRE(c && x && y, GRL_ERR_ARG, "grl_swiglu_act: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_swiglu_act: bad dtype %d", dtype);
    GRL_REQUIRE(rows >= 0 && h >= 0, GRL_ERR_SHAPE, "grl_swiglu_act: negative size");
    if (rows * h == 0) return GRL_OK;
    if (dtype == GRL_F32) hipLaunchKernelGGL(swiglu_act_kernel<float>, dim3(ew_grid(rows * h)), dim3(256), 0, c->stream, (const float*)x, (float*)y, rows, h);
    else hipLaunchKernelGGL(swiglu_act_kernel<uint16_t>, dim3(ew_grid(rows * h)), dim3(256), 0, c->stream, (const uint16_t*)x, (uint16_t*)y, rows, h);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// ------------------------------------------------------------------ plain copy
// Four 16-byte streaming loads in flight per lane, then four streaming stores; moves every byte once in and
// once out (6.1 TB/s on a 1 GiB copy, against 4.6 TB/s for a one-vector grid-stride loop).
__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
    constexpr int UN = 4;
    const int64_t stride = (int64_t)gridDim.x * 256 * UN;
    for (int64_t i = (int64_t)blockIdx.x * 256 * UN + threadIdx.x; i < n16; i += stride) {
        u32x4 v[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (i + u * 256 < n16) v[u] = __builtin_nontemporal_load(src + i + u * 256);
#pragma unroll
        for (int u = 0; u < UN; ++u)
            if (i + u * 256 < n16) __builtin_nontemporal_store(v[u], dst + i + u * 256);
    }
}

int grl_copy_kernel_launch(grl_ctx* c, void* dst, const void* src, size_t bytes) {
    const int64_t n16 = (int64_t)(bytes / 16);
    const int64_t blocks = (n16 + 1023) / 1024;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)(blocks < 32768 ? blocks : 32768)), dim3(256), 0, c->stream, (const u32x4*)src, (u32x4*)dst, n16);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// ------------------------------------------------------------------ casts
template <typename S, typename D>
__global__ __launch_bounds__(256) void cast_kernel(const S* __restrict__ s, D* __restrict__ d, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        elem<D>::st(d + i, elem<S>::ld(s + i));
}

extern "C" int grl_cast(grl_ctx* c, int sd, int dd, int64_t n, const void* src, void* dst) {
    GRL_REQUIRE(c && src && dst, GRL_ERR_ARG, "grl_cast: null argument");
    GRL_REQUIRE(grl_valid_dtype(sd) && grl_valid_dtype(dd), GRL_ERR_ARG, "grl_cast: bad dtype");
    GRL_REQUIRE(n >= 0, GRL_ERR_SHAPE, "grl_cast: negative size");
    if (n == 0) return GRL_OK;
    dim3 g(ew_grid(n)), b(256);
    if (sd == GRL_F32 && dd == GRL_BF16) hipLaunchKernelGGL((cast_kernel<float, uint16_t>), g, b, 0, c->stream, (const float*)src, (uint16_t*)dst, n);
    else if (sd == GRL_BF16 && dd == GRL_F32) hipLaunchKernelGGL((cast_kernel<uint16_t, float>), g, b, 0, c->stream, (const uint16_t*)src, (float*)dst, n);
    else return grl_d2d(c, dst, src, (size_t)n * grl_dtype_size(sd));
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// ------------------------------------------------------------------ RoPE
// inv_freq[p] is the correctly rounded fp32 value of base^(fe), fe = fp32(-2*p)/fp32(D), computed
// on the host in double; the angle is then formed in fp32 exactly as the shaders do:
//   half style        theta = (pos / scaling) * inv_freq      shaders/rope.glsl:114-118
//   interleaved style theta = (pos * inv_freq) / scaling      shaders/flash-attention2-rope.glsl:75-78,124-125
struct RopeFreq { float inv_freq[64]; };

void grl_rope_freqs(RopeFreq* f, int D, float base) {
    for (int p = 0; p < 64; ++p) {
        float fe = (-2.0f * (float)p) / (float)D;
        f->inv_freq[p] = p < D / 2 ? (float)pow((double)base, (double)fe) : 0.f;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void rope_kernel(const T* __restrict__ x, const int32_t* __restrict__ pos_ids,
                                                  T* __restrict__ y, int64_t total_pairs, int S, int H, int D,
                                                  int style, float scaling, RopeFreq fr, int64_t x_stride) {
    const int half = D >> 1;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_pairs; i += stride) {
        int p = (int)(i % half);
        int64_t vec = i / half;                 // (b,s,h) flat
        int64_t bs = vec / H;                   // (b,s) flat
        int s = (int)(bs % S);
        float pos = pos_ids ? (float)pos_ids[bs] : (float)s;
        float theta = style == GRL_ROPE_HALF ? (pos / scaling) * fr.inv_freq[p] : (pos * fr.inv_freq[p]) / scaling;
        float sn, cs;
        sincosf(theta, &sn, &cs);
        const int hh = (int)(vec - bs * H);
        const int64_t xin = bs * x_stride + (int64_t)hh * D;     // input may be strided by position
        int64_t i0, i1;
        if (style == GRL_ROPE_HALF) { i0 = p; i1 = p + half; }
        else { i0 = 2 * p; i1 = i0 + 1; }
        float a = elem<T>::ld(x + xin + i0), b = elem<T>::ld(x + xin + i1);
        elem<T>::st(y + vec * D + i0, a * cs - b * sn);
        elem<T>::st(y + vec * D + i1, b * cs + a * sn);
    }
}

int grl_rope_strided(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                     const int32_t* position_ids, void* y, int style, float rope_base, float rope_scaling);
int grl_build_rope_table_styled(grl_ctx* c, float* tab, int S, int D, float base, float scaling, int style);
int grl_rope_apply_table(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                         void* y, const float* table);
int grl_rope_half_apply_table(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                              void* y, const float* table);

extern "C" int grl_rope(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x,
                        const int32_t* position_ids, void* y, int style, float rope_base, float rope_scaling) {
    return grl_rope_strided(c, dtype, B, S, H, D, x, H * D, position_ids, y, style, rope_base, rope_scaling);
}

// x may have a position stride larger than H*D (a column block of a packed QKV buffer); y is dense
int grl_rope_strided(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                     const int32_t* position_ids, void* y, int style, float rope_base, float rope_scaling) {
    GRL_REQUIRE(c && x && y, GRL_ERR_ARG, "grl_rope: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_rope: bad dtype %d", dtype);
    GRL_REQUIRE(style == GRL_ROPE_HALF || style == GRL_ROPE_INTERLEAVED, GRL_ERR_ARG, "grl_rope: bad style %d", style);
    GRL_REQUIRE(B >= 0 && S >= 0 && H >= 0 && D > 0 && D % 2 == 0 && D <= 128, GRL_ERR_SHAPE,
                "grl_rope: head_dim must be even and <= 128 (got %lld)", (long long)D);
    GRL_REQUIRE(rope_scaling != 0.f && rope_base > 0.f, GRL_ERR_ARG, "grl_rope: bad base/scaling");
    GRL_REQUIRE(S < (1LL << 31) && H < (1LL << 31), GRL_ERR_SHAPE, "grl_rope: dimension too large");
    int64_t pairs = B * S * H * (D / 2);
    if (pairs == 0) return GRL_OK;
    // Positions 0..S-1 and 16-byte granular rows: angles from a (S, D/2) table built once per call with the same
    // fp32 angle arithmetic, rows moved as 16-byte chunks (the per-pair kernel below evaluates sincosf per pair).
    {
        const int64_t es = (int64_t)grl_dtype_size(dtype), epc = 16 / es;
        const bool chunks = style == GRL_ROPE_HALF ? (D / 2) % epc == 0 : D % epc == 0;
        if (!position_ids && chunks && ((((uintptr_t)x) | ((uintptr_t)y)) & 15u) == 0 && (x_stride * es) % 16 == 0 && S * (D / 2) < (1LL << 31)) {
            const float* tab = nullptr;
            int rc = grl_rope_table_get(c, (int)S, (int)D, rope_base, rope_scaling, style, &tab);
            if (rc) return rc;
            return style == GRL_ROPE_HALF ? grl_rope_half_apply_table(c, dtype, B, S, H, D, x, x_stride, y, tab)
                                          : grl_rope_apply_table(c, dtype, B, S, H, D, x, x_stride, y, tab);
        }
    }
    RopeFreq fr; grl_rope_freqs(&fr, (int)D, rope_base);
    dim3 g(ew_grid(pairs)), b(256);
    if (dtype == GRL_F32) hipLaunchKernelGGL(rope_kernel<float>, g, b, 0, c->stream, (const float*)x, position_ids, (float*)y, pairs, (int)S, (int)H, (int)D, style, rope_scaling, fr, x_stride);
    else hipLaunchKernelGGL(rope_kernel<uint16_t>, g, b, 0, c->stream, (const uint16_t*)x, position_ids, (uint16_t*)y, pairs, (int)S, (int)H, (int)D, style, rope_scaling, fr, x_stride);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// cos/sin table (S, D/2) pairs for the fused-RoPE attention kernel, interleaved-style angle.
__global__ __launch_bounds__(256) void rope_table_kernel(float2* __restrict__ tab, int S, int half, float scaling, RopeFreq fr, int style) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= S * half) return;
    int s = i / half, p = i - s * half;
    float theta = style == GRL_ROPE_HALF ? ((float)s / scaling) * fr.inv_freq[p] : ((float)s * fr.inv_freq[p]) / scaling;
    float sn, cs;
    sincosf(theta, &sn, &cs);
    tab[i] = make_float2(cs, sn);
}

int grl_build_rope_table_styled(grl_ctx* c, float* tab, int S, int D, float base, float scaling, int style) {
    RopeFreq fr; grl_rope_freqs(&fr, D, base);
    int n = S * (D / 2);
    hipLaunchKernelGGL(rope_table_kernel, dim3((n + 255) / 256), dim3(256), 0, c->stream, (float2*)tab, S, D / 2, scaling, fr, style);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}
int grl_build_rope_table(grl_ctx* c, float* tab, int S, int D, float base, float scaling) {
    return grl_build_rope_table_styled(c, tab, S, D, base, scaling, GRL_ROPE_INTERLEAVED);
}

int grl_rope_table_get(grl_ctx* c, int S, int D, float base, float scaling, int style, const float** out) {
    std::lock_guard<std::mutex> lk(c->tab_mu);
    for (auto& t : c->rope_tables)
        if (t.D == D && t.style == style && t.base == base && t.scaling == scaling && t.S >= S) { *out = (const float*)t.dev; return GRL_OK; }
    // Not there (or too short): build one.  The pointer handed out leaves this function without any hold on the
    // table (another thread of the same context may be between its lookup and its launch), so a table is NEVER
    // freed while the context lives: a superseded one moves to the retired list and keeps its memory until
    // grl_destroy.  Lengths are rounded up to a power of two (at least 1024 positions), so one kind of table is
    // rebuilt at most once per doubling of the sequence length and the retired ones add up to less than the live one.
    int64_t cap = 1024;
    while (cap < S) cap *= 2;
    if (cap * (D / 2) >= (1LL << 31)) cap = S;
    for (size_t i = 0; i < c->rope_tables.size(); ++i) {
        auto& t = c->rope_tables[i];
        if ((t.D == D && t.style == style && t.base == base && t.scaling == scaling) || c->rope_tables.size() >= 16) {
            c->retired_tables.push_back(t.dev);
            c->rope_tables.erase(c->rope_tables.begin() + i);
            break;
        }
    }
    void* dev = grl_malloc(c, (size_t)cap * (D / 2) * sizeof(float2));
    if (!dev) return GRL_ERR_OOM;
    int rc = grl_build_rope_table_styled(c, (float*)dev, (int)cap, D, base, scaling, style);
    if (rc) { grl_free(c, dev); return rc; }
    c->rope_tables.push_back({(int)cap, D, style, base, scaling, dev});
    *out = (const float*)dev;
    return GRL_OK;
}

// Interleaved RoPE from a precomputed (S, D/2) {cos, sin} table: one 16-byte chunk per thread,
// every row read once and written once (the K pre-rotation of the fused-RoPE attention path).
template <typename T>
__global__ __launch_bounds__(256) void rope_table_apply_kernel(const T* __restrict__ x, int64_t x_stride, T* __restrict__ y,
                                                              const float2* __restrict__ tab, int64_t nchunks, int S, int H, int D) {
    constexpr int EPC = 16 / (int)sizeof(T), PPC = EPC / 2;
    const int cpr = D / EPC;                       // chunks per (position, head) row
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nchunks; i += stride) {
        const int c = (int)(i % cpr);
        const int64_t vec = i / cpr;               // (b,s,h) flat
        const int64_t bs = vec / H;
        const int h = (int)(vec - bs * H), s = (int)(bs % S);
        u32x4 v = *(const u32x4*)(x + bs * x_stride + (int64_t)h * D + c * EPC);
        const float2* t = tab + (int64_t)s * (D / 2) + c * PPC;
        u32x4 o;
        if (sizeof(T) == 2) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float2 cs = t[j];
                const float x0 = bf16lo(v[j]), x1 = bf16hi(v[j]);
                o[j] = pack_bf16x2(x0 * cs.x - x1 * cs.y, x0 * cs.y + x1 * cs.x);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const float2 cs = t[j];
                const float x0 = u2f(v[2 * j]), x1 = u2f(v[2 * j + 1]);
                o[2 * j] = f2u(x0 * cs.x - x1 * cs.y);
                o[2 * j + 1] = f2u(x0 * cs.y + x1 * cs.x);
            }
        }
        *(u32x4*)(y + vec * D + c * EPC) = o;
    }
}

int grl_rope_apply_table(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                         void* y, const float* table) {
    const int64_t epc = dtype == GRL_BF16 ? 8 : 4;
    const int64_t nchunks = B * S * H * (D / epc);
    if (nchunks == 0) return GRL_OK;
    dim3 g(ew_grid(nchunks)), b(256);
    if (dtype == GRL_F32) hipLaunchKernelGGL(rope_table_apply_kernel<float>, g, b, 0, c->stream, (const float*)x, x_stride, (float*)y, (const float2*)table, nchunks, (int)S, (int)H, (int)D);
    else hipLaunchKernelGGL(rope_table_apply_kernel<uint16_t>, g, b, 0, c->stream, (const uint16_t*)x, x_stride, (uint16_t*)y, (const float2*)table, nchunks, (int)S, (int)H, (int)D);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// Rotate-half RoPE from a (S, D/2) {cos, sin} table: a thread takes one 16-byte chunk of the first half of a
// (position, head) row and its partner chunk D/2 further on (shaders/rope.glsl:74-125 pairs d with d + D/2).
template <typename T>
__global__ __launch_bounds__(256) void rope_half_apply_kernel(const T* __restrict__ x, int64_t x_stride, T* __restrict__ y,
                                                             const float2* __restrict__ tab, int64_t nchunks, int S, int H, int D) {
    constexpr int EPC = 16 / (int)sizeof(T);
    const int half = D / 2, cph = half / EPC;      // chunks per half row
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nchunks; i += stride) {
        const int c = (int)(i % cph);
        const int64_t vec = i / cph;               // (b,s,h) flat
        const int64_t bs = vec / H;
        const int h = (int)(vec - bs * H), s = (int)(bs % S);
        const T* xr = x + bs * x_stride + (int64_t)h * D + c * EPC;
        const u32x4 lo = *(const u32x4*)xr, hi = *(const u32x4*)(xr + half);
        const float2* t = tab + (int64_t)s * half + c * EPC;
        u32x4 olo, ohi;
        if (sizeof(T) == 2) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float2 c0 = t[2 * j], c1 = t[2 * j + 1];
                const float a0 = bf16lo(lo[j]), a1 = bf16hi(lo[j]), b0 = bf16lo(hi[j]), b1 = bf16hi(hi[j]);
                olo[j] = pack_bf16x2(a0 * c0.x - b0 * c0.y, a1 * c1.x - b1 * c1.y);
                ohi[j] = pack_bf16x2(b0 * c0.x + a0 * c0.y, b1 * c1.x + a1 * c1.y);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float2 cs = t[j];
                const float a = u2f(lo[j]), b = u2f(hi[j]);
                olo[j] = f2u(a * cs.x - b * cs.y);
                ohi[j] = f2u(b * cs.x + a * cs.y);
            }
        }
        T* yr = y + vec * D + c * EPC;
        *(u32x4*)yr = olo;
        *(u32x4*)(yr + half) = ohi;
    }
}

int grl_rope_half_apply_table(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                              void* y, const float* table) {
    const int64_t epc = dtype == GRL_BF16 ? 8 : 4;
    const int64_t nchunks = B * S * H * ((D / 2) / epc);
    if (nchunks == 0) return GRL_OK;
    dim3 g(ew_grid(nchunks)), b(256);
    if (dtype == GRL_F32) hipLaunchKernelGGL(rope_half_apply_kernel<float>, g, b, 0, c->stream, (const float*)x, x_stride, (float*)y, (const float2*)table, nchunks, (int)S, (int)H, (int)D);
    else hipLaunchKernelGGL(rope_half_apply_kernel<uint16_t>, g, b, 0, c->stream, (const uint16_t*)x, x_stride, (uint16_t*)y, (const float2*)table, nchunks, (int)S, (int)H, (int)D);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// ------------------------------------------------------------------ embedding gather
template <typename T>
__global__ __launch_bounds__(256) void embed_kernel(const int32_t* __restrict__ ids, const float* __restrict__ tok,
                                                   const float* __restrict__ pos, const float* __restrict__ typ,
                                                   T* __restrict__ x, int64_t rows, int S, int F, int vocab) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    int id = ids[row];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // the host validates; this only keeps loads in bounds
    const int s = (int)(row % S);
    const float* t = tok + (int64_t)id * F;
    T* o = x + row * (int64_t)F;
    if (pos && typ) {
        const float* p = pos + (int64_t)s * F;
        for (int f = lane; f < F; f += 64) elem<T>::st(o + f, t[f] + typ[f] + p[f]);
    } else {                                            // tables a model does not have (wave-uniform branch)
        const float* p = pos ? pos + (int64_t)s * F : nullptr;
        for (int f = lane; f < F; f += 64) elem<T>::st(o + f, t[f] + (typ ? typ[f] : 0.f) + (p ? p[f] : 0.f));
    }
}

// F % 4 == 0 and 16-byte aligned tables: a lane owns 4 adjacent features of its wave's row (16-byte table loads, one 8- or
// 16-byte streaming store), eight rows per workgroup
template <typename T>
__global__ __launch_bounds__(512) void embed_vec_kernel(const int32_t* __restrict__ ids, const float* __restrict__ tok,
                                                       const float* __restrict__ pos, const float* __restrict__ typ,
                                                       T* __restrict__ x, int64_t rows, int S, int F, int vocab) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 6);
    if (row >= rows) return;
    int id = ids[row];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // the host validates; this only keeps loads in bounds
    const float* t = tok + (int64_t)id * F;
    const float* p = pos ? pos + (int64_t)(row % S) * F : nullptr;
    T* o = x + row * (int64_t)F;
    for (int f = lane * 4; f < F; f += 256) {
        f32x4 v = *(const f32x4*)(t + f);
        // the shader's order: token + type + position
        if (typ) v += *(const f32x4*)(typ + f);
        if (p) v += *(const f32x4*)(p + f);
        vec4<T> out;
#pragma unroll
        for (int i = 0; i < 4; ++i) out.set(i, v[i]);
        out.store_stream(o + f);
    }
}

extern "C" int grl_embed(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t F, int64_t vocab, const int32_t* ids,
                         const float* tok_emb, const float* pos_emb, const float* type_emb, void* x) {
    GRL_REQUIRE(c && ids && tok_emb && x, GRL_ERR_ARG, "grl_embed: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_embed: bad dtype %d", dtype);
    GRL_REQUIRE(B >= 0 && S > 0 && F > 0 && vocab > 0 && S < (1LL << 31) && F < (1LL << 31) && vocab < (1LL << 31),
                GRL_ERR_SHAPE, "grl_embed: bad shape");
    int64_t rows = B * S;
    if (rows == 0) return GRL_OK;
    if (F % 4 == 0 && aligned16(tok_emb) && aligned16(x) && (!pos_emb || aligned16(pos_emb)) && (!type_emb || aligned16(type_emb))) {
        dim3 g8((unsigned)((rows + 7) / 8)), b8(512);
        if (dtype == GRL_F32) hipLaunchKernelGGL(embed_vec_kernel<float>, g8, b8, 0, c->stream, ids, tok_emb, pos_emb, type_emb, (float*)x, rows, (int)S, (int)F, (int)vocab);
        else hipLaunchKernelGGL(embed_vec_kernel<uint16_t>, g8, b8, 0, c->stream, ids, tok_emb, pos_emb, type_emb, (uint16_t*)x, rows, (int)S, (int)F, (int)vocab);
        GRL_CHECK_LAUNCH();
        return GRL_OK;
    }
    dim3 g((unsigned)((rows + 3) / 4)), b(256);
    if (dtype == GRL_F32) hipLaunchKernelGGL(embed_kernel<float>, g, b, 0, c->stream, ids, tok_emb, pos_emb, type_emb, (float*)x, rows, (int)S, (int)F, (int)vocab);
    else hipLaunchKernelGGL(embed_kernel<uint16_t>, g, b, 0, c->stream, ids, tok_emb, pos_emb, type_emb, (uint16_t*)x, rows, (int)S, (int)F, (int)vocab);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// Embedding gather and the LayerNorm that follows it in one pass: a wave gathers its row (token + type + position, in
// that order), rounds it to the storage type as the two-kernel sequence stores it, and normalises it in registers
// (two-pass mean / variance like layernorm_rows_kernel).  F % 4 == 0, F <= 2048, 16-byte aligned tables.
template <typename T>
__global__ __launch_bounds__(256) void embed_layernorm_kernel(const int32_t* __restrict__ ids, const float* __restrict__ tok,
                                                             const float* __restrict__ pos, const float* __restrict__ typ,
                                                             const float* __restrict__ gamma, const float* __restrict__ beta,
                                                             T* __restrict__ x, int64_t rows, int S, int F, int vocab, float eps) {
    constexpr int MAXC = 8;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    int id = ids[row];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // the host validates; this only keeps loads in bounds
    const float* tr = tok + (int64_t)id * F;
    const float* pr = pos ? pos + (int64_t)(row % S) * F : nullptr;
    const int nch = F >> 2;
    float t[MAXC][4];
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int ch = lane + c * 64;
        if (ch < nch) {
            f32x4 v = *(const f32x4*)(tr + ch * 4);
            if (typ) v += *(const f32x4*)(typ + ch * 4);
            if (pr) v += *(const f32x4*)(pr + ch * 4);
            vec4<T> q;                                   // through the storage type: what grl_embed would have written
#pragma unroll
            for (int i = 0; i < 4; ++i) q.set(i, v[i]);
#pragma unroll
            for (int i = 0; i < 4; ++i) { t[c][i] = q.get(i); s += t[c][i]; }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) t[c][i] = 0.f;
        }
    }
    const float mean = wave_sum(s) / (float)F;
    float q2 = 0.f;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        if (lane + c * 64 < nch) {
#pragma unroll
            for (int i = 0; i < 4; ++i) { const float d = t[c][i] - mean; q2 += d * d; }
        }
    }
    const float sd = sqrtf(wave_sum(q2) / (float)F + eps);
    T* yr = x + row * (int64_t)F;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int ch = lane + c * 64;
        if (ch < nch) {
            const f32x4 g = *(const f32x4*)(gamma + ch * 4);
            const f32x4 b = *(const f32x4*)(beta + ch * 4);
            vec4<T> o;
#pragma unroll
            for (int i = 0; i < 4; ++i) o.set(i, g[i] * ((t[c][i] - mean) / sd) + b[i]);
            o.store(yr + ch * 4);      // plain: the first GEMM reads these rows at once
        }
    }
}

extern "C" int grl_layernorm(grl_ctx* c, int dtype, int64_t rows, int64_t F, const void* x, const void* residual,
                             const float* gamma, const float* beta, float eps, void* y);

extern "C" int grl_embed_layernorm(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t F, int64_t vocab, const int32_t* ids,
                                   const float* tok_emb, const float* pos_emb, const float* type_emb,
                                   const float* gamma, const float* beta, float eps, void* x) {
    GRL_REQUIRE(c && ids && tok_emb && gamma && beta && x, GRL_ERR_ARG, "grl_embed_layernorm: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_embed_layernorm: bad dtype %d", dtype);
    GRL_REQUIRE(B >= 0 && S > 0 && F > 0 && vocab > 0 && S < (1LL << 31) && F < (1LL << 31) && vocab < (1LL << 31),
                GRL_ERR_SHAPE, "grl_embed_layernorm: bad shape");
    const int64_t rows = B * S;
    if (rows == 0) return GRL_OK;
    const bool fused = F % 4 == 0 && F <= 2048 && aligned16(tok_emb) && aligned16(x) && aligned16(gamma) && aligned16(beta) &&
                       (!pos_emb || aligned16(pos_emb)) && (!type_emb || aligned16(type_emb));
    if (!fused) {
        int rc = grl_embed(c, dtype, B, S, F, vocab, ids, tok_emb, pos_emb, type_emb, x);
        return rc ? rc : grl_layernorm(c, dtype, rows, F, x, nullptr, gamma, beta, eps, x);
    }
    dim3 g((unsigned)((rows + 3) / 4)), b(256);
    if (dtype == GRL_F32) hipLaunchKernelGGL(embed_layernorm_kernel<float>, g, b, 0, c->stream, ids, tok_emb, pos_emb, type_emb, gamma, beta, (float*)x, rows, (int)S, (int)F, (int)vocab, eps);
    else hipLaunchKernelGGL(embed_layernorm_kernel<uint16_t>, g, b, 0, c->stream, ids, tok_emb, pos_emb, type_emb, gamma, beta, (uint16_t*)x, rows, (int)S, (int)F, (int)vocab, eps);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// ------------------------------------------------------------------ masked mean pool (+ L2 normalise)
// grid (ceil(F/256), B).  F % 4 == 0: a lane owns 4 adjacent features (8- or 16-byte loads), the NW waves
// of a workgroup take every NW-th position of the sequence and their partial sums meet in LDS (sixteen waves: a
// batch of 128 sequences is only a few hundred workgroups, and the loads in flight per CU are what the rate hangs on).
template <typename T, int NW>
__global__ __launch_bounds__(NW * 64) void mean_pool_kernel(const T* __restrict__ x, const float* __restrict__ mask,
                                                           float* __restrict__ out, int S, int F) {
    __shared__ float part[NW][256];
    __shared__ float cpart[NW];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int f0 = blockIdx.x * 256 + lane * 4;
    const int64_t b = blockIdx.y;
    float a[4] = {0.f, 0.f, 0.f, 0.f}, cnt = 0.f;
    const T* xb = x + b * S * (int64_t)F + f0;
    const bool live = f0 < F;
#pragma unroll 8
    for (int s = wave; s < S; s += NW) {
        const float m = mask ? mask[b * S + s] : 1.0f;
        cnt += m;
        if (live) {
            vec4<T> v; v.load_stream(xb + (int64_t)s * F);
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] += m * v.get(i);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) part[wave][lane * 4 + i] = a[i];
    if (lane == 0) cpart[wave] = cnt;
    __syncthreads();
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (threadIdx.x < 256 && f < F) {
        float tot = 0.f, c = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) { tot += part[w][threadIdx.x]; c += cpart[w]; }
        out[b * F + f] = tot / fmaxf(c, 1e-9f);
    }
}

// any F: thread f sums its feature over the sequence (coalesced across f)
template <typename T>
__global__ __launch_bounds__(256) void mean_pool_generic_kernel(const T* __restrict__ x, const float* __restrict__ mask,
                                                               float* __restrict__ out, int S, int F) {
    const int f = blockIdx.x * 256 + threadIdx.x;
    const int64_t b = blockIdx.y;
    if (f >= F) return;
    float acc = 0.f, cnt = 0.f;
    for (int s = 0; s < S; ++s) {
        float m = mask ? mask[b * S + s] : 1.0f;
        cnt += m;
        acc += m * elem<T>::ld(x + (b * S + s) * (int64_t)F + f);
    }
    out[b * F + f] = acc / fmaxf(cnt, 1e-9f);
}

__global__ __launch_bounds__(256) void l2_normalize_kernel(float* __restrict__ v, int F) {
    __shared__ float part[4];
    float* r = v + (int64_t)blockIdx.x * F;
    float s = 0.f;
    for (int f = threadIdx.x; f < F; f += 256) s += r[f] * r[f];
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    float n = fmaxf(sqrtf(part[0] + part[1] + part[2] + part[3]), 1e-12f);
    for (int f = threadIdx.x; f < F; f += 256) r[f] = r[f] / n;
}

extern "C" int grl_mean_pool(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t F, const void* x,
                             const float* mask, float* out, int l2_normalize) {
    GRL_REQUIRE(c && x && out, GRL_ERR_ARG, "grl_mean_pool: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_mean_pool: bad dtype %d", dtype);
    GRL_REQUIRE(B >= 0 && B < 65536 && S > 0 && F > 0 && S < (1LL << 31) && F < (1LL << 31), GRL_ERR_SHAPE, "grl_mean_pool: bad shape");
    if (B == 0) return GRL_OK;
    constexpr int PW = 16;                                  // waves per workgroup of the vector kernel
    dim3 g((unsigned)((F + 255) / 256), (unsigned)B), b(256), bv(PW * 64);
    const bool vec = F % 4 == 0 && aligned16(x);
    if (dtype == GRL_F32) {
        if (vec) hipLaunchKernelGGL((mean_pool_kernel<float, PW>), g, bv, 0, c->stream, (const float*)x, mask, out, (int)S, (int)F);
        else hipLaunchKernelGGL(mean_pool_generic_kernel<float>, g, b, 0, c->stream, (const float*)x, mask, out, (int)S, (int)F);
    } else {
        if (vec) hipLaunchKernelGGL((mean_pool_kernel<uint16_t, PW>), g, bv, 0, c->stream, (const uint16_t*)x, mask, out, (int)S, (int)F);
        else hipLaunchKernelGGL(mean_pool_generic_kernel<uint16_t>, g, b, 0, c->stream, (const uint16_t*)x, mask, out, (int)S, (int)F);
    }
    GRL_CHECK_LAUNCH();
    if (l2_normalize) {
        hipLaunchKernelGGL(l2_normalize_kernel, dim3((unsigned)B), dim3(256), 0, c->stream, out, (int)F);
        GRL_CHECK_LAUNCH();
    }
    return GRL_OK;
}

// ------------------------------------------------------------------ 2-D transpose (for gemm_nn)
// in (R,C) row-major -> out (C,R); 64x64 tiles through LDS, one extra column against bank conflicts.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ in, T* __restrict__ out, int64_t R, int64_t C) {
    __shared__ T tile[64][65];
    const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int j = ty; j < 64; j += 4)
        if (r0 + j < R && c0 + tx < C) tile[j][tx] = in[(r0 + j) * C + c0 + tx];
    __syncthreads();
    for (int j = ty; j < 64; j += 4)
        if (c0 + j < C && r0 + tx < R) out[(c0 + j) * R + r0 + tx] = tile[tx][j];
}

int grl_transpose2d(grl_ctx* c, int dtype, int64_t R, int64_t C, const void* in, void* out) {
    dim3 g((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64)), b(256);
    GRL_REQUIRE(g.y < 65536, GRL_ERR_SHAPE, "transpose: too many rows (%lld)", (long long)R);
    if (dtype == GRL_F32) hipLaunchKernelGGL(transpose_kernel<float>, g, b, 0, c->stream, (const float*)in, (float*)out, R, C);
    else hipLaunchKernelGGL(transpose_kernel<uint16_t>, g, b, 0, c->stream, (const uint16_t*)in, (uint16_t*)out, R, C);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}
