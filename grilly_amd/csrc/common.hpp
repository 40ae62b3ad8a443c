// Shared host/device helpers for libgrilly_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <cstdio>
#include <cstdarg>
#include <map>
#include <mutex>
#include <vector>
#include "../../include/grilly_hip.h"

// ---------------------------------------------------------------- context
#define GRL_MAX_LAPS 256
struct grl_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    hipEvent_t laps[GRL_MAX_LAPS] = {};   // lap events (grl_timer_lap), created on first use
    int lap_next = -1;                    // >= 0: the layer entry points record a lap after each of their launches (grl_timer_lap_trace)
    hipDeviceProp_t prop{};
    std::mutex mu;          // guards the pool
    std::mutex timer_mu;    // guards the event pair
    // caching pool: bucket size -> free blocks; live pointer -> bucket size
    std::map<size_t, std::vector<void*>> free_blocks;
    std::map<void*, size_t> live;
    grl_pool_stats stats{};
    // cos/sin tables of the rotary embedding, built once per (head dim, base, scaling, pairing) and kept until the
    // context goes away; a table built for S positions serves every shorter sequence.  A table that a longer one
    // replaces is retired, not freed: callers hold its raw pointer between lookup and launch (grl_destroy frees
    // every live pool block, retired tables included)
    struct rope_table { int S, D, style; float base, scaling; void* dev; };
    std::mutex tab_mu;
    std::vector<rope_table> rope_tables;
    std::vector<void*> retired_tables;
    // pinned staging ring for small host -> device copies (grl_h2d): the caller's buffer is copied here and the transfer
    // runs asynchronously on the stream; a wrap-around waits for the stream, i.e. for every transfer still reading the ring
    std::mutex stage_mu;
    char* stage = nullptr;
    size_t stage_cap = 0, stage_off = 0;
    bool stage_failed = false;          // pinned allocation refused once: stay on the blocking path
    // shader-clock probe (grl_clock_probe_begin / _end): its own stream, so that it runs beside the work it observes
    hipStream_t probe_stream = nullptr;
    uint64_t* probe_out = nullptr;      // device: {shader cycles, 100 MHz ticks}
    bool probe_pending = false;         // a probe was launched and its result not read yet (under timer_mu)
};

// device pointer to a (>= S, D/2) table of {cos, sin}; builds it on first use (on the context stream)
int grl_rope_table_get(grl_ctx* c, int S, int D, float base, float scaling, int style, const float** out);

void grl_set_error(const char* fmt, ...);

// one lap event behind the launches enqueued so far, when a lap trace is on (and has indices left); used by the
// entry points that launch several kernels, so that a caller can time the launches inside them
void grl_lap_mark(grl_ctx* c);

#define GRL_CHECK_HIP(expr)                                                              \
    do {                                                                                 \
        hipError_t _e = (expr);                                                          \
        if (_e != hipSuccess) {                                                          \
            grl_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, __LINE__); \
            return GRL_ERR_HIP;                                                          \
        }                                                                                \
    } while (0)

#define GRL_REQUIRE(cond, code, ...)                                                     \
    do {                                                                                 \
        if (!(cond)) {                                                                   \
            grl_set_error(__VA_ARGS__);                                                  \
            return (code);                                                               \
        }                                                                                \
    } while (0)

// Checks the launch itself (bad configuration, missing code object); kernel faults
// surface at the next synchronisation.
#define GRL_CHECK_LAUNCH()  GRL_CHECK_HIP(hipGetLastError())

static inline bool grl_valid_dtype(int d) { return d == GRL_F32 || d == GRL_BF16; }
static inline size_t grl_dtype_size(int d) { return d == GRL_BF16 ? 2 : 4; }

// pool-backed temporary that is returned to the pool when it goes out of scope;
// safe because every kernel of a context runs in order on the one stream.
struct grl_temp {
    grl_ctx* ctx; void* p;
    grl_temp(grl_ctx* c, size_t bytes) : ctx(c), p(grl_malloc(c, bytes)) {}
    ~grl_temp() { if (p) grl_free(ctx, p); }
    grl_temp(const grl_temp&) = delete;
    grl_temp& operator=(const grl_temp&) = delete;
};

// ---------------------------------------------------------------- device helpers
#if defined(__HIPCC__)
typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// fp32 -> bf16 bits, round to nearest even; NaN stays NaN.
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}
// two floats -> packed pair of bf16 (lo in bits 0..15); one v_cvt_pk_bf16_f32 (RNE) on gfx950
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// bit reinterpretation through a by-value copy: __builtin_bit_cast applied directly to an
// element of an ext_vector (v[i]) reads element 0 whatever i is.
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float bf16lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }

// ---- global -> LDS transfer the compiler does not see (buffer_load_dwordx4 ... lds).
// The wave writes 64 x 16 B to LDS at lds_dst (wave-uniform) + lane*16; each lane fetches from
// resource base + voff; lanes whose voff is out of range transfer zeros.  Issued through inline
// asm so that the compiler's wait-count insertion does not treat it as a pending LDS write that
// later LDS accesses (notably the transposing reads) must fully wait for; the caller places the
// s_waitcnt vmcnt(N) itself.
typedef __attribute__((ext_vector_type(4))) int rsrc_words;
__device__ __forceinline__ rsrc_words make_rsrc_words(const void* base, uint32_t num_bytes) {
    const uint64_t a = (uint64_t)base;
    // wave-uniform by construction; readfirstlane tells the compiler so (the words must sit in SGPRs)
    rsrc_words r = {(int)__builtin_amdgcn_readfirstlane((uint32_t)a), (int)__builtin_amdgcn_readfirstlane((uint32_t)((a >> 32) & 0xffffu)),
                    (int)__builtin_amdgcn_readfirstlane(num_bytes), 0x00020000};
    return r;
}
__device__ __forceinline__ void dma16(rsrc_words rs, const void* lds_dst_wave_uniform, int voff) {
    const uint32_t la = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)lds_dst_wave_uniform);
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(la), "v"(voff), "s"(rs) : "memory");
}

// ---- LDS slot swizzle -------------------------------------------------------------------
// A tile row holds NCH 16-byte chunks; chunk c of row r is stored at slot c ^ lds_swz<NCH>(r).
// gfx950's LDS moves 256 B per clock (64 banks): a ds_read_b128 is conflict-free when every 16
// consecutive lanes (16 consecutive rows, same logical chunk) land in 16 different 16-byte bank
// groups, and a ds_read_b64_tr_b16 when the four consecutive rows that 32 lanes touch (64 contiguous
// logical bytes of each) land in four different 64-byte groups.  Both hold with:
//   64-byte rows:  4 rows share 256 B, rows r and r+4 must differ            -> (r >> 2) & 3
//   128-byte rows: rows of equal parity must differ, r and r+2 in bit 2      -> ((r >> 1) & 1) << 2 | (r >> 2) & 3
//   256-byte rows and longer: 16 rows must differ, r..r+3 in bits 2-3        -> (r & 3) << 2 | (r >> 2) & 3
// (measured with ds_read_b128: 220 B/clk per CU, against 120 B/clk for a swizzle by r & 7).
template <int NCH> __device__ __forceinline__ int lds_swz(int r) {
    if constexpr (NCH <= 4) return (r >> 2) & 3;
    else if constexpr (NCH == 8) return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);
    else return ((r & 3) << 2) | ((r >> 2) & 3);
}

// Swizzle for tiles that are only read through ds_read_b64_tr_b16 (the attention V operand): moving
// just the 64-byte group of a row keeps every compile-time part of the read address (tile, key block,
// head-dim block) an immediate offset.
template <int NCH> __device__ __forceinline__ int lds_swz_v(int r) {
    if constexpr (NCH <= 4) return 0;                       // 4 rows are 256 contiguous bytes already
    else if constexpr (NCH == 8) return ((r >> 1) & 1) << 2;
    else return (r & 3) << 2;
}

// the same with a wave-uniform byte offset in a scalar register (address = base + voff + soff).
// For these raw resources the range check is made on voff + soff (a transfer whose scalar part alone
// passes num_records returns zeros: checked on the hardware), so rows past the tensor are never touched.
__device__ __forceinline__ void dma16s(rsrc_words rs, const void* lds_dst_wave_uniform, int voff, int soff) {
    const uint32_t la = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)lds_dst_wave_uniform);
    const int so = __builtin_amdgcn_readfirstlane(soff);
    asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(la), "v"(voff), "s"(rs), "s"(so) : "memory");
}

// Reductions over the two 32-lane halves of a wave (lane i with lane i+32) through the half-swap
// instruction: one VALU operation instead of an LDS permute and its round trip.  After the swap the
// first result holds the lower half's values in both halves, the second the upper half's.
__device__ __forceinline__ float halves_max(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
__device__ __forceinline__ float halves_sum(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}

// All-reduce (sum) over groups of 16, 32 or 64 consecutive lanes without LDS permutes: four rotations
// inside each 16-lane row (DPP operands of the additions), then the row-pair swap and the half swap.
// All lanes of a group must be active.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int LANES> __device__ __forceinline__ float group_sum(float v) {
    static_assert(LANES == 16 || LANES == 32 || LANES == 64, "16, 32 or 64 lanes");
    v += dpp_move<0x128>(v);      // row_ror:8
    v += dpp_move<0x124>(v);      // row_ror:4
    v += dpp_move<0x122>(v);      // row_ror:2
    v += dpp_move<0x121>(v);      // row_ror:1
    if constexpr (LANES >= 32) {
        const unsigned u = __builtin_bit_cast(unsigned, v);
        const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);   // rows (0,1) and (2,3) exchange
        v = __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
    }
    if constexpr (LANES == 64) v = halves_sum(v);
    return v;
}

template <typename T> struct elem;
template <> struct elem<float> {
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct elem<uint16_t> {   // bf16 storage
    static __device__ __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
    static __device__ __forceinline__ void st(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
};

// ---- activation closed forms of the reference shaders
// shaders/fused-linear-gelu.glsl:45-63 and shaders/activation-gelu.glsl:33-50
__device__ __forceinline__ float gelu_ref(float x) {
    float c = fminf(fmaxf(x, -50.0f), 50.0f);
    float inner = 0.7978845608028654f * (c + 0.044715f * (c * c * c));
    float r = 0.5f * x * (1.0f + tanhf(inner));
    if (fabsf(x) > 50.0f) r = x > 0.0f ? x : 0.0f;
    return r;
}
// Fast forms for GEMM epilogues: v_exp_f32 (base 2) and v_rcp_f32, both within 1 ulp, instead
// of the multi-instruction IEEE division.
// shaders/fused-linear-silu.glsl:43-48: x * 1/(1+exp(-clamp(x,-88,88)))
__device__ __forceinline__ float silu_clamped(float x) {
    float c = __builtin_amdgcn_fmed3f(x, -88.0f, 88.0f);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * c));
}
// shaders/fused-swiglu.glsl:44-46: x/(1+exp(-x)); exp overflow gives x*0 = -0 like the division
__device__ __forceinline__ float silu_plain(float x) {
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}
__device__ __forceinline__ void silu_plain4(float (&v)[4]) {       // four values stage by stage, like gelu_fast4 below
    float e[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = __builtin_amdgcn_exp2f(-1.4426950408889634f * v[i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = 1.0f + e[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = __builtin_amdgcn_rcpf(e[i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = v[i] * e[i];
}
// v_mul_legacy_f32 (0 times anything, infinities and NaN included, is 0).  clang has no builtin for it, so it is
// one inline-asm instruction.  The hazard recognizer does not look inside inline asm: a transcendental result (the
// reciprocal below) needs one wait state before an ordinary VALU instruction reads it, hence the leading s_nop.
__device__ __forceinline__ float fmul_legacy(float a, float b) {
    float r;
    asm("s_nop 0\n\tv_mul_legacy_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
// shaders/fused-linear-gelu.glsl:45-63 rewritten with tanh(u) = 2/(1+exp(-2u)) - 1:
//   0.5 x (1 + tanh(u)) = x / (1 + exp(-2u)),  u = sqrt(2/pi) (c + 0.044715 c^3), c = clamp(x, +-50).
// The +-50 clamp needs no instruction of its own: beyond |x| = 50 (already from |x| > 7) the exponential saturates
// to 0 / +inf, also when x*x overflows, which yields x and (-)0: the shader's rule for |x| > 50.  x = -inf would give
// (-inf)*0 = NaN with an IEEE multiply; the last product is v_mul_legacy_f32 (0 times anything is 0), which returns the
// shader's 0 there and is the same product everywhere else; +inf stays +inf.
__device__ __forceinline__ float gelu_fast(float x) {
    float e = x * (-2.302208198f + -0.10294324f * (x * x));     // -2u*log2(e)
    return fmul_legacy(x, __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(e)));
}
// four values stage by stage: the result of an exponential or reciprocal is then never needed by the very next
// instruction (one s_nop per value otherwise, in epilogues that are bound by instruction issue)
__device__ __forceinline__ void gelu_fast4(float (&v)[4]) {
    float e[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = v[i] * (-2.302208198f + -0.10294324f * (v[i] * v[i]));
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = __builtin_amdgcn_exp2f(e[i]);
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = 1.0f + e[i];
#pragma unroll
    for (int i = 0; i < 4; ++i) e[i] = __builtin_amdgcn_rcpf(e[i]);
    // the four products in one statement behind one wait state (whichever reciprocal the scheduler placed last)
    asm("s_nop 0\n\tv_mul_legacy_f32 %0, %0, %4\n\tv_mul_legacy_f32 %1, %1, %5\n\tv_mul_legacy_f32 %2, %2, %6\n\tv_mul_legacy_f32 %3, %3, %7"
        : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]) : "v"(e[0]), "v"(e[1]), "v"(e[2]), "v"(e[3]));
}
#endif
