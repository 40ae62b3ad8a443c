// MFMA GEMM family for gfx950:  C[m,n] = epi( sum_k A[m,k]*W[n,k] + bias[n] )
//
// Both operands are K-contiguous, which is the layout MFMA wants: every lane feeds the
// matrix core 16 contiguous bytes of one row (8 bf16 for v_mfma_f32_32x32x16_bf16, or
// 4 fp32 that drive four v_mfma_f32_32x32x2_f32).  A workgroup owns a BM x BN tile of C
// and walks K in slabs of 128 bytes per row (64 bf16 / 32 fp32):
//
//   HBM --128-bit loads--> VGPR --ds_write_b128--> LDS (2 stages, XOR-swizzled 16-B chunks)
//       --ds_read_b128--> MFMA operands --> fp32 accumulators (registers, never spilled to LDS)
//       --> bias / GELU / SiLU / SwiGLU epilogue in registers --> 8/16-byte stores
//
// The loads for slab t+1 are issued before the MFMAs of slab t and parked in registers, so
// HBM/L2 latency hides behind the matrix work; one barrier per slab.
//
// MFMA operand roles are swapped (the weight rows are the "A" operand, the activation rows
// the "B" operand) so that each lane ends up with 4 consecutive output columns of one
// output row: stores are 8 B (bf16) / 16 B (fp32) wide and bias is a 4-vector per lane.
//
// LDS bank behaviour: a tile row is 128 B = 8 chunks of 16 B; chunk c of row r lives at
// slot c ^ lds_swz<8>(r), which makes 16 consecutive rows of one logical chunk (what 16 lanes of a
// ds_read_b128 fragment read touch) cover all 64 banks exactly once.
#pragma once
#include "common.hpp"
#include <type_traits>
#include <cstdlib>
#include <algorithm>

int grl_transpose2d(grl_ctx* c, int dtype, int64_t R, int64_t C, const void* in, void* out);

struct GemmArgs {
    const void* A;       // (M,K)
    const void* W;       // (N,K)
    const void* W2;      // (N,K) second weight (SwiGLU "up"), else null
    const float* bias;   // (N) or null
    const float* bias2;  // (N) or null
    void* C;             // (M,N)
    float* cache1;       // fp32 (M,N) pre-activation of W  (SwiGLU gate) or null
    float* cache2;       // fp32 (M,N) pre-activation of W2 (SwiGLU up) or null
    int M, N, K;
    int tiles_m, tiles_n;
    int group;           // tile-rows per band of the tile walk
    int act;             // run-time activation code of the EPI_RT / dual epilogues (a GRL_EPI_* value)
    float alpha, beta;   // RoSwish parameters
    const void* residual; // (M,N) of the output type, added to the result (EPI_RES), else null
    // LayerNorm folded into the GEMM (template flag LN): A holds the raw rows, W the weight scaled by gamma;
    // sum_k LN(x)[m,k] W0[n,k] = rstd_m * (acc[m,n] - mean_m * c[n]) + sum_k beta[k] W0[n,k], c[n] = sum_k W[n,k]
    const float* ln_stats; // (M,2): {rstd, rstd*mean} per row
    const float* ln_c;     // (N) column sums of the scaled weight W
    const float* ln_c2;    // (N) the same for W2, else null
    // EPI_RESLN: the residual is LayerNorm(residual) re-formed from the raw rows in `residual`, their statistics and
    // the norm's parameters; the row statistics of the OUTPUT leave the kernel as one partial per (column tile, row)
    const float* res_stats;  // (M,2): {rstd, rstd*mean} of the residual rows
    const float* res_gamma;  // (N)
    const float* res_beta;   // (N)
    float* part_out;         // (tiles_n, M, 2): {sum, sum of squares} of each output row's columns in that tile
    // split K (register-staged 64 x 64 kernel, template flag SPLITK): workgroup (x, y) multiplies the y-th share of the K
    // slabs of tile x and writes its raw fp32 sums to kpart[y]; gemm_splitk_finish_kernel adds the shares and runs the epilogue
    int ksplit;              // number of shares (grid.y)
    float* kpart;            // (ksplit, M, N) fp32
    bool no_alloc;           // host side: the caller must not touch the buffer pool (split K takes its buffer there): no split
};

// Epilogue template codes.  NONE / GELU / SILU are compiled in (the encoder's hot shapes); EPI_RT picks
// ReLU / GCU / RoSwish from GemmArgs::act at run time (one more instantiation instead of three), and the
// dual-weight epilogue EPI_GLU picks the gate activation (SiLU / ReLU / GELU) the same way.
// EPI_RES adds a residual tensor of the output type where the result is stored (C may be the residual itself).
// EPI_RESLN adds LayerNorm(residual) formed on the fly (GemmArgs::res_*) and writes per-tile row statistics of the
// result; only the direct-to-LDS kernels with the LDS-staged epilogue implement it (the host checks).
enum { EPI_NONE = 0, EPI_GELU = 1, EPI_SILU = 2, EPI_RT = 3, EPI_GLU = 4, EPI_RES = 5, EPI_RESLN = 6 };

// shaders/fused-linear-relu.glsl:63, fused-linear-gcu.glsl:44-46 (x*cos(x)), fused-linear-roswish.glsl:46-58
// ((x+alpha)*sigmoid(beta*x) - alpha/2; the shader's sign-split sigmoid equals 1/(1+exp(-beta*x)) with the
// exponential saturating to 0 / +inf)
__device__ __forceinline__ float act_runtime(float v, const GemmArgs& p) {
    if (p.act == GRL_EPI_RELU) return fmaxf(v, 0.0f);
    if (p.act == GRL_EPI_GCU) {
        // cos through the hardware instruction on the fractional number of turns (any finite argument)
        const float turns = v * 0.15915494309189535f;
        return v * __builtin_amdgcn_cosf(__builtin_amdgcn_fractf(turns));
    }
    const float sg = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * (p.beta * v)));
    return (v + p.alpha) * sg - 0.5f * p.alpha;
}
template <int EPI> __device__ __forceinline__ float epi_apply(float v, const GemmArgs& p) {
    if (EPI == EPI_GELU) return gelu_fast(v);
    if (EPI == EPI_SILU) return silu_clamped(v);
    if (EPI == EPI_RT) return act_runtime(v, p);
    return v;
}
// gate * act(up): shaders/fused-swiglu.glsl:44-79 (x/(1+exp(-x))), fused-reglu.glsl:74 (max(0,up)),
// fused-geglu.glsl:44-49,80 (tanh GELU without the clamp rule)
__device__ __forceinline__ float glu_apply(float gate, float up, const GemmArgs& p) {
    if (p.act == GRL_EPI_RELU) return gate * fmaxf(up, 0.0f);
    if (p.act == GRL_EPI_GELU) return gate * gelu_fast(up);
    return gate * silu_plain(up);
}
// the same for four adjacent outputs, the transcendental activations stage by stage (see gelu_fast4)
__device__ __forceinline__ void glu_apply4(float (&gate)[4], float (&up)[4], const GemmArgs& p) {
    if (p.act == GRL_EPI_RELU) {
#pragma unroll
        for (int e = 0; e < 4; ++e) gate[e] *= fmaxf(up[e], 0.0f);
        return;
    }
    if (p.act == GRL_EPI_GELU) gelu_fast4(up);
    else silu_plain4(up);
#pragma unroll
    for (int e = 0; e < 4; ++e) gate[e] *= up[e];
}

// ---- one 128-byte-per-row K slab on the matrix cores --------------------------------------
template <typename T> struct MfmaSlab;
template <> struct MfmaSlab<uint16_t> {   // bf16: 16 B = 8 values, k = 8*(lane/32)+e
    static __device__ __forceinline__ void run(const u32x4& w, const u32x4& x, f32x16& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, x), acc, 0, 0, 0);
    }
    // acc = w.x + c: the first product of a tile starts from c (zeros or the bias) without a copy
    static __device__ __forceinline__ void run_from(const u32x4& w, const u32x4& x, const f32x16& c, f32x16& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, x), c, 0, 0, 0);
    }
};
template <> struct MfmaSlab<float> {      // fp32: 16 B = 4 values, each feeds one 32x32x2 MFMA
    static __device__ __forceinline__ void run(const u32x4& w, const u32x4& x, f32x16& acc) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u2f(w[e]), u2f(x[e]), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ void run_from(const u32x4& w, const u32x4& x, const f32x16& c, f32x16& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u2f(w[0]), u2f(x[0]), c, 0, 0, 0);
#pragma unroll
        for (int e = 1; e < 4; ++e)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u2f(w[e]), u2f(x[e]), acc, 0, 0, 0);
    }
};

// ---- acc[m,n] += xs[m] * ws[n] on the matrix cores (one extra k-slab with register-built operands): the term
// -mean_m * c[n] of the LayerNorm-folded GEMM.  bf16: each factor is split into three bf16 numbers (hi + mid + lo, exact
// to 2^-24) and the nine cross products sit at k = 0..8 of one 32x32x16 instruction (k = 8*(lane/32) + e);
// fp32: one 32x32x2 instruction with the factors at k = 0.
// (conversions through v_cvt_pk_bf16_f32; the value sits in both halves of the returned words)
__device__ __forceinline__ void split3_bf16(float v, uint32_t& hh, uint32_t& mm, uint32_t& ll) {
    hh = pack_bf16x2(v, v);
    const float r1 = v - bf16hi(hh);
    mm = pack_bf16x2(r1, r1);
    const float r2 = r1 - bf16hi(mm);
    ll = pack_bf16x2(r2, r2);
}
__device__ __forceinline__ uint32_t lo_hi(uint32_t a, uint32_t b) { return __builtin_amdgcn_perm(b, a, 0x07060100u); }   // low half of a | high half of b
template <typename T> struct MfmaOuter;
template <> struct MfmaOuter<uint16_t> {
    // activation-row side (MFMA "B" operand): [h,h,h,m,m,m,l,l | l,0,...]
    static __device__ __forceinline__ u32x4 xfrag(float v, int lg) {
        uint32_t h, m, l;
        split3_bf16(v, h, m, l);
        const u32x4 lo = {h, lo_hi(h, m), m, l};
        const u32x4 hi = {l & 0xffffu, 0u, 0u, 0u};
        return lg ? hi : lo;
    }
    // weight-row side (MFMA "A" operand): [h,m,l,h,m,l,h,m | l,0,...]
    static __device__ __forceinline__ u32x4 wfrag(float v, int lg) {
        uint32_t h, m, l;
        split3_bf16(v, h, m, l);
        const uint32_t hm = lo_hi(h, m);
        const u32x4 lo = {hm, lo_hi(l, h), lo_hi(m, l), hm};
        const u32x4 hi = {l & 0xffffu, 0u, 0u, 0u};
        return lg ? hi : lo;
    }
    static __device__ __forceinline__ void run(const u32x4& w, const u32x4& x, f32x16& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w), __builtin_bit_cast(bf16x8, x), acc, 0, 0, 0);
    }
};
template <> struct MfmaOuter<float> {
    static __device__ __forceinline__ u32x4 xfrag(float v, int lg) { return u32x4{lg ? 0u : f2u(v), 0u, 0u, 0u}; }
    static __device__ __forceinline__ u32x4 wfrag(float v, int lg) { return u32x4{lg ? 0u : f2u(v), 0u, 0u, 0u}; }
    static __device__ __forceinline__ void run(const u32x4& w, const u32x4& x, f32x16& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u2f(w[0]), u2f(x[0]), acc, 0, 0, 0);
    }
};

// compile-time loop: f(std::integral_constant<int, 0..N-1>)
template <int N, typename F> __device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

template <typename OutT> __device__ __forceinline__ void store4(OutT* p, float a, float b, float c, float d);
template <> __device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
    f32x4 v = {a, b, c, d};
    *(f32x4*)p = v;
}
template <> __device__ __forceinline__ void store4<uint16_t>(uint16_t* p, float a, float b, float c, float d) {
    u32x2 v = {pack_bf16x2(a, b), pack_bf16x2(c, d)};
    *(u32x2*)p = v;
}

// residual helpers: 4 values of the output type at r added to v; one 16-byte chunk of outputs plus the
// matching residual chunk (8 bf16 or 4 fp32 values, fp32 sum, one rounding)
template <typename OutT> __device__ __forceinline__ void add4(const OutT* r, float (&v)[4]);
template <> __device__ __forceinline__ void add4<float>(const float* r, float (&v)[4]) {
    const f32x4 t = *(const f32x4*)r;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] += t[e];
}
template <> __device__ __forceinline__ void add4<uint16_t>(const uint16_t* r, float (&v)[4]) {
    const u32x2 t = *(const u32x2*)r;
    v[0] += bf16lo(t[0]); v[1] += bf16hi(t[0]); v[2] += bf16lo(t[1]); v[3] += bf16hi(t[1]);
}
template <typename OutT> __device__ __forceinline__ u32x4 add_chunk(u32x4 c, u32x4 r);
template <> __device__ __forceinline__ u32x4 add_chunk<float>(u32x4 c, u32x4 r) {
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = f2u(u2f(c[e]) + u2f(r[e]));
    return o;
}
template <> __device__ __forceinline__ u32x4 add_chunk<uint16_t>(u32x4 c, u32x4 r) {
    u32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t cw = c[e], rw = r[e];
        o[e] = pack_bf16x2(bf16lo(cw) + bf16lo(rw), bf16hi(cw) + bf16hi(rw));
    }
    return o;
}

// one 16-byte chunk of outputs <-> its 8 (bf16) or 4 (fp32) values
template <typename OutT> struct Chunk;
template <> struct Chunk<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void unpack(const u32x4& c, float (&v)[4]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = u2f(c[e]);
    }
    static __device__ __forceinline__ u32x4 pack(const float (&v)[4]) { return u32x4{f2u(v[0]), f2u(v[1]), f2u(v[2]), f2u(v[3])}; }
    // sum and sum of squares of the chunk's values as stored
    static __device__ __forceinline__ void moments(const u32x4&, const float (&v)[4], float& s, float& q) {
#pragma unroll
        for (int e = 0; e < 4; ++e) { s += v[e]; q = fmaf(v[e], v[e], q); }
    }
};
template <> struct Chunk<uint16_t> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void unpack(const u32x4& c, float (&v)[8]) {
#pragma unroll
        for (int e = 0; e < 4; ++e) { const uint32_t w = c[e]; v[2 * e] = bf16lo(w); v[2 * e + 1] = bf16hi(w); }
    }
    static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
        return u32x4{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
    }
    // sum and sum of squares of the chunk's values as stored (the rounded bf16 pairs, two per dot instruction)
    static __device__ __forceinline__ void moments(const u32x4& c, const float (&)[8], float& s, float& q) {
        typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2v;
        const bf16x2v one2 = __builtin_bit_cast(bf16x2v, 0x3f803f80u);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bf16x2v w = __builtin_bit_cast(bf16x2v, (uint32_t)c[e]);
            s = __builtin_amdgcn_fdot2_f32_bf16(w, one2, s, false);
            q = __builtin_amdgcn_fdot2_f32_bf16(w, w, q, false);
        }
    }
};

// ---- direct epilogue: lane (li, lg) holds, for output row m = .. + li, the columns
// n = .. + 8*q + 4*lg + {0..3} in accumulator registers 4q..4q+3 and stores them itself
// (8- or 16-byte stores).  Every index into the accumulators is a compile-time constant so
// they stay in registers.  Used for ragged N, for the SwiGLU pre-activation outputs and by the
// staged kernel.
template <typename OutT, int TM, int TN, int TNO, int WM, int WNO, int EPI, bool DUAL, bool LN = false>
__device__ __forceinline__ void epilogue_direct(f32x16 (&acc)[TM][TN], const GemmArgs& p, int m0, int n0, int wm, int wn, int li, int lg) {
    OutT* C = (OutT*)p.C;
    const bool vec_ok = (p.N & 3) == 0;
    static_for<TM>([&](auto ia) {
        constexpr int a = decltype(ia)::value;
        const int m = m0 + wm * WM + a * 32 + li;
        float rs = 1.f, rsm = 0.f;
        if (LN && m < p.M) { rs = p.ln_stats[2 * (int64_t)m]; rsm = p.ln_stats[2 * (int64_t)m + 1]; }
        static_for<TNO>([&](auto ib) {
            constexpr int b = decltype(ib)::value;
            static_for<4>([&](auto iq) {
                constexpr int q = decltype(iq)::value;
                const int n = n0 + wn * WNO + b * 32 + 8 * q + 4 * lg;
                if (m < p.M && n < p.N) {
                    float v[4], u[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = acc[a][b][4 * q + e];
                        u[e] = DUAL ? acc[a][DUAL ? b + TNO : b][4 * q + e] : 0.f;
                        if (LN && n + e < p.N) {
                            v[e] = v[e] * rs - rsm * p.ln_c[n + e];
                            if (DUAL) u[e] = u[e] * rs - rsm * p.ln_c2[n + e];
                        }
                    }
                    const int64_t o = (int64_t)m * p.N + n;
                    if (vec_ok) {
                        if (p.bias) {
                            f32x4 bv = *(const f32x4*)(p.bias + n);
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] += bv[e];
                        }
                        if (DUAL) {
                            if (p.bias2) {
                                f32x4 bv = *(const f32x4*)(p.bias2 + n);
#pragma unroll
                                for (int e = 0; e < 4; ++e) u[e] += bv[e];
                            }
                            if (p.cache1) store4<float>(p.cache1 + o, v[0], v[1], v[2], v[3]);
                            if (p.cache2) store4<float>(p.cache2 + o, u[0], u[1], u[2], u[3]);
                            glu_apply4(v, u, p);
                        } else {
                            if constexpr (EPI == EPI_GELU) gelu_fast4(v);
                            else
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] = epi_apply<EPI>(v[e], p);
                            if constexpr (EPI == EPI_RES) add4<OutT>((const OutT*)p.residual + o, v);
                        }
                        store4<OutT>(C + o, v[0], v[1], v[2], v[3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if (n + e < p.N) {
                                float x = v[e] + (p.bias ? p.bias[n + e] : 0.f);
                                if (DUAL) {
                                    float y = u[e] + (p.bias2 ? p.bias2[n + e] : 0.f);
                                    if (p.cache1) p.cache1[o + e] = x;
                                    if (p.cache2) p.cache2[o + e] = y;
                                    x = glu_apply(x, y, p);
                                } else {
                                    x = epi_apply<EPI>(x, p);
                                    if constexpr (EPI == EPI_RES) x += elem<OutT>::ld((const OutT*)p.residual + o + e);
                                }
                                elem<OutT>::st(C + o + e, x);
                            }
                        }
                    }
                }
            });
        });
    });
}

// BN counts LDS rows of the weight tile; with DUAL it is 2x the output-column count of the
// tile (first half gate rows, second half up rows).
template <typename T, typename OutT, int BM, int BN, int WGM, int WGN, int EPI, bool DUAL, bool LN = false, bool SPLITK = false>
__global__ __launch_bounds__(WGM * WGN * 64) void gemm_nt_kernel(GemmArgs p) {
    static_assert(!SPLITK || (!DUAL && !LN), "split K: plain single-weight products only (the epilogue runs in the finishing kernel)");
    constexpr int NT = WGM * WGN * 64;
    constexpr int EPC = 16 / (int)sizeof(T);     // elements per 16-byte chunk
    constexpr int BK = 8 * EPC;                  // elements per 128-byte slab row
    constexpr int WM = BM / WGM, WN = BN / WGN;  // per-wave tile (WN in LDS rows)
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int BNO = DUAL ? BN / 2 : BN;      // output columns per tile
    constexpr int WNO = DUAL ? WN / 2 : WN;      // output columns per wave
    constexpr int TNO = DUAL ? TN / 2 : TN;
    constexpr int CA = BM * 8 / NT, CB = BN * 8 / NT;
    static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile rows must divide over the threads");
    static_assert(!DUAL || (BN / 2) % (NT / 8) == 0, "a staging pass must not straddle the two weights");
    static_assert(WM % 32 == 0 && WN % 32 == 0 && (!DUAL || TN % 2 == 0), "wave tile is made of 32x32 MFMA tiles");
    constexpr int STAGE = (BM + BN) * 128;
    __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];

    // the wave index is wave-uniform; telling the compiler so keeps everything derived from it (LDS stage addresses of
    // the transfers, the wave's tile coordinates, the branch that picks the requesting wave) in scalar registers
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int li = lane & 31, lg = lane >> 5;

    // ---- workgroup -> tile: give each XCD (workgroups are dealt round-robin over the 8 XCDs)
    // a contiguous run of tiles, and walk tiles in bands of 8 tile-rows so that the 32 CUs of
    // an XCD share a small set of A and W row panels in their L2.
    int tile_m, tile_n;
    {
        const int nb = gridDim.x, pid = blockIdx.x;
        const int per = nb >> 3, rem = nb & 7, xcd = pid & 7, loc = pid >> 3;
        const int npid = xcd * per + (xcd < rem ? xcd : rem) + loc;
        constexpr int GROUP = 8;
        const int width = GROUP * p.tiles_n;
        const int first_m = (npid / width) * GROUP;
        const int gsize = p.tiles_m - first_m < GROUP ? p.tiles_m - first_m : GROUP;
        tile_m = first_m + (npid % width) % gsize;
        tile_n = (npid % width) / gsize;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BNO;

    // ---- global -> register staging through buffer loads: the resource starts at the tile's
    // first row and ends with the tensor, so rows past the edge read as zero in hardware; the
    // slab offset travels in a scalar register.  Thread t owns chunk (t & 7) of row (t >> 3)
    // of every 32-row pass; K chunks past the end are zeroed when the slab is written to LDS.
    constexpr int RPP = NT / 8;                   // rows per pass
    const int row_t = tid >> 3, c_t = tid & 7;
    const int64_t rowbytes = (int64_t)p.K * (int64_t)sizeof(T);
    auto make_rsrc = [&](const void* base, int first_row, int rows_total) {
        int64_t left = (int64_t)(rows_total - first_row) * rowbytes;
        if (left < 0) left = 0;
        uint32_t nrec = left > 0xffffffffLL ? 0xffffffffu : (uint32_t)left;
        return __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)base + (int64_t)first_row * rowbytes), 0, (int)nrec, 0x00020000);
    };
    const __amdgpu_buffer_rsrc_t rsA = make_rsrc(p.A, m0, p.M);
    const __amdgpu_buffer_rsrc_t rsW = make_rsrc(p.W, n0, p.N);
    const __amdgpu_buffer_rsrc_t rsW2 = make_rsrc(DUAL ? p.W2 : p.W, n0, p.N);
    const int voff = row_t * (int)rowbytes + c_t * 16;
    const int pass_stride = RPP * (int)rowbytes;
    static_assert(RPP % 16 == 0, "the swizzle repeats every 16 rows");
    const int soff_t = row_t * 128 + ((c_t ^ lds_swz<8>(row_t)) << 4);

    u32x4 ra[CA], rb[CB];
    auto load_slab = [&](int kt) {
        const int sbyte = kt * 128;
#pragma unroll
        for (int i = 0; i < CA; ++i)
            ra[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsA, voff + i * pass_stride, sbyte, 0));
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const bool second = DUAL && (i * RPP >= BNO);
            const int vo = voff + (second ? i - BNO / RPP : i) * pass_stride;
            rb[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(second ? rsW2 : rsW, vo, sbyte, 0));
        }
    };
    // the K-tail select sits here, after the MFMAs of the previous slab, so that nothing
    // between the load and this point waits on the data
    auto stash_slab = [&](int kt) {
        char* s = lds + (kt & 1) * STAGE + soff_t;
        const bool live = kt * BK + c_t * EPC < p.K;
        const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < CA; ++i) *(u32x4*)(s + i * RPP * 128) = live ? ra[i] : zero;
#pragma unroll
        for (int i = 0; i < CB; ++i) *(u32x4*)(s + BM * 128 + i * RPP * 128) = live ? rb[i] : zero;
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

    // LDS row of this lane inside each 32-row operand tile
    int rowX[TM], rowW[TN];
#pragma unroll
    for (int a = 0; a < TM; ++a) rowX[a] = wm * WM + a * 32 + li;
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        int base = DUAL ? ((b >= TNO ? BNO : 0) + wn * WNO + (b % TNO) * 32) : (wn * WN + b * 32);
        rowW[b] = base + li;
    }

    const int KT = (p.K + BK - 1) / BK;
    int kt0 = 0, kt1 = KT;
    if constexpr (SPLITK) {                       // this workgroup's share of the slabs (the host leaves no share empty)
        const int per = (KT + p.ksplit - 1) / p.ksplit;
        kt0 = (int)blockIdx.y * per;
        kt1 = kt0 + per < KT ? kt0 + per : KT;
    }
    load_slab(kt0);
    stash_slab(kt0);
    __syncthreads();
    for (int kt = kt0; kt < kt1; ++kt) {
        const bool more = kt + 1 < kt1;
        if (more) load_slab(kt + 1);
        const char* s = lds + (kt & 1) * STAGE;
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            const int ch = 2 * sl + lg;
            u32x4 xf[TM], wf[TN];
#pragma unroll
            for (int a = 0; a < TM; ++a) xf[a] = *(const u32x4*)(s + rowX[a] * 128 + ((ch ^ lds_swz<8>(rowX[a])) << 4));
#pragma unroll
            for (int b = 0; b < TN; ++b) wf[b] = *(const u32x4*)(s + BM * 128 + rowW[b] * 128 + ((ch ^ lds_swz<8>(rowW[b])) << 4));
            static_for<TM>([&](auto ia) {
                static_for<TN>([&](auto ib) {
                    MfmaSlab<T>::run(wf[decltype(ib)::value], xf[decltype(ia)::value], acc[decltype(ia)::value][decltype(ib)::value]);
                });
            });
        }
        if (more) stash_slab(kt + 1);
        __syncthreads();
    }

    if constexpr (SPLITK) {
        GemmArgs q = p;                            // raw sums of this share, fp32, no bias / activation / residual
        q.C = p.kpart + (int64_t)blockIdx.y * p.M * p.N;
        q.bias = nullptr;
        epilogue_direct<float, TM, TN, TNO, WM, WNO, EPI_NONE, false, false>(acc, q, m0, n0, wm, wn, li, lg);
    } else {
        epilogue_direct<OutT, TM, TN, TNO, WM, WNO, EPI, DUAL, LN>(acc, p, m0, n0, wm, wn, li, lg);
    }
}

// Second half of a split-K product: C = epilogue(sum of the shares + bias) (+ residual), four adjacent outputs per thread
// (N is a multiple of 4 here).  The shares are added in ascending order, so the result does not depend on scheduling.
template <typename OutT, int EPI>
__global__ __launch_bounds__(256) void gemm_splitk_finish_kernel(GemmArgs p) {
    const int64_t quads = (int64_t)p.M * p.N / 4;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= quads) return;
    const int64_t o = i * 4;
    const int n = (int)(o % p.N);
    f32x4 acc = *(const f32x4*)(p.kpart + o);
    for (int sidx = 1; sidx < p.ksplit; ++sidx) {
        const f32x4 t = *(const f32x4*)(p.kpart + (int64_t)sidx * p.M * p.N + o);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] += t[e];
    }
    float v[4] = {acc[0], acc[1], acc[2], acc[3]};
    if (p.bias) {
        const f32x4 bv = *(const f32x4*)(p.bias + n);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += bv[e];
    }
    if constexpr (EPI == EPI_GELU) gelu_fast4(v);
    else
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = epi_apply<EPI>(v[e], p);
    if constexpr (EPI == EPI_RES) add4<OutT>((const OutT*)p.residual + o, v);
    store4<OutT>((OutT*)p.C + o, v[0], v[1], v[2], v[3]);
}

// =====================================================================================
// Main kernel: persistent workgroups, global -> LDS without passing through registers.
//
//   buffer_load_dwordx4 ... lds   writes each wave's 64 x 16 B straight into 1 KiB of LDS
//   (8 tile rows); the lane -> chunk assignment carries the XOR swizzle, so the LDS image is
//   the same as in the staged kernel above and the MFMA fragment reads are unchanged.
//   No staging VGPRs, no ds_write, no select: the slab t+1 transfer runs entirely under the
//   MFMAs of slab t.  8 waves per 256x256 tile (2 per SIMD) so that one wave's LDS waits hide
//   under the other's matrix work.
//
//   One workgroup per CU walks over its tiles.  When a tile's K loop ends, the first slab of
//   the NEXT tile is already requested into LDS stage 0 before the epilogue starts, so its
//   HBM/L2 latency hides under the epilogue, which stages the output through LDS stage 1.
//
//   Needs K to be a whole number of 128-byte slabs (the transfer cannot zero a K tail);
//   M and N are free: rows past the edge are out of range for the buffer resource, read as
//   zero, and feed only accumulators that are never stored.
//
//   Epilogue: accumulators -> bias/activation -> OutT -> LDS (row-major, 16-byte chunks XOR
//   swizzled by row) -> 16-byte row-contiguous global stores, 32 output rows per wave-row
//   per pass, two staging regions used alternately so a pass costs one barrier.
// =====================================================================================
// (launch bounds: the four-wave workgroups of the 128 x 128 tiles run two to a CU, i.e. two waves per SIMD, like the one
// eight-wave workgroup of the 256 x 256 tiles: the register budget is 256 per lane either way, and an instantiation that
// would take more must spill rather than halve the occupancy)
template <typename T, typename OutT, int BM, int BN, int WGM, int WGN, int EPI, bool DUAL, bool LN = false>
__global__ __launch_bounds__(WGM * WGN * 64, (WGM * WGN <= 4 ? 2 : 1)) void gemm_nt_dma_kernel(GemmArgs p) {
    constexpr int NW = WGM * WGN, NT = NW * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int BNO = DUAL ? BN / 2 : BN;
    constexpr int WNO = DUAL ? WN / 2 : WN;
    constexpr int TNO = DUAL ? TN / 2 : TN;
    constexpr int GA = BM / 8 / NW, GB = BN / 8 / NW;      // 8-row groups per wave
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "row groups must divide over the waves");
    static_assert(!DUAL || (NW % 2 == 0), "the two weights split the waves evenly");
    constexpr int STAGE = (BM + BN) * 128;
    constexpr int OES = (int)sizeof(OutT);
    constexpr int CROWB = BNO * OES;                        // bytes per staged output row
    constexpr int CPR = CROWB / 16;                         // 16-byte chunks per staged row
    constexpr int RG = WGM * 32 * CROWB;                    // one staging region
    constexpr int NREG = 2 * RG <= STAGE ? 2 : 1;
    static_assert(RG <= STAGE && (CPR & (CPR - 1)) == 0, "output staging must fit in LDS stage 1");
    // one tile's per-column vectors, fp32: bias slice(s); with LN also the column sums c (c2) behind them and the
    // tile's BM row-statistics pairs
    constexpr int COLB = BN * 4;
    constexpr bool RL = EPI == EPI_RESLN;                   // LayerNorm(residual) formed in the epilogue + row statistics out
    static_assert(!(LN && RL) && !(RL && DUAL), "one set of row statistics per tile");
    constexpr int BIASB = (LN || RL) ? 2 * COLB + BM * 8 : COLB;
    static_assert(!LN || NW >= 4, "the per-tile vectors are fetched by distinct waves");
    __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE + 2 * BIASB];

    // the wave index is wave-uniform; telling the compiler so keeps everything derived from it (LDS stage addresses of
    // the transfers, the wave's tile coordinates, the branch that picks the requesting wave) in scalar registers
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int li = lane & 31, lg = lane >> 5;
    const int ntiles = p.tiles_m * p.tiles_n;

    // workgroup id -> tile: give each XCD (workgroup ids are dealt round-robin over the 8 XCDs,
    // and the persistent stride is a multiple of 8) a contiguous run of tiles, walked in bands
    // of 8 tile-rows so that the 32 CUs of an XCD share few A and W row panels in their L2.
    auto tile_of = [&](int pid, int& m0, int& n0) {
        const int per = ntiles >> 3, rem = ntiles & 7, xcd = pid & 7, loc = pid >> 3;
        const int npid = xcd * per + (xcd < rem ? xcd : rem) + loc;
        const int GROUP = p.group;
        const int width = GROUP * p.tiles_n;
        const int first_m = (npid / width) * GROUP;
        const int gsize = p.tiles_m - first_m < GROUP ? p.tiles_m - first_m : GROUP;
        m0 = (first_m + (npid % width) % gsize) * BM;
        n0 = ((npid % width) / gsize) * BNO;
    };

    const int64_t rowbytes = (int64_t)p.K * (int64_t)sizeof(T);
    auto make_rsrc = [&](const void* base, int first_row, int rows_total) {
        int64_t left = (int64_t)(rows_total - first_row) * rowbytes;
        if (left < 0) left = 0;
        uint32_t nrec = left > 0xffffffffLL ? 0xffffffffu : (uint32_t)left;
        return __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)base + (int64_t)first_row * rowbytes), 0, (int)nrec, 0x00020000);
    };
    // with two weights the lower half of the waves fetches the gate rows, the upper half the up rows
    const bool second = DUAL && (wave >= NW / 2);
    const void* Wsrc = second ? p.W2 : p.W;
    const int lr = lane >> 3, ls = lane & 7;
    // lane -> (row lr of an 8-row group, slot ls): LDS slot ls of row r holds chunk ls ^ lds_swz<8>(r).
    // The swizzle depends on bits 1-3 of r, i.e. on lr and on whether the group is an even or odd one.
    static_assert(GA % 2 == 0 && GB % 2 == 0, "group parity is the transfer index parity");
    const int lane_off_p[2] = {lr * (int)rowbytes + ((ls ^ lds_swz<8>(lr)) << 4), lr * (int)rowbytes + ((ls ^ lds_swz<8>(8 + lr)) << 4)};
    const int a_row0 = wave * GA * 8;                                    // first A tile row of this wave
    const int b_row0_lds = wave * GB * 8;                                // LDS row in the weight region
    const int b_row0_glb = second ? b_row0_lds - BNO : b_row0_lds;       // row relative to n0 in its matrix

    // the transfers of wave v's share of slab kt (v is wave-uniform; sec: v's weight rows come from W2)
    auto issue_for = [&](__amdgpu_buffer_rsrc_t rsA, __amdgpu_buffer_rsrc_t rsWv, int kt, int v, bool sec) {
        char* st = lds + (kt & 1) * STAGE;
        const int sbyte = kt * 128;
        const int ar = v * GA * 8, br = v * GB * 8, bg = sec ? br - BNO : br;
#pragma unroll
        for (int j = 0; j < GA; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsA, (__attribute__((address_space(3))) void*)(st + (ar + j * 8) * 128), 16,
                                                     lane_off_p[j & 1] + (ar + j * 8) * (int)rowbytes, sbyte, 0, 0);
#pragma unroll
        for (int j = 0; j < GB; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsWv, (__attribute__((address_space(3))) void*)(st + BM * 128 + (br + j * 8) * 128), 16,
                                                     lane_off_p[j & 1] + (bg + j * 8) * (int)rowbytes, sbyte, 0, 0);
    };
    auto issue = [&](__amdgpu_buffer_rsrc_t rsA, __amdgpu_buffer_rsrc_t rsW, int kt) { issue_for(rsA, rsW, kt, wave, second); };
    // Inside the K loop of the 8-wave workgroup only one wave of each SIMD requests the next slab, for itself
    // and for its SIMD partner (waves w and w^4 share a SIMD), and the two take turns slab by slab: the
    // requesting wave sits in instruction issue while the address unit works through the queue (measured:
    // that queue is full 60 % of the time), and its partner keeps the matrix core busy meanwhile.
    constexpr bool PAIRED = NW == 8;
    const int pw = wave ^ 4;
    const bool second_p = DUAL && (pw >= NW / 2);
    const void* Wsrc_p = second_p ? p.W2 : p.W;

    // The bias slice of a tile travels to LDS with the tile's first slab (two buffers, alternating per
    // tile), so the epilogue reads it with LDS latency instead of one global round trip per column group.
    // Wave 0 fetches bias[n0 .. n0+BNO), the first wave of the upper half bias2 (columns past N read zero).
    auto issue_bias = [&](int n0t, int buf) {
        const bool w1 = wave == 0 && p.bias, w2 = DUAL && wave == NW / 2 && p.bias2;
        if ((w1 || w2) && lane < BNO / 4) {
            const float* src = (w2 ? p.bias2 : p.bias) + n0t;
            int left = (p.N - n0t) * 4;
            __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, left > 0 ? left : 0, 0x00020000);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void*)(lds + 2 * STAGE + buf * BIASB + (w2 ? BNO * 4 : 0)),
                                                     16, lane * 16, 0, 0, 0);
        }
        if constexpr (LN) {
            // wave 1: c[n0 .. n0+BNO), the second wave of the upper half: c2
            const bool w3 = wave == 1, w4 = DUAL && wave == NW / 2 + 1;
            if ((w3 || w4) && lane < BNO / 4) {
                const float* src = (w4 ? p.ln_c2 : p.ln_c) + n0t;
                int left = (p.N - n0t) * 4;
                __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, left > 0 ? left : 0, 0x00020000);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void*)(lds + 2 * STAGE + buf * BIASB + COLB + (w4 ? BNO * 4 : 0)),
                                                         16, lane * 16, 0, 0, 0);
            }
        }
    };
    // rows m0t .. m0t+BM of the statistics (rows past M read zero), fetched by the last wave
    auto issue_stats = [&](int m0t, int buf) {
        if constexpr (LN || RL) {
            if (wave == NW - 1) {
                int left = (p.M - m0t) * 8;
                const float* sbase = LN ? p.ln_stats : p.res_stats;
                __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc((void*)(sbase + 2 * (int64_t)m0t), 0, left > 0 ? left : 0, 0x00020000);
#pragma unroll
                for (int j = 0; j < BM * 8 / 1024; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (__attribute__((address_space(3))) void*)(lds + 2 * STAGE + buf * BIASB + 2 * COLB + j * 1024),
                                                             16, lane * 16, j * 1024, 0, 0);      // one per-lane offset for every transfer of the tile's vectors
            }
        }
    };

    int rowX[TM], rowW[TN];
#pragma unroll
    for (int a = 0; a < TM; ++a) rowX[a] = wm * WM + a * 32 + li;
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        int base = DUAL ? ((b >= TNO ? BNO : 0) + wn * WNO + (b % TNO) * 32) : (wn * WN + b * 32);
        rowW[b] = base + li;
    }

    constexpr int BKE = 128 / (int)sizeof(T);
    const int KT = p.K / BKE;
    OutT* C = (OutT*)p.C;
    const bool staged = ((int64_t)p.N * OES) % 16 == 0 && !p.cache1 && !p.cache2;

    int pid = blockIdx.x;
    int m0, n0;
    tile_of(pid, m0, n0);
    __amdgpu_buffer_rsrc_t rsA = make_rsrc(p.A, m0, p.M);
    __amdgpu_buffer_rsrc_t rsW = make_rsrc(Wsrc, n0, p.N);
    __amdgpu_buffer_rsrc_t rsWp = make_rsrc(Wsrc_p, n0, p.N);
    issue(rsA, rsW, 0);
    int bbuf = 0;
    issue_bias(n0, bbuf);
    issue_stats(m0, bbuf);

    for (;;) {
        // not zeroed: the first slab's multiplications start every accumulator from a constant zero
        f32x16 acc[TM][TN];

        // where the next tile is: index arithmetic done here hides under the wait for the first slab
        const int npid = pid + (int)gridDim.x;
        const bool has_next = npid < ntiles;
        int m0n = 0, n0n = 0;
        __amdgpu_buffer_rsrc_t rsAn = rsA, rsWn = rsW, rsWpn = rsWp;
        if (has_next) {
            tile_of(npid, m0n, n0n);
            rsAn = make_rsrc(p.A, m0n, p.M);
            rsWn = make_rsrc(Wsrc, n0n, p.N);
            rsWpn = make_rsrc(Wsrc_p, n0n, p.N);
        }

        __builtin_amdgcn_s_waitcnt(0x0f70);      // vmcnt(0): this wave's transfers (and earlier stores) are done
        __syncthreads();                         // ... and everybody else's; all staging reads of the last tile too
        // What every accumulator block starts from: the bias of its columns when the LDS-staged epilogue follows (the first
        // MFMA of a block takes it as its C operand, so the epilogue has no bias add left), else zeros (the direct
        // epilogue adds the bias itself; the folded LayerNorm scales the sum before its bias).  Accumulator register
        // 4q+e of block b holds column 8q + 4*(lane/32) + e of the block.
        constexpr bool BIASC = !LN;
        f32x16 c0[TN];
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) c0[b][r] = 0.f;
        if (BIASC && staged) {
            const char* bl = lds + 2 * STAGE + bbuf * BIASB;
#pragma unroll
            for (int b = 0; b < TN; ++b) {
                const bool up = DUAL && b >= TNO;
                const float* bsrc = up ? p.bias2 : p.bias;
                if (bsrc) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int nl = wn * WNO + (b % TNO) * 32 + 8 * q + 4 * lg;
                        const f32x4 v = *(const f32x4*)(bl + (up ? BNO * 4 : 0) + nl * 4);
#pragma unroll
                        for (int e = 0; e < 4; ++e) c0[b][4 * q + e] = v[e];
                    }
                }
                if constexpr (RL) {
                    // the beta of the LayerNorm that the epilogue re-forms on the residual is a per-column constant too
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int n = n0 + wn * WNO + b * 32 + 8 * q + 4 * lg;      // N is a multiple of 4 here
                        if (n < p.N) {
                            const f32x4 v = *(const f32x4*)(p.res_beta + n);
#pragma unroll
                            for (int e = 0; e < 4; ++e) c0[b][4 * q + e] += v[e];
                        }
                    }
                }
            }
        }
        auto k_slab = [&](int kt, auto ifirst) {
            constexpr bool FIRST = decltype(ifirst)::value;
            if (kt + 1 < KT) {
                if (!PAIRED) issue(rsA, rsW, kt + 1);
                else if (((wave >> 2) & 1) == (kt & 1)) {
                    issue_for(rsA, rsW, kt + 1, wave, second);
                    issue_for(rsA, rsWp, kt + 1, pw, second_p);
                }
            }
            const char* s = lds + (kt & 1) * STAGE;
            auto load_frags = [&](int sl, u32x4 (&xf)[TM], u32x4 (&wf)[TN]) {
                const int ch = 2 * sl + lg;
#pragma unroll
                for (int a = 0; a < TM; ++a) xf[a] = *(const u32x4*)(s + rowX[a] * 128 + ((ch ^ lds_swz<8>(rowX[a])) << 4));
#pragma unroll
                for (int b = 0; b < TN; ++b) wf[b] = *(const u32x4*)(s + BM * 128 + rowW[b] * 128 + ((ch ^ lds_swz<8>(rowW[b])) << 4));
            };
            auto run_mfmas = [&](int sl, const u32x4 (&xf)[TM], const u32x4 (&wf)[TN]) {
                static_for<TM>([&](auto ia) {
                    static_for<TN>([&](auto ib) {
                        constexpr int a = decltype(ia)::value, b = decltype(ib)::value;
                        if (FIRST && sl == 0) MfmaSlab<T>::run_from(wf[b], xf[a], c0[b], acc[a][b]);
                        else MfmaSlab<T>::run(wf[b], xf[a], acc[a][b]);
                    });
                });
            };
            // Two fragment sets: the LDS reads of the next 16-deep step are issued in front of this step's eight MFMAs, and
            // fences keep the scheduler from regrouping them (left to itself it sinks the reads to save registers, down to
            // one activation fragment at a time and a wait in front of every second MFMA in the kernels with the larger
            // epilogues; pinned and double-buffered, every GEMM here gains 3 to 8 %).
            u32x4 xf[2][TM], wf[2][TN];
            load_frags(0, xf[0], wf[0]);
#pragma unroll
            for (int sl = 0; sl < 4; ++sl) {
                if (sl + 1 < 4) load_frags(sl + 1, xf[(sl + 1) & 1], wf[(sl + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
                run_mfmas(sl, xf[sl & 1], wf[sl & 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_waitcnt(0x0f70);
            __syncthreads();
        };
        if (LN && staged) {
            // Folded LayerNorm: sum_k LN(x)[m,k] W0[n,k] = rstd_m * (acc[m,n] - mean_m * c[n]) + b'[n].  The outer product
            // -mean_m * c[n] is what the accumulators start from: one MFMA per 32x32 block whose operands are built from
            // the tile's row statistics and column sums (they arrived in LDS with the first slab).  What is left for
            // the epilogue is one multiply-add per element, the instruction count of the plain bias add.
            if constexpr (LN) {
                const char* bl = lds + 2 * STAGE + bbuf * BIASB;
                const float* stl = (const float*)(bl + 2 * COLB);
                const float* cl = (const float*)(bl + COLB);
                u32x4 xm[TM], wc[TN];
#pragma unroll
                for (int a = 0; a < TM; ++a) {
                    const float rs = stl[2 * rowX[a]], rsm = stl[2 * rowX[a] + 1];
                    // -mean = -(mean/sd) / (1/sd); rows past M carry zero statistics (0 * 1/0 = NaN in rows that are never stored)
                    xm[a] = MfmaOuter<T>::xfrag(-rsm * __builtin_amdgcn_rcpf(rs), lg);
                }
#pragma unroll
                for (int b = 0; b < TN; ++b) wc[b] = MfmaOuter<T>::wfrag(cl[rowW[b]], lg);
                static_for<TM>([&](auto ia) {
                    static_for<TN>([&](auto ib) {
                        constexpr int a = decltype(ia)::value, b = decltype(ib)::value;
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
                        MfmaOuter<T>::run(wc[b], xm[a], acc[a][b]);
                    });
                });
            }
            k_slab(0, std::false_type{});
        } else {
            k_slab(0, std::true_type{});          // the host never launches this kernel with K == 0
        }
        for (int kt = 1; kt < KT; ++kt) k_slab(kt, std::false_type{});

        // both LDS stages are free now: request the next tile's first slab into stage 0
        auto issue_next = [&]() {
            if (has_next) {
                issue(rsAn, rsWn, 0);
                issue_bias(n0n, bbuf ^ 1);
                issue_stats(m0n, bbuf ^ 1);
            }
        };

        if (staged) {
            // ---- LDS-staged epilogue in stage 1, one 32-row band of every wave-row per pass
            constexpr int EPCO = 16 / OES;
            char* stg = lds + STAGE;
            const char* bias_lds = lds + 2 * STAGE + bbuf * BIASB;
            // bias of this lane's 4-column groups, once per tile (columns past N hold zero)
            // (the dual-weight kernel with the folded LayerNorm reads them from LDS where they are used instead: two bias
            // sets in registers next to its two accumulator sets and the row factor do not fit)
            constexpr bool BREG = LN && !DUAL;         // (without the folded LayerNorm the bias is in the accumulators already)
            f32x4 bv1[BREG ? TNO : 1][4], bv2[BREG ? TNO : 1][4];
            if constexpr (BREG) {
#pragma unroll
                for (int b = 0; b < TNO; ++b)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int nl = wn * WNO + b * 32 + 8 * q + 4 * lg;
                        bv1[b][q] = p.bias ? *(const f32x4*)(bias_lds + nl * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
                        if (DUAL) bv2[b][q] = p.bias2 ? *(const f32x4*)(bias_lds + BNO * 4 + nl * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
                    }
            }
            // LN: 1/sd of this lane's row in each of the TM bands, read up front (a read inside the band loop would make the
            // loop wait for the staged rows that are on their way back from LDS at that point)
            float rsv[LN ? TM : 1];
            if constexpr (LN) {
#pragma unroll
                for (int a = 0; a < TM; ++a) rsv[a] = ((const float*)(bias_lds + 2 * COLB))[2 * (wm * WM + a * 32 + li)];
            }
            constexpr int TOTAL = WGM * 32 * CPR;
            static_assert(TOTAL % NT == 0, "staged chunks divide over the threads");
            constexpr int PER = TOTAL / NT;
            const int r_w = wm * 32 + li;
            // bias/activation/convert band `a` of every wave-row into its staging region.  Columns past N
            // carry zero accumulators (their weight rows read as zero); they are converted like the rest
            // and dropped at the global store.
            auto stage_band = [&](auto ia) {
                constexpr int a = decltype(ia)::value;
                char* crow = stg + (NREG == 2 ? (a & 1) * RG : 0) + r_w * CROWB;
                const float rs = LN ? rsv[LN ? a : 0] : 1.f;
                static_for<TNO>([&](auto ib) {
                    constexpr int b = decltype(ib)::value;
                    static_for<4>([&](auto iq) {
                        constexpr int q = decltype(iq)::value;
                        const int nl = wn * WNO + b * 32 + 8 * q + 4 * lg;
                        float v[4];
                        f32x4 b1 = {0.f, 0.f, 0.f, 0.f}, b2 = {0.f, 0.f, 0.f, 0.f};
                        if constexpr (BREG) {
                            b1 = bv1[BREG ? b : 0][q];
                        } else if constexpr (LN) {
                            b1 = *(const f32x4*)(bias_lds + nl * 4);            // the folded biases always exist
                            b2 = *(const f32x4*)(bias_lds + BNO * 4 + nl * 4);
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = LN ? acc[a][b][4 * q + e] * rs + b1[e] : acc[a][b][4 * q + e];
                        if (DUAL) {
                            float up[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                up[e] = acc[a][DUAL ? b + TNO : b][4 * q + e];
                                if constexpr (LN) up[e] = up[e] * rs + b2[e];
                            }
                            glu_apply4(v, up, p);
                        } else {
                            if constexpr (EPI == EPI_GELU) gelu_fast4(v);
                            else
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] = epi_apply<EPI>(v[e], p);
                        }
                        const int byte = nl * OES;
                        const int chunk = (byte >> 4) ^ (r_w & (CPR - 1));
                        store4<OutT>((OutT*)(crow + (chunk << 4) + (byte & 15)), v[0], v[1], v[2], v[3]);
                    });
                });
            };
            auto fetch_band = [&](auto ia, u32x4 (&val)[PER]) {
                constexpr int a = decltype(ia)::value;
                const char* reg = stg + (NREG == 2 ? (a & 1) * RG : 0);
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    const int id = tid + i * NT;
                    const int r = id / CPR, cc = id % CPR;
                    val[i] = *(const u32x4*)(reg + r * CROWB + ((cc ^ (r & (CPR - 1))) << 4));
                }
            };
            // EPI_RES: this thread's residual chunks of band a, requested while the band is still on its way
            // through LDS (chunks outside the matrix are not read)
            // EPI_RESLN: this thread's columns are the same in every chunk it handles (the chunk index advances by a
            // multiple of the chunks per row), so the norm's gamma / beta for them are loaded once per tile
            static_assert(NT % CPR == 0, "a thread keeps its chunk column");
            float gq[RL ? EPCO : 1];
            if constexpr (RL) {
                const int nq = n0 + (tid % CPR) * EPCO;          // N is a multiple of the chunk here: whole chunks in or out
#pragma unroll
                for (int e = 0; e < EPCO; e += 4) {
                    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                    const f32x4 gv = nq + e < p.N ? *(const f32x4*)(p.res_gamma + nq + e) : zero;
#pragma unroll
                    for (int k = 0; k < 4; ++k) gq[e + k] = gv[k];
                }
            }
            // last step of a staged chunk: residual (plain, or LayerNorm re-formed from the raw residual rows and
            // their statistics in LDS), the tile's share of the output row statistics, and the global store.
            // Called by every lane for the same (a, i): the row reduction runs over the CPR lanes that hold one row.
            auto fetch_rstats = [&](auto ia, f32x2_t (&rst)[PER]) {
                constexpr int a = decltype(ia)::value;
                if constexpr (RL) {
#pragma unroll
                    for (int i = 0; i < PER; ++i) {
                        const int r = (tid + i * NT) / CPR;
                        rst[i] = *(const f32x2_t*)(bias_lds + 2 * COLB + 8 * ((r >> 5) * WM + a * 32 + (r & 31)));
                    }
                }
            };
            auto emit = [&](auto ia, int i, u32x4 out, u32x4 rres, f32x2_t rstat) {
                constexpr int a = decltype(ia)::value;
                const int id = tid + i * NT;
                const int r = id / CPR, cc = id % CPR;
                const int rt = (r >> 5) * WM + a * 32 + (r & 31);
                const int m = m0 + rt;
                const int n = n0 + cc * EPCO;
                const bool in = m < p.M && n < p.N;
                if constexpr (EPI == EPI_RES) {
                    out = add_chunk<OutT>(out, rres);
                    // keep the sum in front of the range test: sunk into the conditional store, every chunk's first use of
                    // its residual registers sits behind a branch, and the wait-count pass then puts a full vmcnt(0) (which
                    // also waits for the stores of the chunks before) in front of each of them
                    uint32_t o0 = out[0], o1 = out[1], o2 = out[2], o3 = out[3];
                    asm volatile("" : "+v"(o0), "+v"(o1), "+v"(o2), "+v"(o3));
                    out = u32x4{o0, o1, o2, o3};
                }
                if constexpr (RL) {
                    const float rs = rstat[0], rsm = rstat[1];
                    float xr[EPCO], g[EPCO], o[EPCO];
                    Chunk<OutT>::unpack(rres, xr);
                    Chunk<OutT>::unpack(out, g);
                    // sum and sum of squares of the row's columns in this tile (columns past N contribute 0: gamma, beta,
                    // bias and the products are 0 there); the two reductions are independent and interleave
                    // (the norm's beta travels with the bias in the accumulators' starting values)
                    float sum = 0.f, sq = 0.f;
#pragma unroll
                    for (int e = 0; e < EPCO; ++e) o[e] = fmaf(fmaf(xr[e], rs, -rsm), gq[e], g[e]);
                    out = Chunk<OutT>::pack(o);
                    Chunk<OutT>::moments(out, o, sum, sq);
                    sum = group_sum<CPR>(sum);
                    sq = group_sum<CPR>(sq);
                    if (cc == 0 && m < p.M) {
                        const f32x2_t pr = {sum, sq};
                        *(f32x2_t*)(p.part_out + ((int64_t)(n0 / BNO) * p.M + m) * 2) = pr;
                    }
                }
                // written once, read by another kernel: keep it from displacing the operand panels in L2
                if (in) __builtin_nontemporal_store(out, (u32x4*)(C + (int64_t)m * p.N + n));
            };
            auto fetch_res = [&](auto ia, u32x4 (&res)[PER]) {
                constexpr int a = decltype(ia)::value;
                if constexpr (EPI == EPI_RES || RL) {
#pragma unroll
                    for (int i = 0; i < PER; ++i) {
                        const int id = tid + i * NT;
                        const int r = id / CPR, cc = id % CPR;
                        const int m = m0 + (r >> 5) * WM + a * 32 + (r & 31);
                        const int n = n0 + cc * EPCO;
                        res[i] = u32x4{0u, 0u, 0u, 0u};
                        if (m < p.M && n < p.N) res[i] = __builtin_nontemporal_load((const u32x4*)((const OutT*)p.residual + (int64_t)m * p.N + n));
                    }
                }
            };
            auto store_band = [&](auto ia, const u32x4 (&val)[PER], const u32x4 (&res)[PER], const f32x2_t (&rst)[PER]) {
#pragma unroll
                for (int i = 0; i < PER; ++i) emit(ia, i, val[i], res[i], rst[i]);
            };
            // Barriers here are LDS-only (a fence would also wait for the global stores of earlier bands).
            if constexpr (NREG == 2) {
                // two regions: band a+1 is converted and written while band a's staged rows are on their
                // way back from LDS, one barrier per band.
                // Residual chunks: the memory counter retires in issue order, so a load requested behind a band's stores
                // can only be waited for together with those stores (a round trip to HBM per band).  All of the tile's
                // residual chunks are therefore requested before its first store: the first RESAHEAD bands up front, the
                // rest as soon as the accumulators of the bands already staged have freed their registers.
                constexpr bool HASRES = EPI == EPI_RES || RL;
                constexpr int RESAHEAD = TM < 2 ? TM : 2;
                u32x4 res[HASRES ? TM : 1][PER];
                issue_next();
                if constexpr (HASRES) static_for<RESAHEAD>([&](auto ia) { fetch_res(ia, res[decltype(ia)::value]); });
                stage_band(std::integral_constant<int, 0>{});
                static_for<TM>([&](auto ia) {
                    constexpr int a = decltype(ia)::value;
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    u32x4 val[PER];
                    f32x2_t rst[PER];
                    fetch_band(ia, val);
                    fetch_rstats(ia, rst);
                    if constexpr (a + 1 < TM) stage_band(std::integral_constant<int, a + 1>{});
                    if constexpr (HASRES && a == 0 && TM > RESAHEAD)
                        static_for<TM - RESAHEAD>([&](auto ib) { fetch_res(std::integral_constant<int, decltype(ib)::value + RESAHEAD>{}, res[decltype(ib)::value + RESAHEAD]); });
                    store_band(ia, val, res[HASRES ? a : 0], rst);
                });
            } else {
                issue_next();
                static_for<TM>([&](auto ia) {
                    stage_band(ia);
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    u32x4 val[PER];
                    f32x2_t rst[PER];
                    fetch_band(ia, val);
                    fetch_rstats(ia, rst);
                    if constexpr (EPI == EPI_RES || RL) {
                        // residual chunks in two halves: a whole band of them next to the staged values and
                        // the other band's accumulators does not fit the register file
                        constexpr int a = decltype(ia)::value;
                        constexpr int HP = PER >= 2 ? PER / 2 : PER;
#pragma unroll
                        for (int h = 0; h < PER / HP; ++h) {
                            u32x4 rr[HP];
                            bool in[HP];
#pragma unroll
                            for (int j = 0; j < HP; ++j) {
                                const int id = tid + (h * HP + j) * NT;
                                const int r = id / CPR, cc = id % CPR;
                                const int m = m0 + (r >> 5) * WM + a * 32 + (r & 31);
                                const int n = n0 + cc * EPCO;
                                in[j] = m < p.M && n < p.N;
                                rr[j] = u32x4{0u, 0u, 0u, 0u};
                                if (in[j]) rr[j] = __builtin_nontemporal_load((const u32x4*)((const OutT*)p.residual + (int64_t)m * p.N + n));
                            }
#pragma unroll
                            for (int j = 0; j < HP; ++j) emit(ia, h * HP + j, val[h * HP + j], rr[j], rst[h * HP + j]);
                        }
                    } else {
                        u32x4 res[PER];
                        store_band(ia, val, res, rst);
                    }
                    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
                });
            }
        } else if constexpr (!RL) {        // EPI_RESLN exists in the staged form only: the host launches it for nothing else
            issue_next();
            epilogue_direct<OutT, TM, TN, TNO, WM, WNO, EPI, DUAL, LN>(acc, p, m0, n0, wm, wn, li, lg);
        }
        if (!has_next) break;
        pid = npid; m0 = m0n; n0 = n0n; rsA = rsAn; rsW = rsWn; rsWp = rsWpn; bbuf ^= 1;
    }
}

// ---- any shape / any alignment: one thread per output, ascending-k fp32 sum (the summation
// order of shaders/fnn-linear.glsl:45-49).  Used only when rows are not 16-byte aligned.
template <typename T, typename OutT, int EPI, bool DUAL, bool LN = false>
__global__ __launch_bounds__(256) void gemm_nt_scalar_kernel(GemmArgs p) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)p.M * p.N) return;
    const int m = (int)(idx / p.N), n = (int)(idx % p.N);
    const T* a = (const T*)p.A + (int64_t)m * p.K;
    const T* w = (const T*)p.W + (int64_t)n * p.K;
    float s = 0.f;
    for (int k = 0; k < p.K; ++k) s += elem<T>::ld(a + k) * elem<T>::ld(w + k);
    float rs = 1.f, rsm = 0.f;
    if (LN) { rs = p.ln_stats[2 * (int64_t)m]; rsm = p.ln_stats[2 * (int64_t)m + 1]; s = s * rs - rsm * p.ln_c[n]; }
    if (p.bias) s += p.bias[n];
    if (DUAL) {
        const T* w2 = (const T*)p.W2 + (int64_t)n * p.K;
        float u = 0.f;
        for (int k = 0; k < p.K; ++k) u += elem<T>::ld(a + k) * elem<T>::ld(w2 + k);
        if (LN) u = u * rs - rsm * p.ln_c2[n];
        if (p.bias2) u += p.bias2[n];
        if (p.cache1) p.cache1[idx] = s;
        if (p.cache2) p.cache2[idx] = u;
        s = glu_apply(s, u, p);
    } else {
        s = epi_apply<EPI>(s, p);
        if constexpr (EPI == EPI_RES) s += elem<OutT>::ld((const OutT*)p.residual + idx);
    }
    elem<OutT>::st((OutT*)p.C + idx, s);
}

// ------------------------------------------------------------------ host dispatch
// 256 x 256 tiles (one persistent workgroup per CU) or 128 x 128 tiles (two per CU)?  Big tiles move half the operand
// bytes per FLOP, but a launch is as long as its fullest CU: n_big tiles take ceil(n_big / CUs) tile times, and e.g. 320
// tiles on 256 CUs leave the second pass three quarters empty.  Modelled in units of one 128 x 128 tile's work at full
// speed: a pass of big tiles costs 4; a full pass of small tiles (two share a CU) 2 x p, a last pass that leaves every
// CU at most one of them 1 x p, with p the small tile's handicap (measured: none in fp32, whose matrix rate is the
// bound; 1.17 in bf16, where the global -> LDS path is).  Small tiles are taken when the model gives them 7 % or more
// (measured at 2048 ... 32768 rows against 384 ... 4096 columns: 13 - 30 % faster where the model says so, within 4 %
// of the better choice everywhere); below 192 big tiles they are taken anyway.
static inline bool prefer_big_tiles(int64_t n_big, int64_t n_small, int64_t cus, size_t elem_size) {
    if (n_big < 192) return false;
    const double p = elem_size == 4 ? 1.0 : 1.17;
    const double t_big = 4.0 * (double)((n_big + cus - 1) / cus);
    const int64_t full = n_small / (2 * cus), rest = n_small % (2 * cus);
    const double t_small = p * (2.0 * (double)full + (rest == 0 ? 0.0 : (rest <= cus ? 1.0 : 2.0)));
    return !(t_small < 0.93 * t_big);
}

// Which kernel a 16-byte aligned problem gets: 1 register-staged 256 x 256 tiles, 2 register-staged 128 x 128, 3 direct-to-LDS
// 256 x 256 (persistent), 4 direct-to-LDS 128 x 128, 5 register-staged 64 x 64.  The direct-to-LDS kernels need K to be a
// whole number of 128-byte slabs.  Problems that 128 x 128 tiles would spread over a fraction of the CUs (single
// sentences, small batches, the README-sized operators) take 64 x 64 tiles: four times the workgroups, each with a quarter
// of the serial K loop, and no rows padded up to 128.  Measured at 32 ... 2048 rows against the BERT-base widths: in fp32,
// whose matrix rate is the bound, they win up to about four 64 x 64 tiles per CU (32 x 2304 x 768: 56 -> 24 us,
// 1024 x 768 x 3072: 203 -> 83 us), in bf16 up to one per CU (128 x 768 x 768: 12.8 -> 10.4 us, 1024 x 768 x 3072:
// 37.9 -> 31.9 us; beyond that the direct-to-LDS kernel is ahead).  `dual`: the gated kernels, whose 128-row tiles hold
// half as many output columns.
static inline int gemm_variant(int64_t M, int64_t N, int64_t K, size_t elem_size, bool dual, int64_t cus) {
    const int64_t bke = 128 / (int64_t)elem_size;
    const int64_t big_m = (M + 255) / 256, big_n = (N + (dual ? 127 : 255)) / (dual ? 128 : 256);
    const int64_t sm = (M + 127) / 128, sn = (N + (dual ? 63 : 127)) / (dual ? 64 : 128);
    const int64_t t64 = ((M + 63) / 64) * ((N + 63) / 64);
    if (t64 <= cus * (elem_size == 4 ? 4 : 1)) return 5;
    const bool slabs = K % bke == 0;
    const bool big = prefer_big_tiles(big_m * big_n, sm * sn, cus, elem_size);
    return slabs ? (big ? 3 : 4) : (big ? 1 : 2);
}

template <typename T, typename OutT, int EPI, bool DUAL, bool LN = false>
static int launch_gemm(grl_ctx* c, GemmArgs& a) {
    const int64_t epc = 16 / (int64_t)sizeof(T);
    const bool aligned = (a.K % epc == 0) && ((((uintptr_t)a.A) | ((uintptr_t)a.W) | ((uintptr_t)a.W2)) & 15u) == 0 &&
                         ((((uintptr_t)a.C) | ((uintptr_t)a.bias) | ((uintptr_t)a.bias2) | ((uintptr_t)a.cache1) | ((uintptr_t)a.cache2) | ((uintptr_t)a.residual) |
                           ((uintptr_t)a.ln_stats) | ((uintptr_t)a.ln_c) | ((uintptr_t)a.ln_c2)) & 15u) == 0;
    if (!aligned) {
        int64_t total = (int64_t)a.M * a.N;
        GRL_REQUIRE((total + 255) / 256 < (1LL << 31), GRL_ERR_SHAPE, "gemm: unaligned problem too large for the scalar kernel");
        hipLaunchKernelGGL((gemm_nt_scalar_kernel<T, OutT, EPI, DUAL, LN>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, c->stream, a);
        GRL_CHECK_LAUNCH();
        return GRL_OK;
    }
    // Tile choice: gemm_variant().  GRL_GEMM_VARIANT (1..5) forces one variant, for tuning runs.
    static const int forced = [] { const char* e = getenv("GRL_GEMM_VARIANT"); return e ? atoi(e) : 0; }();
    // band height of the tile walk: rows of 8 KiB and more do better with narrow bands (measured)
    static const int group = [] { const char* e = getenv("GRL_GEMM_GROUP"); return e ? atoi(e) : 0; }();
    a.group = group > 0 ? group : (a.K * (int64_t)sizeof(T) >= 8192 ? 2 : 8);
    const int64_t bke = 128 / (int64_t)sizeof(T);
    const int64_t big_m = (a.M + 255) / 256, big_n = (a.N + (DUAL ? 127 : 255)) / (DUAL ? 128 : 256);
    const int64_t sm = (a.M + 127) / 128, sn = (a.N + (DUAL ? 63 : 127)) / (DUAL ? 64 : 128);
    GRL_REQUIRE(sm * sn < (1LL << 31), GRL_ERR_SHAPE, "gemm: too many tiles");
    GRL_REQUIRE(a.K * (int64_t)sizeof(T) * 256 < (1LL << 31), GRL_ERR_SHAPE, "gemm: K too large (256 rows must span < 2 GiB)");
    const bool slabs = a.K % bke == 0;
    const int64_t cus = c->prop.multiProcessorCount;     // one 128 KiB-LDS workgroup per CU, two of the 64 KiB ones
    const int64_t tm = (a.M + 63) / 64, tn = (a.N + 63) / 64;      // 64 output columns per tile (with two weights: 128 LDS rows)
    int variant = gemm_variant(a.M, a.N, a.K, sizeof(T), DUAL, cus);
    if (forced >= 1 && forced <= 5 && (slabs || forced <= 2 || forced == 5)) variant = forced;
    switch (variant) {
        case 5: {
            a.tiles_m = (int)tm; a.tiles_n = (int)tn;
            // Few tiles and a long K (one sentence through a feed-forward block: 24 tiles, 96 slabs in fp32) leave most CUs
            // idle behind a serial K loop whose every slab costs a memory round trip: the slabs are shared out over up to
            // 8 workgroups per tile (16 slabs or more, at least 4 per share, at most about two workgroups per CU in all), which write raw
            // fp32 sums to a pool buffer, and a small second kernel adds them and runs the epilogue.  GRL_GEMM_SPLITK=0
            // switches it off, for tuning runs.
            static const int splitk_env = [] { const char* e = getenv("GRL_GEMM_SPLITK"); return e ? atoi(e) : -1; }();
            int ks = 1;
            if constexpr (!DUAL && !LN && (EPI == EPI_NONE || EPI == EPI_GELU || EPI == EPI_SILU || EPI == EPI_RT || EPI == EPI_RES)) {
                const int64_t KT = (a.K + bke - 1) / bke, t64 = tm * tn;
                if (splitk_env != 0 && !a.no_alloc && a.N % 4 == 0 && KT >= 16 && t64 <= cus) {
                    ks = (int)std::min<int64_t>(std::min<int64_t>(8, 2 * cus / t64), KT / 4);
                    while (ks > 1 && ((KT + ks - 1) / ks) * (ks - 1) >= KT) --ks;      // no empty share
                    if (ks == 2 && KT < 48) ks = 1;                                      // two short halves: the second launch costs more
                }
                if (ks > 1) {
                    a.ksplit = ks;
                    a.kpart = (float*)grl_malloc(c, (size_t)ks * a.M * a.N * sizeof(float));
                    if (!a.kpart) return GRL_ERR_OOM;
                    hipLaunchKernelGGL((gemm_nt_kernel<T, OutT, 64, 64, 2, 2, EPI, false, false, true>), dim3((unsigned)(tm * tn), (unsigned)ks), dim3(256), 0, c->stream, a);
                    const int64_t quads = (int64_t)a.M * a.N / 4;
                    hipLaunchKernelGGL((gemm_splitk_finish_kernel<OutT, EPI>), dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, c->stream, a);
                    grl_free(c, a.kpart);          // back to the pool: later users are ordered behind these launches on the stream
                    break;
                }
            }
            hipLaunchKernelGGL((gemm_nt_kernel<T, OutT, 64, (DUAL ? 128 : 64), 2, 2, EPI, DUAL, LN>), dim3((unsigned)(tm * tn)), dim3(256), 0, c->stream, a);
            break;
        }
        case 1:
            a.tiles_m = (int)big_m; a.tiles_n = (int)big_n;
            hipLaunchKernelGGL((gemm_nt_kernel<T, OutT, 256, 256, 2, 2, EPI, DUAL, LN>), dim3((unsigned)(big_m * big_n)), dim3(256), 0, c->stream, a);
            break;
        case 2:
            a.tiles_m = (int)sm; a.tiles_n = (int)sn;
            hipLaunchKernelGGL((gemm_nt_kernel<T, OutT, 128, 128, 2, 2, EPI, DUAL, LN>), dim3((unsigned)(sm * sn)), dim3(256), 0, c->stream, a);
            break;
        case 3:
            a.tiles_m = (int)big_m; a.tiles_n = (int)big_n;
            hipLaunchKernelGGL((gemm_nt_dma_kernel<T, OutT, 256, 256, 2, 4, EPI, DUAL, LN>), dim3((unsigned)std::min<int64_t>(big_m * big_n, cus)), dim3(512), 0, c->stream, a);
            break;
        default:
            a.tiles_m = (int)sm; a.tiles_n = (int)sn;
            hipLaunchKernelGGL((gemm_nt_dma_kernel<T, OutT, 128, 128, 2, 2, EPI, DUAL, LN>), dim3((unsigned)std::min<int64_t>(sm * sn, 2 * cus)), dim3(256), 0, c->stream, a);
            break;
    }
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// EPI_RESLN: only the direct-to-LDS kernels with their LDS-staged epilogue implement it, so the problem must be one
// they take (whole 128-byte K slabs, 16-byte aligned operands, output rows a multiple of 16 bytes).  *tile_cols
// returns the column width of the tiles, i.e. of the row-statistics partials the kernel writes.
template <typename T, typename OutT>
int launch_gemm_resln(grl_ctx* c, GemmArgs& a, int* tile_cols) {
    const int64_t bke = 128 / (int64_t)sizeof(T);
    const bool aligned = ((((uintptr_t)a.A) | ((uintptr_t)a.W) | ((uintptr_t)a.C) | ((uintptr_t)a.bias) | ((uintptr_t)a.residual) |
                           ((uintptr_t)a.res_stats) | ((uintptr_t)a.res_gamma) | ((uintptr_t)a.res_beta) | ((uintptr_t)a.part_out)) & 15u) == 0;
    GRL_REQUIRE(aligned && a.K % bke == 0 && ((int64_t)a.N * (int64_t)sizeof(OutT)) % 16 == 0, GRL_ERR_SHAPE,
                "gemm (LayerNorm residual): needs 16-byte aligned operands, K a multiple of %lld and output rows a multiple of 16 bytes",
                (long long)bke);
    GRL_REQUIRE(a.K * (int64_t)sizeof(T) * 256 < (1LL << 31), GRL_ERR_SHAPE, "gemm: K too large (256 rows must span < 2 GiB)");
    static const int group = [] { const char* e = getenv("GRL_GEMM_GROUP"); return e ? atoi(e) : 0; }();
    a.group = group > 0 ? group : (a.K * (int64_t)sizeof(T) >= 8192 ? 2 : 8);
    const int64_t big_m = (a.M + 255) / 256, big_n = (a.N + 255) / 256;
    const int64_t sm = (a.M + 127) / 128, sn = (a.N + 127) / 128;
    GRL_REQUIRE(sm * sn < (1LL << 31), GRL_ERR_SHAPE, "gemm: too many tiles");
    const int64_t cus = c->prop.multiProcessorCount;
    if (prefer_big_tiles(big_m * big_n, sm * sn, cus, sizeof(T))) {
        a.tiles_m = (int)big_m; a.tiles_n = (int)big_n; *tile_cols = 256;
        hipLaunchKernelGGL((gemm_nt_dma_kernel<T, OutT, 256, 256, 2, 4, EPI_RESLN, false, false>), dim3((unsigned)std::min<int64_t>(big_m * big_n, cus)), dim3(512), 0, c->stream, a);
    } else {
        a.tiles_m = (int)sm; a.tiles_n = (int)sn; *tile_cols = 128;
        hipLaunchKernelGGL((gemm_nt_dma_kernel<T, OutT, 128, 128, 2, 2, EPI_RESLN, false, false>), dim3((unsigned)std::min<int64_t>(sm * sn, 2 * cus)), dim3(256), 0, c->stream, a);
    }
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

template <typename T, typename OutT>
int dispatch_epi(grl_ctx* c, GemmArgs& a, int epi) {
    switch (epi) {
        case EPI_NONE: return launch_gemm<T, OutT, EPI_NONE, false>(c, a);
        case EPI_GELU: return launch_gemm<T, OutT, EPI_GELU, false>(c, a);
        case EPI_SILU: return launch_gemm<T, OutT, EPI_SILU, false>(c, a);
        case EPI_RT: return launch_gemm<T, OutT, EPI_RT, false>(c, a);
        case EPI_GLU: return launch_gemm<T, OutT, EPI_GLU, true>(c, a);
        case EPI_RES: return launch_gemm<T, OutT, EPI_RES, false>(c, a);
    }
    grl_set_error("gemm: bad epilogue %d", epi);
    return GRL_ERR_ARG;
}

// the LayerNorm-folded forms: plain (bias only) and the gated dual-weight epilogue
template <typename T, typename OutT>
int dispatch_epi_ln(grl_ctx* c, GemmArgs& a, int epi) {
    switch (epi) {
        case EPI_NONE: return launch_gemm<T, OutT, EPI_NONE, false, true>(c, a);
        case EPI_GELU: return launch_gemm<T, OutT, EPI_GELU, false, true>(c, a);
        case EPI_GLU: return launch_gemm<T, OutT, EPI_GLU, true, true>(c, a);
    }
    grl_set_error("gemm: epilogue %d has no LayerNorm-folded form", epi);
    return GRL_ERR_ARG;
}

