// Flash-Attention-2 forward for gfx950, layout (B,S,H,D), optional key-padding mask,
// causal exclusion and fused interleaved RoPE.
//
// A workgroup (4 waves) owns 128 queries of one (batch, head); each wave owns 32 of them and
// keeps, per lane, ONE query: the kernel computes the transposed products
//     S^T = K . Q^T   (keys x queries)      and      O^T = V^T . P^T   (head-dim x queries)
// on 32x32 MFMA tiles, so every accumulator register of a lane belongs to that lane's query.
// The online-softmax state (running max m, running sum l) and the rescale factor are then
// per-lane scalars; the only cross-lane step is one exchange with lane^32 for the row max.
//
// fp32 kernel (fa2_fwd_kernel, register-staged tiles):
//   HBM --128-bit loads--> VGPR --(RoPE on K) --> LDS: K tile [key][d], XOR-swizzled chunks
//                                              --> LDS: V tile [key][d]
//   K/V tiles are double buffered; the next tile's loads are in flight during the MFMAs.
//   S, P and O never leave registers.  The bf16 kernel further down moves its tiles HBM -> LDS directly.
//
// Semantics (constants of shaders/flash-attention2.glsl:95,152,214):
//   score = <q,k>*scale + (mask[b,k]-1)*1e9 ; running max starts at -1e10 ;
//   out = acc / max(sum, 1e-10) ; causal keys (k > q) and keys >= S are excluded outright.
#include "common.hpp"
#include <type_traits>
#include <algorithm>
#include <cstdlib>

int grl_rope_apply_table(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                         void* y, const float* table);
int grl_rope_half_apply_table(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                              void* y, const float* table);
int grl_rope_strided(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, const void* x, int64_t x_stride,
                     const int32_t* position_ids, void* y, int style, float rope_base, float rope_scaling);

struct FaArgs {
    const void* Q; const void* K; const void* V;
    const float* mask;        // (B,S) or null
    void* O;
    const float2* rope;       // (S, D/2) {cos, sin} or null
    int B, S, H;
    float scale;
    int causal;
    int64_t q_stride, k_stride, v_stride, o_stride;   // elements between consecutive positions
};

template <int N, typename F> __device__ __forceinline__ void sfor(F&& f) {
    if constexpr (N > 0) {
        sfor<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

template <typename T> struct Slab;
template <> struct Slab<uint16_t> {
    static __device__ __forceinline__ void run(const u32x4& a, const u32x4& b, f32x16& acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
    }
};
template <> struct Slab<float> {
    static __device__ __forceinline__ void run(const u32x4& a, const u32x4& b, f32x16& acc) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(u2f(a[e]), u2f(b[e]), acc, 0, 0, 0);
    }
};

// rotate the pairs held in one 16-byte chunk; cs[i] = {cos, sin} of pair i
template <typename T> __device__ __forceinline__ u32x4 rope_chunk(u32x4 v, const float2* cs);
template <> __device__ __forceinline__ u32x4 rope_chunk<float>(u32x4 v, const float2* cs) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        float x0 = u2f(v[2 * i]), x1 = u2f(v[2 * i + 1]);
        o[2 * i] = __builtin_bit_cast(uint32_t, x0 * cs[i].x - x1 * cs[i].y);
        o[2 * i + 1] = __builtin_bit_cast(uint32_t, x0 * cs[i].y + x1 * cs[i].x);
    }
    return o;
}
template <> __device__ __forceinline__ u32x4 rope_chunk<uint16_t>(u32x4 v, const float2* cs) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float x0 = bf16lo(v[i]), x1 = bf16hi(v[i]);
        o[i] = pack_bf16x2(x0 * cs[i].x - x1 * cs[i].y, x0 * cs[i].y + x1 * cs[i].x);
    }
    return o;
}
// 8 bf16 values times a scalar, optionally rotated first (one rounding at the end)
template <bool ROT> __device__ __forceinline__ u32x4 scale_chunk_bf16(u32x4 v, const float2* cs, float scale) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float x0 = bf16lo(v[i]), x1 = bf16hi(v[i]);
        if (ROT) {
            const float r0 = x0 * cs[i].x - x1 * cs[i].y, r1 = x0 * cs[i].y + x1 * cs[i].x;
            x0 = r0; x1 = r1;
        }
        o[i] = pack_bf16x2(x0 * scale, x1 * scale);
    }
    return o;
}

template <typename OutT> __device__ __forceinline__ void fa_store4(OutT* p, float a, float b, float c, float d);
template <> __device__ __forceinline__ void fa_store4<float>(float* p, float a, float b, float c, float d) {
    f32x4 v = {a, b, c, d};
    *(f32x4*)p = v;
}
template <> __device__ __forceinline__ void fa_store4<uint16_t>(uint16_t* p, float a, float b, float c, float d) {
    u32x2 v = {pack_bf16x2(a, b), pack_bf16x2(c, d)};
    *(u32x2*)p = v;
}

template <typename T, int D, bool ROPE>
__global__ __launch_bounds__(256) void fa2_fwd_kernel(FaArgs p) {
    static_assert(sizeof(T) == 4, "the register-staged kernel is the fp32 path");
    constexpr int ES = (int)sizeof(T), RB = D * ES, NCH = RB / 16, NS = RB / 32, EPC = 16 / ES;
    constexpr int KT = 64;                              // keys per tile
    constexpr int NKB = KT / 32, DT = D / 32;
    constexpr int CK = KT * NCH / 256;                  // K chunks per thread
    constexpr int CV = CK;
    constexpr int TILE = KT * RB;
    constexpr int PPC = EPC / 2;                        // RoPE pairs per chunk
    static_assert(KT * NCH % 256 == 0, "tile does not divide over 256 threads");
    __shared__ __attribute__((aligned(16))) char ldsK[2][TILE];
    __shared__ __attribute__((aligned(16))) char ldsV[2][TILE];
    __shared__ __attribute__((aligned(16))) float ldsBias[2][KT];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 31, lg = lane >> 5;
    const int b = blockIdx.z, h = blockIdx.y;
    const int qb = p.causal ? (int)gridDim.x - 1 - (int)blockIdx.x : (int)blockIdx.x;   // heavy blocks first
    const int q0 = qb * 128;
    const int S = p.S;
    const int qi = q0 + wave * 32 + li;
    const int qc = qi < S ? qi : S - 1;
    const T* Qg = (const T*)p.Q + (int64_t)b * S * p.q_stride + h * D;
    const T* Kg = (const T*)p.K + (int64_t)b * S * p.k_stride + h * D;
    const T* Vg = (const T*)p.V + (int64_t)b * S * p.v_stride + h * D;

    // ---- this lane's query, as MFMA "B" operand: slab s holds dims (2s+lg)*EPC .. +EPC-1
    u32x4 qf[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const int c = 2 * s + lg;
        u32x4 v = *(const u32x4*)(Qg + (int64_t)qc * p.q_stride + c * EPC);
        if (ROPE) {
            float2 cs[PPC];
#pragma unroll
            for (int i = 0; i < PPC; ++i) cs[i] = p.rope[(int64_t)qc * (D / 2) + c * PPC + i];
            v = rope_chunk<T>(v, cs);
        }
        qf[s] = v;
    }

    int nkt = (S + KT - 1) / KT;
    if (p.causal) {
        int last = (q0 + 127 < S - 1 ? q0 + 127 : S - 1) / KT + 1;
        nkt = nkt < last ? nkt : last;
    }

    // ---- staging registers and their loaders
    u32x4 kreg[CK], vreg[CV];
    float2 kcs[ROPE ? CK : 1][PPC];
    float breg = 0.f;
    auto load_tile = [&](int kt) {
        const int k0 = kt * KT;
#pragma unroll
        for (int i = 0; i < CK; ++i) {
            const int q = tid + i * 256, key = q / NCH, c = q % NCH;
            const int kk = k0 + key, kc = kk < S ? kk : S - 1;
            kreg[i] = *(const u32x4*)(Kg + (int64_t)kc * p.k_stride + c * EPC);
            if (ROPE) {
#pragma unroll
                for (int j = 0; j < PPC; ++j) kcs[i][j] = p.rope[(int64_t)kc * (D / 2) + c * PPC + j];
            }
        }
#pragma unroll
        for (int i = 0; i < CV; ++i) {
            const int q = tid + i * 256, key = q / NCH, c = q % NCH;
            const int kk = k0 + key, kc = kk < S ? kk : S - 1;
            vreg[i] = *(const u32x4*)(Vg + (int64_t)kc * p.v_stride + c * EPC);
        }
        if (tid < KT) {
            const int kk = k0 + tid;
            breg = 0.f;
            if (p.mask && kk < S) breg = (p.mask[(int64_t)b * S + kk] - 1.0f) * 1e9f;
            if (kk >= S) breg = -__builtin_inff();
        }
    };
    auto stash_tile = [&](int kt) {
        const int st = kt & 1, k0 = kt * KT;
        const u32x4 zero = {0u, 0u, 0u, 0u};
        char* Kb = ldsK[st];
        char* Vb = ldsV[st];
#pragma unroll
        for (int i = 0; i < CK; ++i) {
            const int q = tid + i * 256, key = q / NCH, c = q % NCH;
            u32x4 v = kreg[i];
            if (ROPE) v = rope_chunk<T>(v, kcs[i]);
            if (k0 + key >= S) v = zero;
            const int slot = c ^ lds_swz<NCH>(key);
            *(u32x4*)(Kb + key * RB + slot * 16) = v;
        }
#pragma unroll
        for (int i = 0; i < CV; ++i) {
            const int q = tid + i * 256, key = q / NCH, c = q % NCH;
            *(u32x4*)(Vb + key * RB + c * 16) = (k0 + key >= S) ? zero : vreg[i];
        }
        if (tid < KT) ldsBias[st][tid] = breg;
    };

    f32x16 oacc[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[t][r] = 0.f;
    float m_run = -1e10f, l_run = 0.f;

    load_tile(0);
    stash_tile(0);
    __syncthreads();
    for (int kt = 0; kt < nkt; ++kt) {
        const bool more = kt + 1 < nkt;
        if (more) load_tile(kt + 1);
        const int st = kt & 1, k0 = kt * KT;
        const char* Kb = ldsK[st];
        const char* Vb = ldsV[st];

        // ---- S^T = K . Q^T for the tile's NKB blocks of 32 keys
        f32x16 sacc[NKB];
        sfor<NKB>([&](auto it) {
            constexpr int t = decltype(it)::value;
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[t][r] = 0.f;
            const int key = 32 * t + li;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const int c = 2 * s + lg;
                const int slot = c ^ lds_swz<NCH>(key);
                u32x4 kf = *(const u32x4*)(Kb + key * RB + slot * 16);
                Slab<T>::run(kf, qf[s], sacc[t]);
            }
        });

        // ---- scores, running max
        const bool diag = p.causal && (k0 + KT - 1 > q0 + wave * 32);
        float mx = -__builtin_inff();
        sfor<NKB>([&](auto it) {
            constexpr int t = decltype(it)::value;
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int kl = 32 * t + 8 * qd + 4 * lg;          // first of 4 consecutive keys
                f32x4 bias = *(const f32x4*)(&ldsBias[st][kl]);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float s = sacc[t][4 * qd + e] * p.scale + bias[e];
                    if (diag && (k0 + kl + e > qi)) s = -__builtin_inff();
                    sacc[t][4 * qd + e] = s;
                    mx = fmaxf(mx, s);
                }
            }
        });
        mx = halves_max(mx);
        const float m_new = fmaxf(m_run, mx);
        const float alpha = __expf(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
        sfor<NKB>([&](auto it) {
            constexpr int t = decltype(it)::value;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float pv = __expf(sacc[t][r] - m_new);
                sacc[t][r] = pv;
                psum += pv;
            }
        });
        l_run = l_run * alpha + psum;
        sfor<DT>([&](auto idt) {
            constexpr int dt = decltype(idt)::value;
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[dt][r] *= alpha;
        });

        // ---- O^T += V^T . P^T
        sfor<NKB>([&](auto it) {
            constexpr int t = decltype(it)::value;
            sfor<16>([&](auto ir) {
                constexpr int r = decltype(ir)::value;
                const int kl = 32 * t + 8 * (r / 4) + 4 * lg + (r % 4);
                sfor<DT>([&](auto idt) {
                    constexpr int dt = decltype(idt)::value;
                    float vv = *(const float*)(Vb + kl * RB + (32 * dt + li) * 4);
                    oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv, sacc[t][r], oacc[dt], 0, 0, 0);
                });
            });
        });

        if (more) stash_tile(kt + 1);
        __syncthreads();
    }

    // ---- normalise and store: lane holds, for its query, dims 32dt + 8qd + 4lg + {0..3}
    const float l_tot = halves_sum(l_run);
    const float inv = 1.0f / fmaxf(l_tot, 1e-10f);
    if (qi < S) {
        T* Og = (T*)p.O + ((int64_t)b * S + qi) * p.o_stride + h * D;
        sfor<DT>([&](auto idt) {
            constexpr int dt = decltype(idt)::value;
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int d = 32 * dt + 8 * qd + 4 * lg;
                fa_store4<T>(Og + d, oacc[dt][4 * qd] * inv, oacc[dt][4 * qd + 1] * inv, oacc[dt][4 * qd + 2] * inv, oacc[dt][4 * qd + 3] * inv);
            }
        });
    }
}

// =====================================================================================
// bf16 kernel.
//
//   K and V tiles (64 or 128 keys) go HBM -> LDS by buffer_load ... lds (no staging registers), both
//   row-major [key][d] with the 16-byte chunks XOR-swizzled by key, in a ring of 2-8 stages.
//   S^T = K.Q^T reads K with ds_read_b128; O^T += V^T.P^T reads V with the transposing
//   ds_read_b64_tr_b16: inside a 16-lane group, source lane j points at
//   V[k0 + j/4][d0 + 4*(j%4) ..] and result lane i receives V[k0 .. k0+3][d0 + i], i.e. four
//   consecutive keys of ONE head dimension -- the MFMA operand -- without any shuffling.
//   Softmax works in the base-2 domain, p = exp2(s*scale*log2e - m), one v_exp_f32 per score, and the
//   subtraction of m is done by the matrix core (one more k-slab, see the kernel).
//   The kernel is bound by instruction issue, not by any one pipeline (SQ counters: a SIMD issues one
//   instruction of any kind per four cycles, and the sum of its waves' active cycles fills the kernel
//   time), so the tile loop is kept to the instructions the algorithm needs: per 32 queries x 64 keys
//   at head dim 64, 17 MFMA + 32 v_exp + 16 v_cvt_pk + 16 v_dot2c + 17 v_max3 + 24 LDS reads, about
//   45 scalar and 10 wait instructions.  What that takes: wave-uniform values are declared so
//   (readfirstlane), transfers are addressed through scalar registers, the common tile has a loop of its
//   own that nothing else joins, and the PV accumulates are tied in place.
//   RoPE: each Q row is rotated once as it is loaded; K is rotated once per row by the host
//   wrapper into a workspace (rotating K inside the kernel would redo it for every query block).
// =====================================================================================
struct Fa16Args {
    const uint16_t* Q; const uint16_t* K; const uint16_t* V;
    const float* mask; uint16_t* O; const float2* rope;
    int B, S, H;
    float scale;
    int causal;
    int order;            // workgroup -> (head, query block) map, see fa2_bf16_kernel
    int64_t q_stride, k_stride, v_stride, o_stride;
};

typedef __attribute__((ext_vector_type(4))) short s16x4_t;

// s_waitcnt with vmcnt = N and the other counters left open (gfx9 encoding)
template <int N> __device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}
template <int IPT, int MAXT> __device__ __forceinline__ void wait_tiles_outstanding(int tiles) {
    // allow `tiles` later tiles (IPT transfers each) to be still in flight; loads return in order
    if constexpr (MAXT >= 0) {
        if (tiles >= MAXT) wait_vmcnt<IPT * MAXT>();
        else wait_tiles_outstanding<IPT, MAXT - 1>(tiles);
    }
}

template <int N> __device__ __forceinline__ void wait_lgkmcnt() {
    __builtin_amdgcn_s_waitcnt(15 | (3 << 14) | (7 << 4) | ((N & 15) << 8));
}
// a wave-uniform value, said so to the compiler (it then lives in a scalar register and branches on it are scalar)
__device__ __forceinline__ int uni(int v) { return __builtin_amdgcn_readfirstlane(v); }

// The PV accumulates of one 16-key slab as in-place instructions the register allocator cannot untie (with the builtin
// it moves the 32-register accumulator to another place and back around every tile).  The compiler does not know that
// these are matrix instructions and adds no hazard wait states for them:
//   * the s_nop in front keeps two wait states between whatever VALU instruction last wrote an operand register (the
//     accumulators' zero fill, which the compiler sinks to their first use; a conversion; a register move or reload the
//     compiler puts in front of the statement) and the MFMA that reads it;
//   * mfma_drain() before any VALU / memory instruction reads or writes the accumulators.
template <int DT> __device__ __forceinline__ void mfma_inplace(const u32x4 (&a)[DT], const u32x4& b, f32x16 (&acc)[DT]) {
    static_assert(DT == 1 || DT == 2 || DT == 4, "head dims 32, 64, 128");
    if constexpr (DT == 1)
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[0]) : "v"(a[0]), "v"(b));
    else if constexpr (DT == 2)
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %2, %4, %0\n\tv_mfma_f32_32x32x16_bf16 %1, %3, %4, %1"
                     : "+v"(acc[0]), "+v"(acc[1]) : "v"(a[0]), "v"(a[1]), "v"(b));
    else
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %4, %8, %0\n\tv_mfma_f32_32x32x16_bf16 %1, %5, %8, %1\n\t"
                     "v_mfma_f32_32x32x16_bf16 %2, %6, %8, %2\n\tv_mfma_f32_32x32x16_bf16 %3, %7, %8, %3"
                     : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]) : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(b));
}
__device__ __forceinline__ void mfma_drain() { asm volatile("s_nop 15\n\ts_nop 3" ::: "memory"); }

// ROPE_Q: rotation applied to the query rows as they are loaded: 0 none, 1 interleaved pairs (2p, 2p+1), 2 the
// (d, d+D/2) pairing (both halves of a pair sit in chunks this lane loads itself)
// QT = 32-query MFMA tiles per wave, NW waves per workgroup, NSTG-deep ring of KT-key (64 or 128) K/V tiles in LDS
// (NSTG-1 tiles in flight), OCC workgroups per CU the registers are budgeted for.
template <int D, int ROPE_Q, int QT, int NW, int NSTG, bool HAS_MASK, int KT, int OCC = (NW == 4 ? 2 : 1)>
__global__ __launch_bounds__(NW * 64, OCC) void fa2_bf16_kernel(Fa16Args p) {
    constexpr int RB = D * 2, NCH = RB / 16, NS = D / 16;
    constexpr int NKB = KT / 32, DT = D / 32;
    constexpr int TILE = KT * RB;
    constexpr int NT = NW * 64;
    constexpr int TPO = TILE / 1024;
    constexpr int IPT = 2 * TPO / NW + (HAS_MASK ? 1 : 0);
    constexpr int RPI = 1024 / RB;
    constexpr int QW = 32 * QT, QB = NW * QW;
    static_assert((2 * TPO) % NW == 0 && 2 * TPO >= NW, "transfers must divide over the waves");
    static_assert(NSTG >= 2 && IPT * (NSTG - 1) < 64, "ring of at least two stages; vmcnt is a 6-bit counter");
    constexpr int OFF_V = NSTG * TILE, OFF_M = 2 * NSTG * TILE;
    __shared__ __attribute__((aligned(1024))) char lds[2 * NSTG * TILE + (HAS_MASK ? NSTG * 1024 : 0)];

    // Everything that steers control flow or addresses a transfer is wave-uniform and is told so to the compiler
    // (readfirstlane): the loop then branches on scalar conditions and keeps its counters in scalar registers.
    const int tid = threadIdx.x, lane = tid & 63, wave = uni(tid >> 6);
    const int li = lane & 31, lg = lane >> 5;
    const int S = p.S;
    const int nqb = (S + QB - 1) / QB, nbh = p.B * p.H;
    const int nwg = (int)gridDim.x, per = nwg >> 3, rem = nwg & 7, xcd = (int)blockIdx.x & 7, loc = (int)blockIdx.x >> 3;
    const int lin = (p.order & 1) ? xcd * per + (xcd < rem ? xcd : rem) + loc : (int)blockIdx.x;
    int qb, bh;
    if (p.order & 2) { qb = nqb - 1 - lin / nbh; bh = lin % nbh; }
    else if (p.causal) { bh = lin / nqb; qb = nqb - 1 - lin % nqb; }
    else { qb = lin % nqb; bh = lin / nqb; }
    qb = uni(qb); bh = uni(bh);
    const int b = uni(bh / p.H), h = uni(bh % p.H);
    const int q0 = qb * QB;
    const int qw0 = q0 + wave * QW;
    const uint16_t* Qg = p.Q + (int64_t)b * S * p.q_stride + h * D;

    int nkt = (S + KT - 1) / KT;
    if (p.causal) {
        int last = (q0 + QB - 1 < S - 1 ? q0 + QB - 1 : S - 1) / KT + 1;
        nkt = nkt < last ? nkt : last;
    }
    nkt = uni(nkt);

    auto make_rsrc = [&](const uint16_t* base, int64_t stride) __attribute__((always_inline)) {
        int64_t bytes = (int64_t)(S - 1) * stride * 2 + RB;
        uint32_t nrec = bytes > 0xffffffffLL ? 0xffffffffu : (uint32_t)bytes;
        return make_rsrc_words(base + (int64_t)b * S * stride + h * D, nrec);
    };
    // A wave's share of a tile's transfers is all K or all V (K transfers first, then V): which one is a
    // wave-uniform choice made once, so the loop issues its transfers without a branch.
    constexpr int TPW = 2 * TPO / NW;
    constexpr int KVAR = NCH >= 16 ? 4 : (NCH == 8 ? 2 : 1);
    static_assert(TPO % TPW == 0, "a wave's share does not straddle K and V");
    static_assert(TPW % KVAR == 0 && TPO % KVAR == 0 && (RPI * KVAR) % 16 == 0, "swizzle period must divide the transfer split");
    const bool isv = wave * TPW >= TPO;
    const rsrc_words rsT = isv ? make_rsrc(p.V, p.v_stride) : make_rsrc(p.K, p.k_stride);
    const rsrc_words rsM = make_rsrc_words(p.mask ? (const void*)(p.mask + (int64_t)b * S) : (const void*)p.Q, HAS_MASK ? (uint32_t)S * 4u : 0u);
    const int stride_b = uni((int)(isv ? p.v_stride : p.k_stride) * 2);
    const int inst0 = wave * TPW - (isv ? TPO : 0);
    const int t_row = lane / NCH, t_slot = lane % NCH;
    // per-lane part of a transfer address: row inside the transfer x row stride + swizzled chunk (K: KVAR variants,
    // the swizzle looks at row bits the transfer index supplies; V: one)
    int voffT[KVAR];
#pragma unroll
    for (int i = 0; i < KVAR; ++i)
        voffT[i] = t_row * stride_b + ((t_slot ^ (isv ? lds_swz_v<NCH>(t_row) : lds_swz<NCH>(i * RPI + t_row))) << 4);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
    const uint32_t lds_t = lds0 + (isv ? OFF_V : 0) + inst0 * 1024;
    const int soff_w = inst0 * RPI * stride_b, soff_step = RPI * stride_b, soff_tile = KT * stride_b;
    auto issue = [&](int kt, int ST) __attribute__((always_inline)) {
        const int so = kt * soff_tile + soff_w;
#pragma unroll
        for (int j = 0; j < TPW; ++j)
            asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         ::"s"(lds_t + ST * TILE + j * 1024), "v"(voffT[j % KVAR]), "s"(rsT), "s"(so + j * soff_step) : "memory");
        if constexpr (HAS_MASK)
            asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         ::"s"(lds0 + OFF_M + ST * 1024), "v"(lane * 16), "s"(rsM), "s"(kt * KT * 4) : "memory");
    };
    // the stage a runtime tile index lives in (prologue only; the loop knows its stage at compile time)
    auto issue_rt = [&](int kt) __attribute__((always_inline)) { issue(kt, kt % NSTG); };

    f32x16 oacc[QT][DT];
    float lsum[QT], m_run[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        m_run[t] = -1.4426950408889634e10f;
        lsum[t] = 0.f;
#pragma unroll
        for (int d = 0; d < DT; ++d)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[t][d][r] = 0.f;
    }
    const float c2 = p.scale * 1.4426950408889634f;

    issue(0, 0);

    u32x4 qf[QT][NS];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
        const int qi = qw0 + 32 * t + li;
        const int qc = qi < S ? qi : S - 1;
        if constexpr (ROPE_Q == 2) {
            // chunk c = 2s+lg holds dims 8c .. 8c+7; its partner for the (d, d+D/2) pairing is chunk c + NCH/2,
            // i.e. slab s + NS/2 of this same lane.  Table row qc holds {cos, sin} of pair d at [d], d < D/2.
            static_assert(NS % 2 == 0, "the two halves of the head dim split the slabs evenly");
#pragma unroll
            for (int s = 0; s < NS / 2; ++s) {
                const int c = 2 * s + lg;
                const u32x4 lo = *(const u32x4*)(Qg + (int64_t)qc * p.q_stride + c * 8);
                const u32x4 hi = *(const u32x4*)(Qg + (int64_t)qc * p.q_stride + (c + NCH / 2) * 8);
                const float2* cs = p.rope + (int64_t)qc * (D / 2) + c * 8;
                u32x4 olo, ohi;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float2 c0 = cs[2 * i], c1 = cs[2 * i + 1];
                    const float a0 = bf16lo(lo[i]), a1 = bf16hi(lo[i]), b0 = bf16lo(hi[i]), b1 = bf16hi(hi[i]);
                    olo[i] = pack_bf16x2((a0 * c0.x - b0 * c0.y) * c2, (a1 * c1.x - b1 * c1.y) * c2);
                    ohi[i] = pack_bf16x2((b0 * c0.x + a0 * c0.y) * c2, (b1 * c1.x + a1 * c1.y) * c2);
                }
                qf[t][s] = olo;
                qf[t][s + NS / 2] = ohi;
            }
        } else {
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int c = 2 * s + lg;
            u32x4 v = *(const u32x4*)(Qg + (int64_t)qc * p.q_stride + c * 8);
            // queries carry scale*log2(e): the matrix core then delivers scores in the base-2 softmax domain
            float2 cs[4];
            if (ROPE_Q == 1) {
#pragma unroll
                for (int i = 0; i < 4; ++i) cs[i] = p.rope[(int64_t)qc * (D / 2) + c * 4 + i];
            }
            qf[t][s] = scale_chunk_bf16<ROPE_Q == 1>(v, cs, c2);
        }
        }
    }


    f32x16 sacc[QT][NKB];
    constexpr float LAZY = 6.0f;
    const u32x4 kone = {lg == 0 ? 0x3f803f80u : 0u, lg == 0 ? 0x3f80u : 0u, 0u, 0u};   // key side of the reference slab: 1 at k-indices 0, 1, 2
    u32x4 mq[QT];                                                 // query side: -m_run in three parts there
#pragma unroll
    for (int u = 0; u < QT; ++u) mq[u] = u32x4{0u, 0u, 0u, 0u};

    // ---- fragment addresses.  K: row li of a 32-key block, chunk 2s+lg, swizzled by the row (the swizzle has period 16,
    // so block and stage offsets are immediates).  V (transposing read): see phase_PV.
    typedef __attribute__((address_space(3))) char lds_char;
    const lds_char* const ldsp = (const lds_char*)lds;
    const lds_char* kbase[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) kbase[s] = ldsp + li * RB + (((2 * s + lg) ^ lds_swz<NCH>(li)) << 4);
    const int j16 = lane & 15, grp = lane >> 4;
    const lds_char* vbase[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int key = 4 * (grp >> 1) + (j16 >> 2);                    // + 32t + 16hh (+ 8): multiples of 8 leave the swizzle alone
        const int dcol = 32 * dt + 16 * (grp & 1) + 4 * (j16 & 3);
        const int ch = dcol >> 3, sub = (dcol & 7) * 2;
        vbase[dt] = ldsp + OFF_V + key * RB + ((ch ^ lds_swz_v<NCH>(key)) << 4) + sub;
    }

    // ---- score phase: S^T = K . Q'^T for the tile in stage ST; accumulators start from C0 (zero, or -m_run for a lazy tile)
    constexpr int KB = 1;                                    // fragment buffers (2 = next group's reads in flight during a group's MFMAs: measured, no gain)
    constexpr int KG = NS < 4 ? NS : 4;                      // fragments per read group
    constexpr int NFR = NKB * NS, NG = NFR / KG;
    static_assert(NFR % KG == 0 && NS % KG == 0, "read groups stay inside a key block");
    auto phase_S = [&](int ST, auto ilazy) __attribute__((always_inline)) {
        constexpr bool LZ = decltype(ilazy)::value;
        const lds_char* kb[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) kb[s] = kbase[s] + ST * TILE;
        u32x4 kf[KB][KG];
        auto kread = [&](auto ig) __attribute__((always_inline)) {
            constexpr int G = decltype(ig)::value;
            sfor<KG>([&](auto ii) __attribute__((always_inline)) {
                constexpr int i = decltype(ii)::value, f = G * KG + i, t = f / NS, s = f % NS;
                kf[G % KB][i] = *(const __attribute__((address_space(3))) u32x4*)(kb[s] + t * 32 * RB);
            });
        };
        if constexpr (KB == 2) kread(std::integral_constant<int, 0>{});
        if constexpr (LZ) {
            // scores relative to m_run: one more k-slab whose key side is 1 and whose query side is -m_run puts -m_run
            // into every accumulator while the first fragments are on their way
            sfor<NKB>([&](auto it) __attribute__((always_inline)) {
                sfor<QT>([&](auto iu) __attribute__((always_inline)) {
                    constexpr int t = decltype(it)::value, u = decltype(iu)::value;
#pragma unroll
                    for (int r = 0; r < 16; ++r) sacc[u][t][r] = 0.f;
                    Slab<uint16_t>::run(kone, mq[u], sacc[u][t]);
                });
            });
        }
        sfor<NG>([&](auto ig) __attribute__((always_inline)) {
            constexpr int G = decltype(ig)::value;
            if constexpr (KB == 1) kread(ig);
            else if constexpr (G + 1 < NG) kread(std::integral_constant<int, G + 1>{});
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (KB == 2 && G + 1 < NG) wait_lgkmcnt<KG>(); else wait_lgkmcnt<0>();
            sfor<KG>([&](auto ii) __attribute__((always_inline)) {
                constexpr int i = decltype(ii)::value, f = G * KG + i, t = f / NS, s = f % NS;
                sfor<QT>([&](auto iu) __attribute__((always_inline)) {
                    constexpr int u = decltype(iu)::value;
                    if constexpr (s == 0 && !LZ) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) sacc[u][t][r] = 0.f;
                    }
                    Slab<uint16_t>::run(kf[G % KB][i], qf[u][s], sacc[u][t]);
                });
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // maximum over this lane's scores of the tile, then over the two halves of the wave (one query = lanes l and l+32)
    auto tile_max = [&](auto iu) __attribute__((always_inline)) {
        constexpr int u = decltype(iu)::value;
        float m0 = -__builtin_inff(), m1 = -__builtin_inff();
#pragma unroll
        for (int t = 0; t < NKB; ++t)
#pragma unroll
            for (int r = 0; r < 16; r += 4) {
                m0 = __builtin_fmaxf(__builtin_fmaxf(m0, sacc[u][t][r]), sacc[u][t][r + 1]);
                m1 = __builtin_fmaxf(__builtin_fmaxf(m1, sacc[u][t][r + 2]), sacc[u][t][r + 3]);
            }
        return halves_max(__builtin_fmaxf(m0, m1));
    };
    // multiply what has been accumulated for query tile u by alpha (per lane = per query)
    auto rescale = [&](auto iu, float alpha) __attribute__((always_inline)) {
        constexpr int u = decltype(iu)::value;
        lsum[u] *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[u][dt][r] *= alpha;
    };
    // move the scores of the tile and the reference of later lazy tiles by -d (per lane)
    auto shift = [&](auto iu, float d) __attribute__((always_inline)) {
        constexpr int u = decltype(iu)::value;
#pragma unroll
        for (int t = 0; t < NKB; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[u][t][r] -= d;
    };
    // -m_run as the sum of three bf16 numbers (exact for any float: 3 x 8 significant bits), at k-indices 0, 1, 2 of the
    // query side of the reference slab
    auto set_negm = [&](auto iu) __attribute__((always_inline)) {
        constexpr int u = decltype(iu)::value;
        const float x = -m_run[u];
        const uint32_t h1 = f2u(x) & 0xffff0000u;
        const float r1 = x - u2f(h1);
        const uint32_t h2 = f2u(r1) & 0xffff0000u;
        const float r2 = r1 - u2f(h2);
        mq[u][0] = lg == 0 ? ((h1 >> 16) | h2) : 0u;
        mq[u][1] = lg == 0 ? (f2u(r2) >> 16) : 0u;
    };

    // key mask, diagonal and ragged end on the scores of the tile in stage ST (absolute or relative alike: the mask bias
    // is additive, excluded keys become -inf)
    auto mask_apply = [&](int kt, int ST, bool diag, bool tail) __attribute__((always_inline)) {
        const int k0 = kt * KT;
        const __attribute__((address_space(3))) float* Mb = (const __attribute__((address_space(3))) float*)(ldsp + OFF_M + ST * 1024);
        sfor<QT>([&](auto iu) __attribute__((always_inline)) {
            constexpr int u = decltype(iu)::value;
            const int qi = qw0 + 32 * u + li;
#pragma unroll
            for (int t = 0; t < NKB; ++t) {
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    const int kl = 32 * t + 8 * qd + 4 * lg;
                    f32x4 mk = {1.f, 1.f, 1.f, 1.f};
                    if (HAS_MASK) mk = *(const __attribute__((address_space(3))) f32x4*)(Mb + kl);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        // (mask-1)*1e9 as the shader forms it, then into the base-2 domain.  The bias has to be one float
                        // that is then ADDED: contracted into a fused multiply-add, the unrounded product would meet the
                        // rounded one inside a reference taken from masked keys, and keys masked alike would no longer
                        // weigh alike (the mean over all keys that a fully masked row stands for).
#pragma clang fp contract(off)
                        float sv = sacc[u][t][4 * qd + e];
                        if (HAS_MASK) {
                            const float bias = ((mk[e] - 1.0f) * 1e9f) * 1.4426950408889634f;
                            sv = sv + bias;
                        }
                        if ((diag && (k0 + kl + e > qi)) || (tail && (k0 + kl + e >= S))) sv = -__builtin_inff();
                        sacc[u][t][4 * qd + e] = sv;
                    }
                }
            }
        });
    };
    // ---- softmax reference.  The first tile sets the reference m_run to its row maxima.  Every later tile is computed
    // relative to m_run (the reference slab puts -m_run into its score accumulators, so the exponentials need no further
    // arithmetic); m_run moves, with the usual rescale of what has been accumulated, only for rows that overshoot it by
    // more than 2^LAZY, and the tile's scores are then computed again against the new reference.  m_run is thus a
    // reference point at most LAZY below the true running maximum, which the softmax quotient does not depend on.
    // overshoot(): does any row of the wave exceed the reference by more than 2^LAZY?  raise(): move those rows' reference.
    float mx_tile[QT];
    auto overshoot = [&]() __attribute__((always_inline)) {
        bool any = false;
        sfor<QT>([&](auto iu) __attribute__((always_inline)) {
            constexpr int u = decltype(iu)::value;
            mx_tile[u] = tile_max(iu);
            any = any || __builtin_amdgcn_ballot_w64(mx_tile[u] > LAZY) != 0;
        });
        return any;
    };
    // mx_tile holds the tile's ABSOLUTE row maxima: rows that exceed their reference by more than 2^LAZY take the maximum
    // as their new reference, and what they have accumulated is rescaled
    auto raise = [&]() __attribute__((always_inline)) {
        mfma_drain();
        sfor<QT>([&](auto iu) __attribute__((always_inline)) {
            constexpr int u = decltype(iu)::value;
            const float m_new = mx_tile[u] > m_run[u] + LAZY ? mx_tile[u] : m_run[u];
            rescale(iu, __builtin_amdgcn_exp2f(m_run[u] - m_new));
            m_run[u] = m_new;
            set_negm(iu);
        });
    };

    // ---- p = exp2(score), O^T += V^T . P^T; V operand through the transposing LDS read: inside a 16-lane group source
    // lane j points at key j/4, 4 dims at 4*(j%4); keys of MFMA k-index (g, e): 32t + 16hh + 8*(e/4) + 4g + e%4, g = lane/32
    constexpr int VB = 1;                                    // the same choice for the V fragments of a 16-key slab
    constexpr int NSL = 2 * NKB;                             // 16-key slabs per tile
    auto phase_PV = [&](int ST, auto iinplace) __attribute__((always_inline)) {
        // INPLACE: the accumulate through mfma_inplace (first loop); else the builtin, whose hazards and spills the compiler
        // manages itself (tile 0 and the second loop, where register moves do not matter)
        constexpr bool INPLACE = decltype(iinplace)::value;
        const lds_char* vb[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) vb[dt] = vbase[dt] + ST * TILE;
        u32x2 vf[VB][DT][2];
        auto vread = [&](auto isl) __attribute__((always_inline)) {
            constexpr int SL = decltype(isl)::value;
            sfor<DT>([&](auto idt) __attribute__((always_inline)) {
                constexpr int dt = decltype(idt)::value;
                sfor<2>([&](auto ihb) __attribute__((always_inline)) {
                    constexpr int hb = decltype(ihb)::value;
                    const s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4_t*)(vb[dt] + (16 * SL + 8 * hb) * RB));
                    vf[SL % VB][dt][hb] = __builtin_bit_cast(u32x2, v);
                });
            });
        };
        if constexpr (VB == 2) vread(std::integral_constant<int, 0>{});
        sfor<NSL>([&](auto isl) __attribute__((always_inline)) {
            constexpr int SL = decltype(isl)::value, t = SL / 2, hh = SL % 2;
            if constexpr (VB == 1) vread(isl);
            else if constexpr (SL + 1 < NSL) vread(std::integral_constant<int, SL + 1>{});
            u32x4 pf[QT];
            typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2v;
            const bf16x2v one2 = __builtin_bit_cast(bf16x2v, 0x3f803f80u);
#pragma unroll
            for (int u = 0; u < QT; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float p0 = __builtin_amdgcn_exp2f(sacc[u][t][8 * hh + 2 * e]);
                    const float p1 = __builtin_amdgcn_exp2f(sacc[u][t][8 * hh + 2 * e + 1]);
                    pf[u][e] = pack_bf16x2(p0, p1);
                }
            if constexpr (VB == 2 && SL + 1 < NSL) wait_lgkmcnt<2 * DT>(); else wait_lgkmcnt<0>();
            u32x4 v4[DT];
            sfor<DT>([&](auto idt) __attribute__((always_inline)) {
                constexpr int dt = decltype(idt)::value;
                v4[dt] = u32x4{vf[SL % VB][dt][0][0], vf[SL % VB][dt][0][1], vf[SL % VB][dt][1][0], vf[SL % VB][dt][1][1]};
            });
            __builtin_amdgcn_sched_barrier(0);
            // row sums of the rounded values
#pragma unroll
            for (int u = 0; u < QT; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t w = pf[u][e];
                    lsum[u] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2v, w), one2, lsum[u], false);
                }
            __builtin_amdgcn_sched_barrier(0);
            sfor<QT>([&](auto iu) __attribute__((always_inline)) {
                constexpr int u = decltype(iu)::value;
                if constexpr (INPLACE) mfma_inplace<DT>(v4, pf[u], oacc[u]);
                else sfor<DT>([&](auto idt) __attribute__((always_inline)) { Slab<uint16_t>::run(v4[decltype(idt)::value], pf[u], oacc[u][decltype(idt)::value]); });
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // last, partial tile: rows >= S hold whatever the out-of-range transfer left; clear them (all threads)
    auto zero_tail = [&](int kt, int ST) __attribute__((always_inline)) {
        const int first = S - kt * KT;
        for (int i = tid; i < (KT - first) * NCH; i += NT) {
            const u32x4 zero = {0u, 0u, 0u, 0u};
            *(u32x4*)(lds + ST * TILE + first * RB + i * 16) = zero;
            *(u32x4*)(lds + OFF_V + ST * TILE + first * RB + i * 16) = zero;
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    };

    // tile kt's turn: its transfers have landed for everybody, the stage tile kt-1 has left takes the next transfer
    auto enter_tile = [&](int kt, int ST) __attribute__((always_inline)) {
        // tiles kt+1 .. kt+NSTG-2 may still be in flight; tile kt (this wave's part) must have landed.  Barrier without a
        // memory fence (a fence would wait for every transfer in flight): this wave's LDS accesses are drained by
        // lgkmcnt(0), its tile transfers by the counted wait.
        if constexpr (NSTG == 2) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else {
            wait_tiles_outstanding<IPT, NSTG - 2>(nkt - 1 - kt);
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        }
        if (kt + NSTG - 1 < nkt) issue(kt + NSTG - 1, ST == 0 ? NSTG - 1 : ST - 1);
        if (__builtin_expect(kt * KT + KT > S, 0)) zero_tail(kt, ST);
    };
    auto is_diag = [&](int kt) __attribute__((always_inline)) { return p.causal && (kt * KT + KT - 1 > qw0); };
    auto is_tail = [&](int kt) __attribute__((always_inline)) { return kt * KT + KT > S; };
    // What the key mask does to the tile in stage ST, as two wave-uniform answers (each lane looks at KT/64 keys):
    //   biased  - some key's mask differs from 1, so the tile's scores need the bias (most tiles of a padded batch do not,
    //             and run exactly as without a mask);
    //   dark    - every key's mask is at most 0.5: a bias of -5e8 or lower on every score.  For a row whose reference
    //             stands at an ordinary score level, every exponential of such a tile is exactly zero in float.
    auto mask_look = [&](int ST, bool& biased, bool& dark) __attribute__((always_inline)) {
        if constexpr (HAS_MASK) {
            const __attribute__((address_space(3))) float* Mb = (const __attribute__((address_space(3))) float*)(ldsp + OFF_M + ST * 1024);
            bool ne = false, lit = false;
#pragma unroll
            for (int i = 0; i < KT / 64; ++i) {
                const float mk = Mb[lane + 64 * i];
                ne = ne || mk != 1.0f;
                lit = lit || !(mk <= 0.5f);
            }
            biased = __builtin_amdgcn_ballot_w64(ne) != 0;
            dark = __builtin_amdgcn_ballot_w64(lit) == 0;
        } else {
            biased = false; dark = false;
        }
    };
    // no row of this wave still has a reference from masked keys only (around -1.4e9; an ordinary one is a score)
    auto references_lit = [&]() __attribute__((always_inline)) {
        bool low = false;
#pragma unroll
        for (int u = 0; u < QT; ++u) low = low || !(m_run[u] > -1.0e8f);
        return __builtin_amdgcn_ballot_w64(low) == 0;
    };
    auto relative_scores = [&](int kt, int ST, bool biased) __attribute__((always_inline)) {
        phase_S(ST, std::true_type{});
        const bool diag = is_diag(kt), tail = is_tail(kt);
        if (biased || diag || tail) mask_apply(kt, ST, diag, tail);
    };
    auto absolute_scores = [&](int kt, int ST, bool biased) __attribute__((always_inline)) {
        phase_S(ST, std::false_type{});
        const bool diag = is_diag(kt), tail = is_tail(kt);
        if (biased || diag || tail) mask_apply(kt, ST, diag, tail);
    };
    auto next_stage = [&](int st) __attribute__((always_inline)) { return st + 1 == NSTG ? 0 : st + 1; };

    for (int t = 1; t < NSTG - 1 && t < nkt; ++t) issue_rt(t);
    // ---- tile 0 sets the softmax reference: absolute scores, exact row maxima (rounded to bf16)
    {
        enter_tile(0, 0);
        bool biased, dark;
        mask_look(0, biased, dark);
        absolute_scores(0, 0, biased);
        sfor<QT>([&](auto iu) __attribute__((always_inline)) {
            constexpr int u = decltype(iu)::value;
            m_run[u] = tile_max(iu);
            shift(iu, m_run[u]);
            set_negm(iu);
        });
        phase_PV(0, std::false_type{});
    }
    // normalise and store this wave's rows
    auto finish = [&]() __attribute__((always_inline)) {
    mfma_drain();
#pragma unroll
        for (int u = 0; u < QT; ++u) {
            const int qi = qw0 + 32 * u + li;
            const float inv = 1.0f / fmaxf(halves_sum(lsum[u]), 1e-10f);
            if (qi < S) {
                uint16_t* Og = p.O + ((int64_t)b * S + qi) * p.o_stride + h * D;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int qd = 0; qd < 4; ++qd) {
                        const int d = 32 * dt + 8 * qd + 4 * lg;
                        fa_store4<uint16_t>(Og + d, oacc[u][dt][4 * qd] * inv, oacc[u][dt][4 * qd + 1] * inv, oacc[u][dt][4 * qd + 2] * inv, oacc[u][dt][4 * qd + 3] * inv);
                    }
            }
        }
    };
    // ---- all later tiles.  The inner loop is the common case, and nothing in it rewrites the accumulators except the PV
    // matrix products themselves (in place).  A tile whose scores overshoot the reference leaves it, is handled below
    // (reference raised from the tile's absolute scores, accumulated output rescaled, scores formed again), and the inner
    // loop is entered again.  The accumulators come back to it through opaque register moves: handed back as they are, the
    // handler's and the loop's accumulators become one value for the register allocator, which then gives them a second home
    // and moves all of them there and back in every pass of the inner loop.
    auto hand_back = [&]() __attribute__((always_inline)) {
        mfma_drain();      // the moves below are inline asm too: the compiler adds no wait states between the PV MFMAs and them
        sfor<QT>([&](auto iu) __attribute__((always_inline)) {
            sfor<DT>([&](auto idt) __attribute__((always_inline)) {
                constexpr int u = decltype(iu)::value, dt = decltype(idt)::value;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float t;
                    asm volatile("v_mov_b32 %0, %1" : "=v"(t) : "v"(oacc[u][dt][r]));
                    oacc[u][dt][r] = t;
                }
            });
        });
    };
    int kt = 1, st = 1 % NSTG;
    for (;;) {
        int over = 0;
        for (; kt < nkt; ++kt, st = next_stage(st)) {
            enter_tile(kt, st);
            // a wave whose queries all precede the tile has nothing to add (causal): it only keeps the barriers
            if (p.causal && kt * KT > qw0 + QW - 1) continue;
            bool biased, dark;
            mask_look(st, biased, dark);
            // nor has a tile whose keys are all masked out, once every row has seen a key that is not (the padding of a
            // batch): its exponentials are exact zeros
            if (HAS_MASK && dark && references_lit()) continue;
            relative_scores(kt, st, biased);
            if (__builtin_expect(overshoot(), 0)) { over = 1; break; }
            phase_PV(st, std::true_type{});
        }
        // (the flag passes through an opaque statement: the inner loop then has one exit block)
        asm volatile("" : "+s"(over));
        if (__builtin_expect(over == 0, 1)) break;
        // tile kt has been entered and its scores stand in sacc, relative to the present reference, which some row exceeds
        // by more than 2^LAZY.  The new reference comes from the tile's absolute scores (exact whatever the old reference
        // was: relative scores lose their low bits against a reference like the -1.4e9 of a fully masked tile).
        mfma_drain();
        absolute_scores(kt, st, HAS_MASK);
        sfor<QT>([&](auto iu) __attribute__((always_inline)) { mx_tile[decltype(iu)::value] = tile_max(iu); });
        raise();
        relative_scores(kt, st, HAS_MASK);
        // Against the reference just set no score exceeds 2^LAZY - in exact arithmetic.  A reference taken from masked keys
        // (-1.4e9: a row that has seen padding only so far) leaves scores a granularity of 128, and the matrix core, which
        // rounds after every k-slab, can land one step above what the single rounded sum of the absolute pass promised:
        // 2^128 overflows, and the infinity would outlive the rescale by zero that real keys bring later.  Holding the
        // scores at LAZY keeps every weight finite; rows with an ordinary reference are not touched by it.
        sfor<QT>([&](auto iu) __attribute__((always_inline)) {
            constexpr int u = decltype(iu)::value;
#pragma unroll
            for (int t = 0; t < NKB; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[u][t][r] = __builtin_fminf(sacc[u][t][r], LAZY);
        });
        phase_PV(st, std::false_type{});
        ++kt; st = next_stage(st);
        hand_back();
    }
    finish();
}

// OCC / OCCM: workgroups per CU the registers are budgeted for, without / with a key mask (applying the mask takes about
// 40 more registers)
template <int D, int QT, int NW, int NSTG, int KT, int OCC = (NW == 4 ? 2 : 1), int OCCM = OCC>
static int launch_fa16_cfg(grl_ctx* c, const Fa16Args& f, int rope_q) {
    const int qb = 32 * QT * NW;
    const int64_t nwg = (int64_t)((f.S + qb - 1) / qb) * f.H * f.B;
    GRL_REQUIRE(nwg < (1LL << 31), GRL_ERR_SHAPE, "attention: %lld workgroups exceed the grid limit", (long long)nwg);
    dim3 grid((unsigned)nwg), block(NW * 64);
    if (f.mask) {
        if (rope_q == 2) hipLaunchKernelGGL((fa2_bf16_kernel<D, 2, QT, NW, NSTG, true, KT, OCCM>), grid, block, 0, c->stream, f);
        else if (rope_q == 1) hipLaunchKernelGGL((fa2_bf16_kernel<D, 1, QT, NW, NSTG, true, KT, OCCM>), grid, block, 0, c->stream, f);
        else hipLaunchKernelGGL((fa2_bf16_kernel<D, 0, QT, NW, NSTG, true, KT, OCCM>), grid, block, 0, c->stream, f);
    } else {
        if (rope_q == 2) hipLaunchKernelGGL((fa2_bf16_kernel<D, 2, QT, NW, NSTG, false, KT, OCC>), grid, block, 0, c->stream, f);
        else if (rope_q == 1) hipLaunchKernelGGL((fa2_bf16_kernel<D, 1, QT, NW, NSTG, false, KT, OCC>), grid, block, 0, c->stream, f);
        else hipLaunchKernelGGL((fa2_bf16_kernel<D, 0, QT, NW, NSTG, false, KT, OCC>), grid, block, 0, c->stream, f);
    }
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

template <int D>
static int launch_fa16(grl_ctx* c, const FaArgs& a, int rope_q) {
    Fa16Args f{};
    f.Q = (const uint16_t*)a.Q; f.K = (const uint16_t*)a.K; f.V = (const uint16_t*)a.V;
    f.mask = a.mask; f.O = (uint16_t*)a.O; f.rope = a.rope;
    f.B = a.B; f.S = a.S; f.H = a.H; f.scale = a.scale; f.causal = a.causal;
    static const int order_env = [] { const char* e = getenv("GRL_FA_ORDER"); return e ? atoi(e) : -1; }();
    // measured: causal and short sequences do best head by head on XCD-contiguous runs; long dense sequences with
    // the plain id order (32 CUs of an XCD streaming the same K/V tiles in lockstep miss L2 together)
    f.order = order_env >= 0 ? order_env : ((a.causal || a.S <= 1024) ? 1 : 0);
    f.q_stride = a.q_stride; f.k_stride = a.k_stride; f.v_stride = a.v_stride; f.o_stride = a.o_stride;
    // GRL_FA_CFG forces a configuration, for tuning runs:
    //   1: 8 waves, 64-key tiles, deep ring   2: 8 waves, 128-key tiles   3: 4 waves, 64-key tiles, 4 stages (head dims up to 64)
    //   4: 4 waves, 128-key tiles, half-size ring (two workgroups per CU)
    //   5: 4 waves, 64-key tiles, two stages, four workgroups per CU, three with a key mask (head dims up to 64)
    static const int forced = [] { const char* e = getenv("GRL_FA_CFG"); return e ? atoi(e) : 0; }();
    // short sequences are bound by per-workgroup latency (first-tile wait, output stores): two or, where the
    // registers allow it (head dims up to 64), three to four small workgroups per CU hide each other's; long ones:
    // one 8-wave workgroup with the full ring
    int cfg = forced >= 1 && forced <= 5 ? forced : (a.S > 1024 ? 2 : (D <= 64 ? 5 : 4));
    // (head dim 128 has no 4-stage instantiation: it does not fit the 256 registers of two waves per SIMD, and the
    // accumulators must not move to AGPRs next to the in-place MFMAs; the build turns a missed register budget into an error)
    if (D == 128 && cfg == 3) cfg = 4;
    constexpr int DEEP = D == 128 ? 4 : 8;        // 128 KiB of K/V tiles: D=128 -> 4 x 32 KiB, else 8 x 16 (8) KiB
    switch (cfg) {
        case 1: return launch_fa16_cfg<D, 1, 8, DEEP, 64>(c, f, rope_q);
        case 2: return launch_fa16_cfg<D, 1, 8, DEEP / 2, 128>(c, f, rope_q);
        case 4: return launch_fa16_cfg<D, 1, 4, 2, (D == 128 ? 64 : 128)>(c, f, rope_q);
        case 5: if constexpr (D <= 64) return launch_fa16_cfg<D, 1, 4, 2, 64, 4, 3>(c, f, rope_q); else break;
        default: break;
    }
    if constexpr (D <= 64) return launch_fa16_cfg<D, 1, 4, 4, 64>(c, f, rope_q);
    else return launch_fa16_cfg<D, 1, 4, 2, 64>(c, f, rope_q);
}

template <typename T, int D>
static int launch_fa(grl_ctx* c, FaArgs& a, bool rope) {
    dim3 grid((unsigned)((a.S + 127) / 128), (unsigned)a.H, (unsigned)a.B), block(256);
    if (rope) hipLaunchKernelGGL((fa2_fwd_kernel<T, D, true>), grid, block, 0, c->stream, a);
    else hipLaunchKernelGGL((fa2_fwd_kernel<T, D, false>), grid, block, 0, c->stream, a);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// ---- head dims the MFMA kernels have no instantiation for ------------------------------------------
// (b,s,h) rows of D values -> dense rows of DP >= D values, zero filled (and back): a head dim below 128 that is
// not 32 / 64 / 128, or operands that are not 16-byte granular, run the MFMA kernels on zero-padded copies
// (zero columns add nothing to q.k, and the padded output columns are dropped).
template <typename T>
__global__ __launch_bounds__(256) void pad_heads_kernel(const T* src, int64_t src_stride, T* dst, int64_t rows, int H, int D, int DP) {
    const int64_t total = rows * DP, step = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
        const int d = (int)(i % DP);
        const int64_t row = i / DP, bs = row / H;
        const int h = (int)(row - bs * H);
        dst[i] = d < D ? src[bs * src_stride + (int64_t)h * D + d] : (T)0;
    }
}
template <typename T>
__global__ __launch_bounds__(256) void unpad_heads_kernel(const T* src, T* dst, int64_t dst_stride, int64_t rows, int H, int D, int DP) {
    const int64_t total = rows * D, step = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += step) {
        const int d = (int)(i % D);
        const int64_t row = i / D, bs = row / H;
        const int h = (int)(row - bs * H);
        dst[bs * dst_stride + (int64_t)h * D + d] = src[row * DP + d];
    }
}

// Head dims above 128: one wave per query, lanes split the head dim, keys one after the other with the online
// softmax (same constants as the MFMA kernels).  Correct for any D up to 64*NAIVE_MAX; not a fast path.
constexpr int NAIVE_MAX = 16;
template <typename T>
__global__ __launch_bounds__(256) void fa2_naive_kernel(FaArgs p, int D) {
    const int lane = threadIdx.x & 63;
    const int64_t qid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);          // (b, h, i) flat, i fastest
    const int64_t total = (int64_t)p.B * p.H * p.S;
    if (qid >= total) return;
    const int S = p.S, i = (int)(qid % S), h = (int)((qid / S) % p.H), b = (int)(qid / ((int64_t)S * p.H));
    const T* q = (const T*)p.Q + ((int64_t)b * S + i) * p.q_stride + (int64_t)h * D;
    float qv[NAIVE_MAX], o[NAIVE_MAX];
#pragma unroll
    for (int t = 0; t < NAIVE_MAX; ++t) {
        const int d = lane + 64 * t;
        qv[t] = d < D ? elem<T>::ld(q + d) : 0.f;
        o[t] = 0.f;
    }
    float m = -1e10f, l = 0.f;
    const int last = p.causal ? i : S - 1;
    for (int j = 0; j <= last; ++j) {
        const T* k = (const T*)p.K + ((int64_t)b * S + j) * p.k_stride + (int64_t)h * D;
        const T* v = (const T*)p.V + ((int64_t)b * S + j) * p.v_stride + (int64_t)h * D;
        float dot = 0.f;
#pragma unroll
        for (int t = 0; t < NAIVE_MAX; ++t) {
            const int d = lane + 64 * t;
            if (d < D) dot += qv[t] * elem<T>::ld(k + d);
        }
        dot = group_sum<64>(dot);
        float sc = dot * p.scale;
        if (p.mask) sc += (p.mask[(int64_t)b * S + j] - 1.0f) * 1e9f;
        const float mn = fmaxf(m, sc);
        const float alpha = __expf(m - mn), pw = __expf(sc - mn);
        l = l * alpha + pw;
        m = mn;
#pragma unroll
        for (int t = 0; t < NAIVE_MAX; ++t) {
            const int d = lane + 64 * t;
            if (d < D) o[t] = o[t] * alpha + pw * elem<T>::ld(v + d);
        }
    }
    const float inv = 1.0f / fmaxf(l, 1e-10f);
    T* out = (T*)p.O + ((int64_t)b * S + i) * p.o_stride + (int64_t)h * D;
#pragma unroll
    for (int t = 0; t < NAIVE_MAX; ++t) {
        const int d = lane + 64 * t;
        if (d < D) elem<T>::st(out + d, o[t] * inv);
    }
}

static unsigned fa_ew_grid(int64_t n) {
    int64_t g = (n + 255) / 256;
    return (unsigned)(g < 1 ? 1 : (g > 8192 ? 8192 : g));
}

static int fa2_common(grl_ctx* c, const char* who, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                      const void* Q, const void* K, const void* V, const float* mask, void* O,
                      int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                      float scale, int causal, int rope, float rope_base, float rope_scaling, void* workspace);

// Any head dim from 1 to 64*NAIVE_MAX and any alignment (reference backend/attention.py:403-410 reshapes with
// whatever head_dim it is given): up to 128 through zero-padded copies and the MFMA kernels, above through the
// one-wave-per-query kernel.  RoPE (even head dims up to 128) is applied to dense copies first.
static int fa2_generic(grl_ctx* c, const char* who, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                       const void* Q, const void* K, const void* V, const float* mask, void* O,
                       int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                       float scale, int causal, int rope, float rope_base, float rope_scaling) {
    const int64_t es = (int64_t)grl_dtype_size(dtype), rows = B * S * H;
    if (D > 128) {
        GRL_REQUIRE(rope == GRL_ROPE_NONE, GRL_ERR_SHAPE, "%s: RoPE needs head_dim <= 128 (got %lld)", who, (long long)D);
        GRL_REQUIRE((rows + 3) / 4 < (1LL << 31), GRL_ERR_SHAPE, "%s: too many queries", who);
        FaArgs a{};
        a.Q = Q; a.K = K; a.V = V; a.mask = mask; a.O = O;
        a.B = (int)B; a.S = (int)S; a.H = (int)H; a.scale = scale; a.causal = causal ? 1 : 0;
        a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.o_stride = o_stride;
        const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
        if (dtype == GRL_F32) hipLaunchKernelGGL(fa2_naive_kernel<float>, grid, block, 0, c->stream, a, (int)D);
        else hipLaunchKernelGGL(fa2_naive_kernel<uint16_t>, grid, block, 0, c->stream, a, (int)D);
        GRL_CHECK_LAUNCH();
        return GRL_OK;
    }
    const int64_t DP = D <= 32 ? 32 : (D <= 64 ? 64 : 128);
    const size_t dense = (size_t)(rows * D * es), padded = (size_t)(rows * DP * es);
    const void* qs = Q; const void* ks = K;
    int64_t qst = q_stride, kst = k_stride;
    grl_temp qr(c, rope != GRL_ROPE_NONE ? dense : 16), kr(c, rope != GRL_ROPE_NONE ? dense : 16);
    grl_temp qp(c, padded), kp(c, padded), vp(c, padded), op(c, padded);
    if (!qr.p || !kr.p || !qp.p || !kp.p || !vp.p || !op.p) return GRL_ERR_OOM;
    int rc = GRL_OK;
    if (rope != GRL_ROPE_NONE) {
        GRL_REQUIRE(D % 2 == 0, GRL_ERR_SHAPE, "%s: RoPE needs an even head_dim (got %lld)", who, (long long)D);
        rc = grl_rope_strided(c, dtype, B, S, H, D, Q, q_stride, nullptr, qr.p, rope, rope_base, rope_scaling);
        if (!rc) rc = grl_rope_strided(c, dtype, B, S, H, D, K, k_stride, nullptr, kr.p, rope, rope_base, rope_scaling);
        if (rc) return rc;
        qs = qr.p; ks = kr.p; qst = kst = H * D;
    }
    const dim3 grid(fa_ew_grid(rows * DP)), block(256);
    auto pad = [&](const void* src, int64_t stride, void* dst) {
        if (dtype == GRL_F32) hipLaunchKernelGGL(pad_heads_kernel<float>, grid, block, 0, c->stream, (const float*)src, stride, (float*)dst, rows, (int)H, (int)D, (int)DP);
        else hipLaunchKernelGGL(pad_heads_kernel<uint16_t>, grid, block, 0, c->stream, (const uint16_t*)src, stride, (uint16_t*)dst, rows, (int)H, (int)D, (int)DP);
    };
    pad(qs, qst, qp.p); pad(ks, kst, kp.p); pad(V, v_stride, vp.p);
    GRL_CHECK_LAUNCH();
    rc = fa2_common(c, who, dtype, B, S, H, DP, qp.p, kp.p, vp.p, mask, op.p, H * DP, H * DP, H * DP, H * DP, scale, causal,
                    GRL_ROPE_NONE, rope_base, rope_scaling, nullptr);
    if (rc) return rc;
    if (dtype == GRL_F32) hipLaunchKernelGGL(unpad_heads_kernel<float>, grid, block, 0, c->stream, (const float*)op.p, (float*)O, o_stride, rows, (int)H, (int)D, (int)DP);
    else hipLaunchKernelGGL(unpad_heads_kernel<uint16_t>, grid, block, 0, c->stream, (const uint16_t*)op.p, (uint16_t*)O, o_stride, rows, (int)H, (int)D, (int)DP);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

static int fa2_common(grl_ctx* c, const char* who, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                      const void* Q, const void* K, const void* V, const float* mask, void* O,
                      int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                      float scale, int causal, int rope, float rope_base, float rope_scaling, void* workspace) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "%s: null context", who);
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "%s: bad dtype %d", who, dtype);
    GRL_REQUIRE(rope >= GRL_ROPE_NONE && rope <= GRL_ROPE_HALF, GRL_ERR_ARG, "%s: bad rope style %d", who, rope);
    GRL_REQUIRE(B >= 0 && S >= 0 && H >= 0, GRL_ERR_SHAPE, "%s: negative dimension", who);
    GRL_REQUIRE(D >= 1 && D <= 64 * NAIVE_MAX, GRL_ERR_SHAPE, "%s: head_dim must be between 1 and %d (got %lld)", who, 64 * NAIVE_MAX, (long long)D);
    GRL_REQUIRE(B < 65536 && H < 65536 && S < (1LL << 24), GRL_ERR_SHAPE, "%s: B,H must be < 65536 and S < 2^24", who);
    if (B == 0 || S == 0 || H == 0) return GRL_OK;
    GRL_REQUIRE(Q && K && V && O, GRL_ERR_ARG, "%s: null argument", who);
    const int64_t es = (int64_t)grl_dtype_size(dtype), hd = H * D;
    GRL_REQUIRE(q_stride >= hd && k_stride >= hd && v_stride >= hd && o_stride >= hd, GRL_ERR_SHAPE,
                "%s: position stride smaller than num_heads*head_dim", who);
    if (rope != GRL_ROPE_NONE) GRL_REQUIRE(rope_base > 0.f && rope_scaling != 0.f, GRL_ERR_ARG, "%s: bad rope base/scaling", who);
    const bool granular = ((((uintptr_t)Q) | ((uintptr_t)K) | ((uintptr_t)V) | ((uintptr_t)O)) & 15u) == 0 &&
                          ((q_stride | k_stride | v_stride | o_stride) * es) % 16 == 0;
    if (!((D == 32 || D == 64 || D == 128) && granular))
        return fa2_generic(c, who, dtype, B, S, H, D, Q, K, V, mask, O, q_stride, k_stride, v_stride, o_stride, scale, causal, rope,
                           rope_base, rope_scaling);

    FaArgs a{};
    a.Q = Q; a.K = K; a.V = V; a.mask = mask; a.O = O;
    a.B = (int)B; a.S = (int)S; a.H = (int)H; a.scale = scale; a.causal = causal ? 1 : 0;
    a.q_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.o_stride = o_stride;

    GRL_REQUIRE(S * std::max(std::max(q_stride, k_stride), std::max(v_stride, o_stride)) * es < (1LL << 31), GRL_ERR_SHAPE,
                "%s: one batch entry must span less than 2 GiB", who);
    void* own = nullptr;      // rotate-half workspace
    void* own2 = nullptr;     // rotated K of the bf16 fused path
    int rc = GRL_OK;
    int rope_q = rope == GRL_ROPE_INTERLEAVED ? 1 : 0;
    if (rope == GRL_ROPE_HALF && dtype == GRL_BF16) {
        // bf16: the kernel rotates the query rows as it loads them (both halves of a pair are chunks of the same
        // lane); every K row is rotated exactly once here, from the table kept on the context
        const float* tab = nullptr;
        rc = grl_rope_table_get(c, (int)S, (int)D, rope_base, rope_scaling, GRL_ROPE_HALF, &tab);
        if (rc) return rc;
        a.rope = (const float2*)tab;
        own2 = grl_malloc(c, (size_t)B * S * H * D * 2);
        if (!own2) return GRL_ERR_OOM;
        rc = grl_rope_half_apply_table(c, dtype, B, S, H, D, K, k_stride, own2, tab);
        a.K = own2; a.k_stride = hd;
        rope_q = 2;
    } else if (rope == GRL_ROPE_HALF) {
        // fp32: rotate Q and K once into a workspace with the standalone kernel, then run the plain kernel on
        // the rotated copies.
        const size_t n = (size_t)B * S * H * D, bytes = n * grl_dtype_size(dtype);
        char* ws = (char*)workspace;
        if (!ws) { own = grl_malloc(c, 2 * bytes); if (!own) return GRL_ERR_OOM; ws = (char*)own; }
        rc = grl_rope_strided(c, dtype, B, S, H, D, Q, q_stride, nullptr, ws, GRL_ROPE_HALF, rope_base, rope_scaling);
        if (!rc) rc = grl_rope_strided(c, dtype, B, S, H, D, K, k_stride, nullptr, ws + bytes, GRL_ROPE_HALF, rope_base, rope_scaling);
        a.Q = ws; a.K = ws + bytes; a.q_stride = hd; a.k_stride = hd;
    } else if (rope == GRL_ROPE_INTERLEAVED) {
        // the (S, D/2) cos/sin table lives on the context and is built once per (D, base, scaling)
        const float* tab = nullptr;
        rc = grl_rope_table_get(c, (int)S, (int)D, rope_base, rope_scaling, GRL_ROPE_INTERLEAVED, &tab);
        if (rc) return rc;
        a.rope = (const float2*)tab;
        if (dtype == GRL_BF16) {
            // every K row is rotated exactly once here; the kernel rotates Q rows as it loads them
            own2 = grl_malloc(c, (size_t)B * S * H * D * 2);
            if (!own2) return GRL_ERR_OOM;
            rc = grl_rope_apply_table(c, dtype, B, S, H, D, K, k_stride, own2, tab);
            a.K = own2; a.k_stride = hd;
        }
    }
    const bool fused = rope == GRL_ROPE_INTERLEAVED;
    if (!rc) {
        if (dtype == GRL_F32) {
            rc = D == 32 ? launch_fa<float, 32>(c, a, fused) : D == 64 ? launch_fa<float, 64>(c, a, fused) : launch_fa<float, 128>(c, a, fused);
        } else {
            rc = D == 32 ? launch_fa16<32>(c, a, rope_q) : D == 64 ? launch_fa16<64>(c, a, rope_q) : launch_fa16<128>(c, a, rope_q);
        }
    }
    if (own) grl_free(c, own);   // stream order keeps the blocks alive until the kernel has finished
    if (own2) grl_free(c, own2);
    return rc;
}

extern "C" int grl_fa2_fwd(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                           const void* Q, const void* K, const void* V, const float* mask, void* O,
                           float scale, int causal, int rope, float rope_base, float rope_scaling, void* workspace) {
    const int64_t hd = H * D;
    return fa2_common(c, "grl_fa2_fwd", dtype, B, S, H, D, Q, K, V, mask, O, hd, hd, hd, hd, scale, causal, rope,
                      rope_base, rope_scaling, workspace);
}

extern "C" int grl_fa2_fwd_strided(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                                   const void* Q, const void* K, const void* V, const float* mask, void* O,
                                   int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                                   float scale, int causal, int rope, float rope_base, float rope_scaling) {
    return fa2_common(c, "grl_fa2_fwd_strided", dtype, B, S, H, D, Q, K, V, mask, O, q_stride, k_stride, v_stride,
                      o_stride, scale, causal, rope, rope_base, rope_scaling, nullptr);
}
