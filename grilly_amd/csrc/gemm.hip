// Host side of the GEMM family: argument checks and the C entry points.  The kernels live in
// gemm_kernels.hpp; their instantiations are spread over gemm_inst_*.hip (one storage-type pair each)
// so that they compile in parallel.
#include "gemm_kernels.hpp"

extern template int dispatch_epi<float, float>(grl_ctx*, GemmArgs&, int);
extern template int dispatch_epi<uint16_t, uint16_t>(grl_ctx*, GemmArgs&, int);
extern template int dispatch_epi<uint16_t, float>(grl_ctx*, GemmArgs&, int);
extern template int dispatch_epi<float, uint16_t>(grl_ctx*, GemmArgs&, int);

static int dispatch_types(grl_ctx* c, GemmArgs& a, int in_dtype, int out_dtype, int epi) {
    if (in_dtype == GRL_F32 && out_dtype == GRL_F32) return dispatch_epi<float, float>(c, a, epi);
    if (in_dtype == GRL_BF16 && out_dtype == GRL_BF16) return dispatch_epi<uint16_t, uint16_t>(c, a, epi);
    if (in_dtype == GRL_BF16 && out_dtype == GRL_F32) return dispatch_epi<uint16_t, float>(c, a, epi);
    if (in_dtype == GRL_F32 && out_dtype == GRL_BF16) return dispatch_epi<float, uint16_t>(c, a, epi);
    grl_set_error("gemm: bad dtype in=%d out=%d", in_dtype, out_dtype);
    return GRL_ERR_ARG;
}

extern template int dispatch_epi_ln<float, float>(grl_ctx*, GemmArgs&, int);
extern template int dispatch_epi_ln<uint16_t, uint16_t>(grl_ctx*, GemmArgs&, int);
extern template int dispatch_epi_ln<uint16_t, float>(grl_ctx*, GemmArgs&, int);
extern template int dispatch_epi_ln<float, uint16_t>(grl_ctx*, GemmArgs&, int);

static int dispatch_types_ln(grl_ctx* c, GemmArgs& a, int in_dtype, int out_dtype, int epi) {
    if (in_dtype == GRL_F32 && out_dtype == GRL_F32) return dispatch_epi_ln<float, float>(c, a, epi);
    if (in_dtype == GRL_BF16 && out_dtype == GRL_BF16) return dispatch_epi_ln<uint16_t, uint16_t>(c, a, epi);
    if (in_dtype == GRL_BF16 && out_dtype == GRL_F32) return dispatch_epi_ln<uint16_t, float>(c, a, epi);
    if (in_dtype == GRL_F32 && out_dtype == GRL_BF16) return dispatch_epi_ln<float, uint16_t>(c, a, epi);
    grl_set_error("gemm: bad dtype in=%d out=%d", in_dtype, out_dtype);
    return GRL_ERR_ARG;
}

static int check_dims(const char* who, int64_t M, int64_t N, int64_t K) {
    GRL_REQUIRE(M >= 0 && N >= 0 && K >= 0, GRL_ERR_SHAPE, "%s: negative dimension", who);
    GRL_REQUIRE(M < (1LL << 31) && N < (1LL << 31) && K < (1LL << 31), GRL_ERR_SHAPE, "%s: dimension exceeds 2^31-1", who);
    return GRL_OK;
}

// K == 0: the sum is empty, C = epi(bias)
template <typename OutT>
__global__ __launch_bounds__(256) void bias_fill_kernel(OutT* C, const float* bias, int64_t total, int N, int epi, GemmArgs p) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    float v = bias ? bias[i % N] : 0.f;
    v = epi == EPI_GELU ? epi_apply<EPI_GELU>(v, p) : epi == EPI_SILU ? epi_apply<EPI_SILU>(v, p) : epi == EPI_RT ? epi_apply<EPI_RT>(v, p) : v;
    elem<OutT>::st(C + i, v);
}

template <typename OutT>
__global__ __launch_bounds__(256) void bias_residual_kernel(OutT* C, const OutT* R, const float* bias, int64_t total, int N) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    elem<OutT>::st(C + i, elem<OutT>::ld(R + i) + (bias ? bias[i % N] : 0.f));
}

// may_allocate == false: for the entry point that promises to allocate nothing (the launcher then leaves the K loop whole
// instead of sharing it out through a pool buffer)
static int gemm_nt_act_impl(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                            const void* A, const void* W, const float* bias, void* C, int epilogue,
                            float alpha, float beta, bool may_allocate) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_gemm_nt: null context");
    GRL_REQUIRE(grl_valid_dtype(in_dtype) && grl_valid_dtype(out_dtype), GRL_ERR_ARG, "grl_gemm_nt: bad dtype");
    GRL_REQUIRE(epilogue >= GRL_EPI_NONE && epilogue <= GRL_EPI_ROSWISH, GRL_ERR_ARG, "grl_gemm_nt: bad epilogue %d", epilogue);
    int rc = check_dims("grl_gemm_nt", M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    GRL_REQUIRE(C && (K == 0 || (A && W)), GRL_ERR_ARG, "grl_gemm_nt: null argument");
    GemmArgs a{};
    a.A = A; a.W = W; a.bias = bias; a.C = C;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.act = epilogue; a.alpha = alpha; a.beta = beta;
    a.no_alloc = !may_allocate;
    const int epi = epilogue <= GRL_EPI_SILU ? epilogue : EPI_RT;
    if (K == 0) {
        int64_t total = M * N;
        GRL_REQUIRE((total + 255) / 256 < (1LL << 31), GRL_ERR_SHAPE, "grl_gemm_nt: output too large");
        if (out_dtype == GRL_F32) hipLaunchKernelGGL(bias_fill_kernel<float>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, c->stream, (float*)C, bias, total, (int)N, epi, a);
        else hipLaunchKernelGGL(bias_fill_kernel<uint16_t>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, c->stream, (uint16_t*)C, bias, total, (int)N, epi, a);
        GRL_CHECK_LAUNCH();
        return GRL_OK;
    }
    return dispatch_types(c, a, in_dtype, out_dtype, epi);
}

extern "C" int grl_gemm_nt_act(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                               const void* A, const void* W, const float* bias, void* C, int epilogue,
                               float alpha, float beta) {
    return gemm_nt_act_impl(c, in_dtype, out_dtype, M, N, K, A, W, bias, C, epilogue, alpha, beta, true);
}

extern "C" int grl_gemm_nt_res(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                               const void* A, const void* W, const float* bias, const void* residual, void* C) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_gemm_nt_res: null context");
    GRL_REQUIRE(grl_valid_dtype(in_dtype) && grl_valid_dtype(out_dtype), GRL_ERR_ARG, "grl_gemm_nt_res: bad dtype");
    int rc = check_dims("grl_gemm_nt_res", M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    GRL_REQUIRE(C && residual && (K == 0 || (A && W)), GRL_ERR_ARG, "grl_gemm_nt_res: null argument");
    if (K == 0) {       // empty sum: C = bias + residual (element-wise, so C may be the residual)
        int64_t total = M * N;
        GRL_REQUIRE((total + 255) / 256 < (1LL << 31), GRL_ERR_SHAPE, "grl_gemm_nt_res: output too large");
        const dim3 grid((unsigned)((total + 255) / 256));
        if (out_dtype == GRL_F32) hipLaunchKernelGGL(bias_residual_kernel<float>, grid, dim3(256), 0, c->stream, (float*)C, (const float*)residual, bias, total, (int)N);
        else hipLaunchKernelGGL(bias_residual_kernel<uint16_t>, grid, dim3(256), 0, c->stream, (uint16_t*)C, (const uint16_t*)residual, bias, total, (int)N);
        GRL_CHECK_LAUNCH();
        return GRL_OK;
    }
    GemmArgs a{};
    a.A = A; a.W = W; a.bias = bias; a.C = C; a.residual = residual;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    return dispatch_types(c, a, in_dtype, out_dtype, EPI_RES);
}

extern "C" int grl_gemm_nt(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                           const void* A, const void* W, const float* bias, void* C, int epilogue) {
    return grl_gemm_nt_act(c, in_dtype, out_dtype, M, N, K, A, W, bias, C, epilogue, 1.0f, 1.0f);
}

extern "C" int grl_glu_nt(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                          const void* x, const void* W_gate, const void* W_up, const float* b_gate,
                          const float* b_up, void* out, float* gate_cache, float* up_cache, int activation) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_glu_nt: null context");
    GRL_REQUIRE(grl_valid_dtype(in_dtype) && grl_valid_dtype(out_dtype), GRL_ERR_ARG, "grl_glu_nt: bad dtype");
    GRL_REQUIRE(activation == GRL_EPI_SILU || activation == GRL_EPI_RELU || activation == GRL_EPI_GELU, GRL_ERR_ARG,
                "grl_glu_nt: activation must be GRL_EPI_SILU, GRL_EPI_RELU or GRL_EPI_GELU (got %d)", activation);
    int rc = check_dims("grl_glu_nt", M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    GRL_REQUIRE(out && K > 0 && x && W_gate && W_up, GRL_ERR_ARG, "grl_glu_nt: null argument or K == 0");
    GemmArgs a{};
    a.A = x; a.W = W_gate; a.W2 = W_up; a.C = out;
    // the reference applies biases only when both are present (backend/_glu_append.py:68)
    if (b_gate && b_up) { a.bias = b_gate; a.bias2 = b_up; }
    a.cache1 = gate_cache; a.cache2 = up_cache;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.act = activation;
    return dispatch_types(c, a, in_dtype, out_dtype, EPI_GLU);
}

int grl_ln_stats(grl_ctx* c, int dtype, int64_t rows, int64_t F, const void* x, float eps, float* stats);

// LayerNorm folded into the GEMM: row statistics of x (one pass over x, 8 bytes per row out), then the GEMM on the
// raw rows with the scaled weight; the normalised rows are never formed.
extern "C" int grl_ln_gemm_nt(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                              const void* W_scaled, const float* colsum, const float* bias_folded, float eps,
                              float* stats, void* out) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_ln_gemm_nt: null context");
    GRL_REQUIRE(grl_valid_dtype(in_dtype) && grl_valid_dtype(out_dtype), GRL_ERR_ARG, "grl_ln_gemm_nt: bad dtype");
    int rc = check_dims("grl_ln_gemm_nt", M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    GRL_REQUIRE(out && K > 0 && x && W_scaled && colsum && stats, GRL_ERR_ARG, "grl_ln_gemm_nt: null argument or K == 0");
    rc = grl_ln_stats(c, in_dtype, M, K, x, eps, stats);
    if (rc) return rc;
    GemmArgs a{};
    a.A = x; a.W = W_scaled; a.bias = bias_folded; a.C = out;
    a.ln_stats = stats; a.ln_c = colsum;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    return dispatch_types_ln(c, a, in_dtype, out_dtype, EPI_NONE);
}

// the same with the row statistics given (computed earlier, e.g. by the GEMM that produced x) and a choice of epilogue
extern "C" int grl_ln_gemm_nt_stats(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                                    const void* W_scaled, const float* colsum, const float* bias_folded,
                                    const float* stats, void* out, int epilogue) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_ln_gemm_nt_stats: null context");
    GRL_REQUIRE(grl_valid_dtype(in_dtype) && grl_valid_dtype(out_dtype), GRL_ERR_ARG, "grl_ln_gemm_nt_stats: bad dtype");
    GRL_REQUIRE(epilogue == GRL_EPI_NONE || epilogue == GRL_EPI_GELU, GRL_ERR_ARG,
                "grl_ln_gemm_nt_stats: epilogue must be GRL_EPI_NONE or GRL_EPI_GELU (got %d)", epilogue);
    int rc = check_dims("grl_ln_gemm_nt_stats", M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    GRL_REQUIRE(out && K > 0 && x && W_scaled && colsum && bias_folded && stats, GRL_ERR_ARG, "grl_ln_gemm_nt_stats: null argument or K == 0");
    GemmArgs a{};
    a.A = x; a.W = W_scaled; a.bias = bias_folded; a.C = out;
    a.ln_stats = stats; a.ln_c = colsum;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.act = epilogue;
    return dispatch_types_ln(c, a, in_dtype, out_dtype, epilogue == GRL_EPI_GELU ? EPI_GELU : EPI_NONE);
}

// which kernel / tile size grl_gemm_nt and its siblings pick for a 16-byte aligned problem (pure host arithmetic)
extern "C" int grl_gemm_plan(int dtype, int64_t M, int64_t N, int64_t K, int dual, int compute_units) {
    if (!grl_valid_dtype(dtype) || M <= 0 || N <= 0 || K <= 0 || compute_units <= 0) return GRL_ERR_ARG;
    return gemm_variant(M, N, K, dtype == GRL_F32 ? 4 : 2, dual != 0, compute_units);
}

// ---- C = A.W^T + bias + LayerNorm(R), and the row statistics of C ------------------------------------------------
extern template int launch_gemm_resln<float, float>(grl_ctx*, GemmArgs&, int*);
extern template int launch_gemm_resln<uint16_t, uint16_t>(grl_ctx*, GemmArgs&, int*);

// per row: the per-tile partials {sum, sum of squares} merged in a fixed order into {1/sd, mean/sd} (var = E[x^2] - mean^2
// in float: rows whose mean is more than about a hundred spreads away from zero lose the variance to cancellation,
// the same conditioning as the folded LayerNorm that consumes the statistics)
__global__ __launch_bounds__(256) void ln_stats_merge_kernel(const float* __restrict__ part, float* __restrict__ stats, int M, int N,
                                                             int nparts, float eps) {
    const int m = blockIdx.x * 256 + threadIdx.x;
    if (m >= M) return;
    float tot = 0.f, sq = 0.f;
    for (int t = 0; t < nparts; ++t) {
        const float2 pr = *(const float2*)(part + ((int64_t)t * M + m) * 2);
        tot += pr.x; sq += pr.y;
    }
    const float mean = tot / (float)N;
    const float var = fmaxf(sq / (float)N - mean * mean, 0.f);
    const float sd = sqrtf(var + eps);
    *(float2*)(stats + 2 * (int64_t)m) = make_float2(1.0f / sd, mean / sd);
}

extern "C" int64_t grl_gemm_nt_resln_workspace(int64_t M, int64_t N) {
    if (M < 0 || N < 0) return -1;
    return ((N + 127) / 128) * M * 8 + 256;          // one {sum, sum of squares} pair per row and 128-column tile (the narrowest tile)
}

extern "C" int grl_gemm_nt_resln(grl_ctx* c, int dtype, int64_t M, int64_t N, int64_t K, const void* A, const void* W,
                                 const float* bias, const void* R, const float* r_stats, const float* r_gamma,
                                 const float* r_beta, void* C, float eps, float* stats_out, void* workspace) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_gemm_nt_resln: null context");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_gemm_nt_resln: bad dtype");
    int rc = check_dims("grl_gemm_nt_resln", M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    GRL_REQUIRE(A && W && R && r_stats && r_gamma && r_beta && C && stats_out && workspace && K > 0, GRL_ERR_ARG,
                "grl_gemm_nt_resln: null argument or K == 0");
    GRL_REQUIRE((((uintptr_t)workspace) & 15u) == 0 && (((uintptr_t)stats_out) & 15u) == 0, GRL_ERR_ARG, "grl_gemm_nt_resln: workspace and stats_out must be 16-byte aligned");
    GemmArgs a{};
    a.A = A; a.W = W; a.bias = bias; a.C = C; a.residual = R;
    a.res_stats = r_stats; a.res_gamma = r_gamma; a.res_beta = r_beta; a.part_out = (float*)workspace;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    int tile_cols = 0;
    rc = dtype == GRL_F32 ? launch_gemm_resln<float, float>(c, a, &tile_cols) : launch_gemm_resln<uint16_t, uint16_t>(c, a, &tile_cols);
    if (rc) return rc;
    const int nparts = (int)((N + tile_cols - 1) / tile_cols);
    hipLaunchKernelGGL(ln_stats_merge_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, c->stream, (const float*)workspace, stats_out,
                       (int)M, (int)N, nparts, eps);
    GRL_CHECK_LAUNCH();
    return GRL_OK;
}

// stats == given: {1/sd, mean/sd} per row of x are the caller's (from grl_ln_stats or a GEMM epilogue); else they are computed here
static int ln_glu_nt_impl(grl_ctx* c, const char* who, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                          const void* Wg_scaled, const void* Wu_scaled, const float* colsum_gate, const float* colsum_up,
                          const float* bias_gate_folded, const float* bias_up_folded, bool given, float eps, float* stats,
                          void* out, int activation) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "%s: null context", who);
    GRL_REQUIRE(grl_valid_dtype(in_dtype) && grl_valid_dtype(out_dtype), GRL_ERR_ARG, "%s: bad dtype", who);
    GRL_REQUIRE(activation == GRL_EPI_SILU || activation == GRL_EPI_RELU || activation == GRL_EPI_GELU, GRL_ERR_ARG,
                "%s: activation must be GRL_EPI_SILU, GRL_EPI_RELU or GRL_EPI_GELU (got %d)", who, activation);
    int rc = check_dims(who, M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    GRL_REQUIRE(out && K > 0 && x && Wg_scaled && Wu_scaled && colsum_gate && colsum_up && bias_gate_folded && bias_up_folded && stats,
                GRL_ERR_ARG, "%s: null argument or K == 0", who);
    if (!given) {
        rc = grl_ln_stats(c, in_dtype, M, K, x, eps, stats);
        if (rc) return rc;
    }
    GemmArgs a{};
    a.A = x; a.W = Wg_scaled; a.W2 = Wu_scaled; a.C = out;
    a.bias = bias_gate_folded; a.bias2 = bias_up_folded;
    a.ln_stats = stats; a.ln_c = colsum_gate; a.ln_c2 = colsum_up;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.act = activation;
    return dispatch_types_ln(c, a, in_dtype, out_dtype, EPI_GLU);
}

extern "C" int grl_ln_glu_nt(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                             const void* Wg_scaled, const void* Wu_scaled, const float* colsum_gate, const float* colsum_up,
                             const float* bias_gate_folded, const float* bias_up_folded, float eps, float* stats,
                             void* out, int activation) {
    return ln_glu_nt_impl(c, "grl_ln_glu_nt", in_dtype, out_dtype, M, N, K, x, Wg_scaled, Wu_scaled, colsum_gate, colsum_up,
                          bias_gate_folded, bias_up_folded, false, eps, stats, out, activation);
}
extern "C" int grl_ln_glu_nt_stats(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                                   const void* Wg_scaled, const void* Wu_scaled, const float* colsum_gate, const float* colsum_up,
                                   const float* bias_gate_folded, const float* bias_up_folded, const float* stats,
                                   void* out, int activation) {
    return ln_glu_nt_impl(c, "grl_ln_glu_nt_stats", in_dtype, out_dtype, M, N, K, x, Wg_scaled, Wu_scaled, colsum_gate, colsum_up,
                          bias_gate_folded, bias_up_folded, true, 0.f, const_cast<float*>(stats), out, activation);
}

extern "C" int grl_swiglu_nt(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                             const void* x, const void* W_gate, const void* W_up, const float* b_gate,
                             const float* b_up, void* out, float* gate_cache, float* up_cache) {
    return grl_glu_nt(c, in_dtype, out_dtype, M, N, K, x, W_gate, W_up, b_gate, b_up, out, gate_cache, up_cache, GRL_EPI_SILU);
}

extern "C" int grl_gemm_nn(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                           const void* A, const void* B, void* C, void* workspace) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_gemm_nn: null context");
    GRL_REQUIRE(grl_valid_dtype(in_dtype) && grl_valid_dtype(out_dtype), GRL_ERR_ARG, "grl_gemm_nn: bad dtype");
    int rc = check_dims("grl_gemm_nn", M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    if (K == 0) return grl_gemm_nt(c, in_dtype, out_dtype, M, N, 0, A, B, nullptr, C, GRL_EPI_NONE);
    GRL_REQUIRE(A && B && C, GRL_ERR_ARG, "grl_gemm_nn: null argument");
    void* ws = workspace;
    void* own = nullptr;
    if (!ws) {
        own = grl_malloc(c, (size_t)K * N * grl_dtype_size(in_dtype));
        if (!own) return GRL_ERR_OOM;
        ws = own;
    }
    rc = grl_transpose2d(c, in_dtype, K, N, B, ws);   // (K,N) -> (N,K)
    if (!rc) rc = grl_gemm_nt(c, in_dtype, out_dtype, M, N, K, A, ws, nullptr, C, GRL_EPI_NONE);
    if (own) grl_free(c, own);   // stream order keeps the block alive until the GEMM has read it
    return rc;
}

// ---------------------------------------------------------------------------------------------------
// C = A.B without any allocation: the transposed copy of B that grl_gemm_nn takes from the caching pool (or
// from a caller's workspace) lives in a file-scope device array instead.  Every GPU the library runs on
// holds its own copy of the array (at its own address) until the process ends.  The array's name is only a
// host-side handle: its device address is looked up once per device with that device current, and from
// then on only that address is handed to kernels.
#define GRL_NN_SCRATCH_BYTES (32u << 20)
static __device__ __align__(256) unsigned char scratch[GRL_NN_SCRATCH_BYTES];

static std::mutex g_scratch_mu;
static std::mutex g_scratch_pair_mu;     // held from a call's transpose launch to its GEMM launch
static void* g_scratch_ptr[64];          // per device ordinal; null until looked up

// device address of this GPU's copy of `scratch` (looked up on first use, with the device current)
static int nn_scratch_address(grl_ctx* c, void** out) {
    GRL_REQUIRE(c->device >= 0 && c->device < 64, GRL_ERR_ARG, "grl_gemm_nn_noalloc: device ordinal %d out of range", c->device);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[c->device]) {
        GRL_CHECK_HIP(hipSetDevice(c->device));
        void* ptr = nullptr;
        GRL_CHECK_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
        GRL_REQUIRE(ptr, GRL_ERR_HIP, "grl_gemm_nn_noalloc: the scratch array has no device address");
        g_scratch_ptr[c->device] = ptr;
    }
    *out = g_scratch_ptr[c->device];
    return GRL_OK;
}

// called by grl_create so that the lookup happens at set-up, not inside a caller's no-allocation region
int grl_gemm_scratch_init(grl_ctx* c) {
    void* p = nullptr;
    return nn_scratch_address(c, &p);
}

extern "C" int64_t grl_gemm_nn_noalloc_max_bytes(void) { return (int64_t)GRL_NN_SCRATCH_BYTES; }

extern "C" int grl_gemm_nn_noalloc(grl_ctx* c, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                                   const void* A, const void* B, void* C) {
    GRL_REQUIRE(c, GRL_ERR_ARG, "grl_gemm_nn_noalloc: null context");
    GRL_REQUIRE(grl_valid_dtype(in_dtype) && grl_valid_dtype(out_dtype), GRL_ERR_ARG, "grl_gemm_nn_noalloc: bad dtype");
    int rc = check_dims("grl_gemm_nn_noalloc", M, N, K);
    if (rc) return rc;
    if (M == 0 || N == 0) return GRL_OK;
    if (K == 0) return gemm_nt_act_impl(c, in_dtype, out_dtype, M, N, 0, A, B, nullptr, C, GRL_EPI_NONE, 1.0f, 1.0f, false);
    GRL_REQUIRE(A && B && C, GRL_ERR_ARG, "grl_gemm_nn_noalloc: null argument");
    const int64_t need = K * N * (int64_t)grl_dtype_size(in_dtype);
    GRL_REQUIRE(need <= (int64_t)GRL_NN_SCRATCH_BYTES, GRL_ERR_SHAPE,
                "grl_gemm_nn_noalloc: B (%lld x %lld, %lld bytes) exceeds the %u-byte static scratch; use grl_gemm_nn",
                (long long)K, (long long)N, (long long)need, GRL_NN_SCRATCH_BYTES);
    void* ws = nullptr;
    rc = nn_scratch_address(c, &ws);
    if (rc) return rc;
    // the transpose overwrites every byte of the (N,K) image the GEMM reads, so nothing of the previous
    // call's contents needs clearing.  The two launches must sit next to each other on the stream: host threads
    // that share a context share its stream, and without the lock thread B's transpose could be enqueued between
    // thread A's transpose and A's GEMM (A would then multiply by B's matrix).
    std::lock_guard<std::mutex> pair(g_scratch_pair_mu);
    rc = grl_transpose2d(c, in_dtype, K, N, B, ws);   // (K,N) -> (N,K)
    if (!rc) rc = gemm_nt_act_impl(c, in_dtype, out_dtype, M, N, K, A, ws, nullptr, C, GRL_EPI_NONE, 1.0f, 1.0f, false);
    return rc;
}
