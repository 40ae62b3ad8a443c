// One post-LN BERT encoder layer as a fixed sequence of launches on the context stream:
//   QKV GEMM (packed weight) -> flash attention on the packed buffer -> out-proj GEMM
//   -> LayerNorm(residual) -> FFN1 GEMM + GELU epilogue -> FFN2 GEMM -> LayerNorm(residual)
// Activations stay in HBM between kernels; nothing returns to the host.
// Recipe: utils/vulkan_sentence_transformer.py:972-1035 (post-LN order, eps passed by the
// caller, tanh GELU, key-padding mask as additive -1e9 bias, heads = plain reshape of the
// last dimension :985-995).
#include "common.hpp"
#include <cmath>

extern "C" int64_t grl_bert_layer_workspace(int dtype, int64_t B, int64_t S, int64_t H, int64_t D, int64_t d_ff) {
    if (!grl_valid_dtype(dtype) || B < 0 || S < 0 || H <= 0 || D <= 0 || d_ff <= 0) return -1;
    const int64_t M = B * S, d = H * D;
    // qkv (M,3d) | attn (M,d) | proj (M,d) | ff (M,d_ff); each region padded to 256 B
    auto pad = [](int64_t v) { return (v + 255) / 256 * 256; };
    const int64_t es = (int64_t)grl_dtype_size(dtype);
    return pad(M * 3 * d * es) + 2 * pad(M * d * es) + pad(M * d_ff * es);
}

extern "C" int grl_bert_layer_fwd(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, int64_t d_ff,
                                  const grl_bert_layer* w, const float* mask, float eps, void* x, void* workspace) {
    GRL_REQUIRE(c && w && x && workspace, GRL_ERR_ARG, "grl_bert_layer_fwd: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_bert_layer_fwd: bad dtype %d", dtype);
    GRL_REQUIRE(B >= 0 && S >= 0 && H > 0 && d_ff > 0, GRL_ERR_SHAPE, "grl_bert_layer_fwd: bad shape");
    GRL_REQUIRE(D >= 1 && D <= 1024, GRL_ERR_SHAPE, "grl_bert_layer_fwd: head_dim must be between 1 and 1024 (got %lld)", (long long)D);
    GRL_REQUIRE(w->w_qkv && w->w_o && w->w_ff1 && w->w_ff2 && w->ln1_g && w->ln1_b && w->ln2_g && w->ln2_b,
                GRL_ERR_ARG, "grl_bert_layer_fwd: null weight");
    if (B == 0 || S == 0) return GRL_OK;
    const int64_t M = B * S, d = H * D, es = (int64_t)grl_dtype_size(dtype);
    auto pad = [](int64_t v) { return (v + 255) / 256 * 256; };
    char* qkv = (char*)workspace;
    char* attn = qkv + pad(M * 3 * d * es);
    char* proj = attn + pad(M * d * es);
    char* ff = proj + pad(M * d * es);
    int rc;
    grl_lap_mark(c);
    if ((rc = grl_gemm_nt(c, dtype, dtype, M, 3 * d, d, x, w->w_qkv, w->b_qkv, qkv, GRL_EPI_NONE))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_fa2_fwd_strided(c, dtype, B, S, H, D, qkv, qkv + d * es, qkv + 2 * d * es, mask, attn,
                                  3 * d, 3 * d, 3 * d, d, 1.0f / sqrtf((float)D), 0, GRL_ROPE_NONE, 10000.f, 1.f))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_gemm_nt(c, dtype, dtype, M, d, d, attn, w->w_o, w->b_o, proj, GRL_EPI_NONE))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_layernorm(c, dtype, M, d, x, proj, w->ln1_g, w->ln1_b, eps, x))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_gemm_nt(c, dtype, dtype, M, d_ff, d, x, w->w_ff1, w->b_ff1, ff, GRL_EPI_GELU))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_gemm_nt(c, dtype, dtype, M, d, d_ff, ff, w->w_ff2, w->b_ff2, proj, GRL_EPI_NONE))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_layernorm(c, dtype, M, d, x, proj, w->ln2_g, w->ln2_b, eps, x))) return rc;
    grl_lap_mark(c);
    return GRL_OK;
}

// ---- the same layer without a LayerNorm pass: the residual stream is kept as raw rows + row statistics ----------
extern "C" int64_t grl_bert_layer_fused_workspace(int dtype, int64_t B, int64_t S, int64_t H, int64_t D, int64_t d_ff) {
    if (!grl_valid_dtype(dtype) || B < 0 || S < 0 || H <= 0 || D <= 0 || d_ff <= 0) return -1;
    const int64_t M = B * S, d = H * D;
    auto pad = [](int64_t v) { return (v + 255) / 256 * 256; };
    const int64_t es = (int64_t)grl_dtype_size(dtype);
    // qkv (M,3d) | attn (M,d) | ff (M,d_ff) | statistics of the middle residual (M,2) | row-statistics partials
    return pad(M * 3 * d * es) + pad(M * d * es) + pad(M * d_ff * es) + pad(M * 8) + pad(grl_gemm_nt_resln_workspace(M, d));
}

extern "C" int grl_bert_layer_fwd_fused(grl_ctx* c, int dtype, int64_t B, int64_t S, int64_t H, int64_t D, int64_t d_ff,
                                        const grl_bert_layer_fused* w, const float* mask, float eps, void* r, float* stats,
                                        void* workspace) {
    GRL_REQUIRE(c && w && r && stats && workspace, GRL_ERR_ARG, "grl_bert_layer_fwd_fused: null argument");
    GRL_REQUIRE(grl_valid_dtype(dtype), GRL_ERR_ARG, "grl_bert_layer_fwd_fused: bad dtype %d", dtype);
    GRL_REQUIRE(B >= 0 && S >= 0 && H > 0 && d_ff > 0, GRL_ERR_SHAPE, "grl_bert_layer_fwd_fused: bad shape");
    GRL_REQUIRE(D >= 1 && D <= 1024, GRL_ERR_SHAPE, "grl_bert_layer_fwd_fused: head_dim must be between 1 and 1024 (got %lld)", (long long)D);
    GRL_REQUIRE(w->ws_qkv && w->c_qkv && w->bf_qkv && w->in_g && w->in_b && w->w_o && w->ln1_g && w->ln1_b && w->ws_ff1 && w->c_ff1 &&
                w->bf_ff1 && w->w_ff2, GRL_ERR_ARG, "grl_bert_layer_fwd_fused: null weight");
    const int64_t M = B * S, d = H * D, es = (int64_t)grl_dtype_size(dtype), slab = 128 / es;
    GRL_REQUIRE(d % slab == 0 && d_ff % slab == 0, GRL_ERR_SHAPE,
                "grl_bert_layer_fwd_fused: d_model (%lld) and d_ff (%lld) must be multiples of %lld; use grl_bert_layer_fwd",
                (long long)d, (long long)d_ff, (long long)slab);
    if (B == 0 || S == 0) return GRL_OK;
    auto pad = [](int64_t v) { return (v + 255) / 256 * 256; };
    char* qkv = (char*)workspace;
    char* attn = qkv + pad(M * 3 * d * es);
    char* ff = attn + pad(M * d * es);
    float* stats1 = (float*)(ff + pad(M * d_ff * es));
    char* part = (char*)stats1 + pad(M * 8);
    int rc;
    grl_lap_mark(c);
    if ((rc = grl_ln_gemm_nt_stats(c, dtype, dtype, M, 3 * d, d, r, w->ws_qkv, w->c_qkv, w->bf_qkv, stats, qkv, GRL_EPI_NONE))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_fa2_fwd_strided(c, dtype, B, S, H, D, qkv, qkv + d * es, qkv + 2 * d * es, mask, attn,
                                  3 * d, 3 * d, 3 * d, d, 1.0f / sqrtf((float)D), 0, GRL_ROPE_NONE, 10000.f, 1.f))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_gemm_nt_resln(c, dtype, M, d, d, attn, w->w_o, w->b_o, r, stats, w->in_g, w->in_b, r, eps, stats1, part))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_ln_gemm_nt_stats(c, dtype, dtype, M, d_ff, d, r, w->ws_ff1, w->c_ff1, w->bf_ff1, stats1, ff, GRL_EPI_GELU))) return rc;
    grl_lap_mark(c);
    if ((rc = grl_gemm_nt_resln(c, dtype, M, d, d_ff, ff, w->w_ff2, w->b_ff2, r, stats1, w->ln1_g, w->ln1_b, r, eps, stats, part))) return rc;
    grl_lap_mark(c);
    return GRL_OK;
}
