/*
 * oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT.
 *
 * A plain-C, CPU restatement of the arithmetic of grilly's transformer-forward shaders,
 * in the shaders' own evaluation order (one output element per "invocation", fp32,
 * ascending-k sums).  It exists to check the HIP kernels and to time the reference
 * algorithm on host cores; nothing in the shipped library may link, load or call it.
 * Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py use it.
 *
 * Every function names the reference text it follows (paths relative to the reference
 * repository).  The reference contains no compilable C/C++ of its own (it is Python +
 * GLSL), so there is no oracle/_ref build; this restatement is pinned instead by
 *   - the float64 closed forms in oracle/oracle_np.py,
 *   - the reference's own known answers (tests/test_pytorch_ops.py:42-48 matmul,
 *     tests/test_gpu_operations.py:109-118 gelu(0)=0, :169-195 swiglu formula,
 *     :197-205 layernorm moments), and
 *   - invariants (linearity, softmax special cases, RoPE relative-position property),
 * all exercised in tests/test_oracle.py.
 *
 * Parity status: the reference holds no numeric test for flash_attention2, the fused
 * linears, fused_swiglu or the QKV projection ("parity unpinned" at the level of the
 * reference's own tests); they are pinned by the closed forms and invariants above.
 *
 * OpenMP parallelises over output rows only; each output element is still computed by one
 * sequential fp32 loop, as one shader invocation would.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define EPI_NONE 0
#define EPI_GELU 1
#define EPI_SILU 2
#define EPI_RELU 3
#define EPI_GCU 4
#define EPI_ROSWISH 5

/* shaders/fused-linear-gelu.glsl:45-63 (same body as shaders/activation-gelu.glsl:33-50) */
static inline float gelu_shader(float x) {
    float c = x < -50.0f ? -50.0f : (x > 50.0f ? 50.0f : x);
    float cubed = c * c * c;
    float inner = 0.7978845608028654f * (c + 0.044715f * cubed);
    float r = 0.5f * x * (1.0f + tanhf(inner));
    if (fabsf(x) > 50.0f) r = (x > 0.0f) ? x : 0.0f;
    return r;
}

/* shaders/fused-linear-silu.glsl:43-48 */
static inline float silu_clamped(float x) {
    float c = x < -88.0f ? -88.0f : (x > 88.0f ? 88.0f : x);
    return x * (1.0f / (1.0f + expf(-c)));
}

/* shaders/fused-swiglu.glsl:44-46 */
static inline float silu_plain(float x) { return x / (1.0f + expf(-x)); }

/* shaders/activation-swiglu.glsl:40-49 */
static inline float sigmoid_split(float v) {
    if (v >= 0.0f) return 1.0f / (1.0f + expf(-v));
    float e = expf(v);
    return e / (1.0f + e);
}

/* y[m,n] = epi(sum_k x[m,k]*W[n,k] + b[n]):  shaders/fnn-linear.glsl:33-58,
 * shaders/fused-linear-gelu.glsl:65-93, shaders/fused-linear-silu.glsl:50-78;
 * with N = 3*H*D and packed weights also shaders/fused-qkv-projection.glsl:48-74. */
/* shaders/fused-linear-roswish.glsl:46-58 */
static inline float roswish_shader(float x, float alpha, float beta) {
    return (x + alpha) * sigmoid_split(beta * x) - 0.5f * alpha;
}

/* shaders/fused-geglu.glsl:44-49: tanh GELU without the +-50 clamp rule */
static inline float gelu_plain(float x) {
    return 0.5f * x * (1.0f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x)));
}

/* epi 0..2 as above; 3 = shaders/fused-linear-relu.glsl:40-68 (max(0,s)); 4 = shaders/fused-linear-gcu.glsl:43-75
 * (s*cos(s)); 5 = shaders/fused-linear-roswish.glsl:60-90 */
void orc_linear_act(const float* x, const float* W, const float* b, float* y, int64_t M, int64_t K, int64_t N, int epi,
                    float alpha, float beta) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            float sum = 0.0f;
            for (int64_t k = 0; k < K; ++k) sum += x[m * K + k] * W[n * K + k];
            if (b) sum += b[n];
            if (epi == EPI_GELU) sum = gelu_shader(sum);
            else if (epi == EPI_SILU) sum = silu_clamped(sum);
            else if (epi == EPI_RELU) sum = sum > 0.0f ? sum : 0.0f;
            else if (epi == EPI_GCU) sum = sum * cosf(sum);
            else if (epi == EPI_ROSWISH) sum = roswish_shader(sum, alpha, beta);
            y[m * N + n] = sum;
        }
    }
}

void orc_linear(const float* x, const float* W, const float* b, float* y, int64_t M, int64_t K, int64_t N, int epi) {
    orc_linear_act(x, W, b, y, M, K, N, epi, 1.0f, 1.0f);
}

/* C = A.B, B (K,N): shaders/gemm_mnk.glsl:35-88 (ascending k over 16-wide tiles = ascending k) */
void orc_gemm_nn(const float* A, const float* B, float* C, int64_t M, int64_t K, int64_t N) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float sum = 0.0f;
            for (int64_t k = 0; k < K; ++k) sum += A[m * K + k] * B[k * N + n];
            C[m * N + n] = sum;
        }
}

/* shaders/fused-swiglu.glsl:48-79: gate*silu(up); biases only when both given
 * (backend/_glu_append.py:68).  gate_c/up_c (optional) receive the pre-activations
 * (backend/_glu_append.py:120-127). */
void orc_fused_glu(const float* x, const float* Wg, const float* Wu, const float* bg, const float* bu,
                   float* out, float* gate_c, float* up_c, int64_t M, int64_t K, int64_t N, int act);

void orc_fused_swiglu(const float* x, const float* Wg, const float* Wu, const float* bg, const float* bu,
                      float* out, float* gate_c, float* up_c, int64_t M, int64_t K, int64_t N) {
    orc_fused_glu(x, Wg, Wu, bg, bu, out, gate_c, up_c, M, K, N, EPI_SILU);
}

/* act 2: the SwiGLU above; act 3: shaders/fused-reglu.glsl:42-75 (gate*max(0,up), backend/_glu_append.py:131-222);
 * act 1: shaders/fused-geglu.glsl:43-82 (gate*gelu(up), backend/_glu_append.py:224-315) */
void orc_fused_glu(const float* x, const float* Wg, const float* Wu, const float* bg, const float* bu,
                   float* out, float* gate_c, float* up_c, int64_t M, int64_t K, int64_t N, int act) {
    int has_bias = bg && bu;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            float gate = 0.0f, up = 0.0f;
            for (int64_t k = 0; k < K; ++k) gate += x[m * K + k] * Wg[n * K + k];
            if (has_bias) gate += bg[n];
            for (int64_t k = 0; k < K; ++k) up += x[m * K + k] * Wu[n * K + k];
            if (has_bias) up += bu[n];
            if (gate_c) gate_c[m * N + n] = gate;
            if (up_c) up_c[m * N + n] = up;
            out[m * N + n] = act == EPI_RELU ? gate * (up > 0.0f ? up : 0.0f) : act == EPI_GELU ? gate * gelu_plain(up) : gate * silu_plain(up);
        }
}

/* shaders/fnn-layernorm.glsl:44-103: mean pass, variance pass (biased), normalise pass.
 * res (optional) is added first: shaders/fnn-residual.glsl:25-34 then layernorm, which is
 * how the encoder chains them (utils/vulkan_sentence_transformer.py:1004,1026). */
void orc_layernorm(const float* x, const float* res, const float* gamma, const float* beta, float* y,
                   int64_t rows, int64_t F, float eps) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float* xr = x + r * F;
        const float* rr = res ? res + r * F : NULL;
        float sum = 0.0f;
        for (int64_t f = 0; f < F; ++f) sum += rr ? xr[f] + rr[f] : xr[f];
        float mean = sum / (float)F;
        float sq = 0.0f;
        for (int64_t f = 0; f < F; ++f) {
            float d = (rr ? xr[f] + rr[f] : xr[f]) - mean;
            sq += d * d;
        }
        float var = sq / (float)F;
        float sd = sqrtf(var + eps);
        for (int64_t f = 0; f < F; ++f) {
            float v = rr ? xr[f] + rr[f] : xr[f];
            y[r * F + f] = gamma[f] * ((v - mean) / sd) + beta[f];
        }
    }
}

/* shaders/fnn-residual.glsl:25-34 */
void orc_residual(const float* a, const float* b, float* out, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
}

/* shaders/activation-gelu.glsl:23-53 */
void orc_gelu(const float* x, float* y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = gelu_shader(x[i]);
}

/* backend/fnn.py:344-391 (activation_silu): x*sigmoid(x) */
void orc_silu(const float* x, float* y, int64_t n) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = x[i] * sigmoid_split(x[i]);
}

/* shaders/activation-swiglu.glsl:21-52: (rows,2h) -> (rows,h), x1*(x2*sigmoid(x2)) */
void orc_swiglu_act(const float* x, float* y, int64_t rows, int64_t h) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t p = 0; p < h; ++p) {
            float x1 = x[r * 2 * h + p], x2 = x[r * 2 * h + h + p];
            y[r * h + p] = x1 * (x2 * sigmoid_split(x2));
        }
}

/* inverse frequency of pair p: the fp32 value of pow(base, fe) with fe = -2*float(p)/float(D)
 * formed in fp32 (shaders/rope.glsl:115-116, shaders/flash-attention2-rope.glsl:75-78); the
 * power itself is taken in double and rounded once, i.e. the exact value the shader's pow()
 * approximates. */
static inline float inv_freq(int p, int D, float base) {
    float fe = (-2.0f * (float)p) / (float)D;
    return (float)pow((double)base, (double)fe);
}

/* style 2 (half):        shaders/rope.glsl:74-125, backend/attention.py:795-835
 *   theta = (pos/scaling)*freq ; y[d] = x[d]cos - x[d+D/2]sin ; y[d+D/2] = x[d+D/2]cos + x[d]sin
 * style 1 (interleaved): shaders/flash-attention2-rope.glsl:75-90,122-137
 *   theta = (pos*freq)/scaling ; (y0,y1) = (x0 cos - x1 sin, x0 sin + x1 cos) on (2p,2p+1) */
void orc_rope(const float* x, const int32_t* pos_ids, float* y, int64_t B, int64_t S, int64_t H, int64_t D,
              int style, float base, float scaling) {
    int half = (int)(D / 2);
#pragma omp parallel for schedule(static)
    for (int64_t bs = 0; bs < B * S; ++bs) {
        float pos = pos_ids ? (float)pos_ids[bs] : (float)(bs % S);
        for (int64_t h = 0; h < H; ++h) {
            const float* xv = x + (bs * H + h) * D;
            float* yv = y + (bs * H + h) * D;
            for (int p = 0; p < half; ++p) {
                float fr = inv_freq(p, (int)D, base);
                float theta = style == 2 ? (pos / scaling) * fr : (pos * fr) / scaling;
                float cs = cosf(theta), sn = sinf(theta);
                int i0 = style == 2 ? p : 2 * p, i1 = style == 2 ? p + half : 2 * p + 1;
                float a = xv[i0], b = xv[i1];
                yv[i0] = a * cs - b * sn;
                yv[i1] = b * cs + a * sn;
            }
        }
    }
}

/* Attention contract, evaluated unfused in fp32 (scores -> softmax -> P.V):
 *   docstring backend/attention.py:374-395; layout (B,S,H,D) :403-410, :573-575;
 *   score = dot*scale (shaders/flash-attention2.glsl:131-147), + (mask-1)*1e9 (:150-154);
 *   running max starts at -1e10 (:95), final divide by max(sum,1e-10) (:214);
 *   causal: keys k_pos > q_pos excluded (shaders/attention-mask.glsl:42-46);
 *   the same closed form as the reference's CPU attention, nn/modules.py:1421-1456 and
 *   utils/vulkan_sentence_transformer.py:1069-1107.
 * The racy two-pass shader body itself (flash-attention2.glsl:161-196) is NOT restated: it
 * has no defined output.
 * rope_style 0 none / 1 interleaved / 2 half: Q,K rotated first (V never,
 * shaders/flash-attention2-rope.glsl:230-236). */
void orc_attention(const float* Q, const float* K, const float* V, const float* mask, float* O,
                   int64_t B, int64_t S, int64_t H, int64_t D, float scale, int causal,
                   int rope_style, float base, float scaling) {
    const float* q = Q;
    const float* k = K;
    float* qr = NULL;
    float* kr = NULL;
    if (rope_style) {
        size_t n = (size_t)(B * S * H * D);
        qr = (float*)malloc(n * sizeof(float));
        kr = (float*)malloc(n * sizeof(float));
        orc_rope(Q, NULL, qr, B, S, H, D, rope_style, base, scaling);
        orc_rope(K, NULL, kr, B, S, H, D, rope_style, base, scaling);
        q = qr; k = kr;
    }
#pragma omp parallel
    {
        float* sc = (float*)malloc((size_t)S * sizeof(float));
#pragma omp for schedule(dynamic, 4) collapse(2)
        for (int64_t bh = 0; bh < B * H; ++bh)
            for (int64_t i = 0; i < S; ++i) {
                int64_t b = bh / H, h = bh % H;
                const float* qv = q + ((b * S + i) * H + h) * D;
                int64_t jend = causal ? i + 1 : S;
                float m = -1e10f;
                for (int64_t j = 0; j < jend; ++j) {
                    const float* kv = k + ((b * S + j) * H + h) * D;
                    float s = 0.0f;
                    for (int64_t d = 0; d < D; ++d) s += qv[d] * kv[d];
                    s *= scale;
                    if (mask) s += (mask[b * S + j] - 1.0f) * 1e9f;
                    sc[j] = s;
                    if (s > m) m = s;
                }
                float l = 0.0f;
                for (int64_t j = 0; j < jend; ++j) { sc[j] = expf(sc[j] - m); l += sc[j]; }
                float inv = 1.0f / (l > 1e-10f ? l : 1e-10f);
                float* ov = O + ((b * S + i) * H + h) * D;
                for (int64_t d = 0; d < D; ++d) {
                    float acc = 0.0f;
                    for (int64_t j = 0; j < jend; ++j) acc += sc[j] * V[((b * S + j) * H + h) * D + d];
                    ov[d] = acc * inv;
                }
            }
        free(sc);
    }
    free(qr);
    free(kr);
}

/* x[b,s,:] = tok[ids] + type[0] + pos[s]: utils/vulkan_sentence_transformer.py:563-707 */
void orc_embed(const int32_t* ids, const float* tok, const float* pos, const float* typ, float* x,
               int64_t B, int64_t S, int64_t F) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < B * S; ++r)
        for (int64_t f = 0; f < F; ++f) x[r * F + f] = tok[(int64_t)ids[r] * F + f] + typ[f] + pos[(r % S) * F + f];
}

/* masked mean pool (+ optional L2 normalise): utils/vulkan_sentence_transformer.py:1177-1201 */
void orc_mean_pool(const float* x, const float* mask, float* out, int64_t B, int64_t S, int64_t F, int l2) {
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; ++b) {
        float cnt = 0.0f;
        for (int64_t s = 0; s < S; ++s) cnt += mask ? mask[b * S + s] : 1.0f;
        if (cnt < 1e-9f) cnt = 1e-9f;
        float nrm = 0.0f;
        for (int64_t f = 0; f < F; ++f) {
            float acc = 0.0f;
            for (int64_t s = 0; s < S; ++s) acc += (mask ? mask[b * S + s] : 1.0f) * x[(b * S + s) * F + f];
            out[b * F + f] = acc / cnt;
            nrm += out[b * F + f] * out[b * F + f];
        }
        if (l2) {
            nrm = sqrtf(nrm);
            if (nrm < 1e-12f) nrm = 1e-12f;
            for (int64_t f = 0; f < F; ++f) out[b * F + f] /= nrm;
        }
    }
}

/* One post-LN BERT layer, utils/vulkan_sentence_transformer.py:972-1035: three linears on the
 * rows of the packed QKV weight (= fused-qkv-projection.glsl), attention with key mask,
 * out-proj, LN(residual, eps), FFN with tanh-GELU, LN(residual, eps).  x is updated in place.
 * scratch must hold M*(3d + d + d + dff) floats. */
void orc_bert_layer(float* x, const float* mask, int64_t B, int64_t S, int64_t H, int64_t D, int64_t dff,
                    const float* w_qkv, const float* b_qkv, const float* w_o, const float* b_o,
                    const float* ln1_g, const float* ln1_b, const float* w_ff1, const float* b_ff1,
                    const float* w_ff2, const float* b_ff2, const float* ln2_g, const float* ln2_b,
                    float eps, float* scratch) {
    int64_t M = B * S, d = H * D;
    float* qkv = scratch;
    float* q = qkv + M * 3 * d;      /* contiguous copies of Q,K,V then reused */
    float* attn = q;                 /* overwritten after the split buffers are consumed */
    float* proj = q + M * d;
    float* ff = proj + M * d;
    orc_linear(x, w_qkv, b_qkv, qkv, M, d, 3 * d, EPI_NONE);
    /* split the packed (M,3d) rows into contiguous (B,S,H,D) tensors; ff is large enough to
     * hold them temporarily when dff >= 3d, else allocate */
    float* split = (float*)malloc((size_t)(3 * M * d) * sizeof(float));
    for (int64_t m = 0; m < M; ++m)
        for (int t = 0; t < 3; ++t) memcpy(split + (size_t)t * M * d + m * d, qkv + m * 3 * d + t * d, (size_t)d * sizeof(float));
    orc_attention(split, split + M * d, split + 2 * M * d, mask, attn, B, S, H, D, 1.0f / sqrtf((float)D), 0, 0, 10000.0f, 1.0f);
    free(split);
    orc_linear(attn, w_o, b_o, proj, M, d, d, EPI_NONE);
    orc_layernorm(x, proj, ln1_g, ln1_b, x, M, d, eps);
    orc_linear(x, w_ff1, b_ff1, ff, M, d, dff, EPI_GELU);
    orc_linear(ff, w_ff2, b_ff2, proj, M, dff, d, EPI_NONE);
    orc_layernorm(x, proj, ln2_g, ln2_b, x, M, d, eps);
}

int orc_num_threads(void) {
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}
