/*
 * grilly_hip.h -- C ABI of libgrilly_hip.so: the gfx950 (MI355X) implementation of
 * grilly's transformer-forward hot path.
 *
 * Every launcher works on DEVICE pointers obtained from grl_malloc (or any hipMalloc'd
 * memory), enqueues on the context's HIP stream and returns immediately; grl_sync()
 * waits.  All functions return 0 on success or a negative grl_status; the message of
 * the last failure on the calling thread is returned by grl_last_error().  There is no
 * CPU fallback anywhere behind this interface.
 *
 * Each entry point names the reference (Grillcheese-AI/grilly) interface it stands in
 * for as  file:line .  The reference drives GLSL compute shaders through Vulkan from
 * Python; a binding for it is therefore a ctypes stub (see grilly_amd/_lib.py).
 *
 * Conventions shared by all launchers
 *   - tensors are dense, row-major, C-contiguous; sizes are element counts
 *   - grl_dtype selects the storage type of activations/weights: GRL_F32 or GRL_BF16
 *     (bfloat16, round-to-nearest-even); accumulation and statistics are always fp32
 *   - bias / gamma / beta vectors are always fp32
 *   - "weights (N,K)" means the reference's (out_features, in_features) layout
 */
#ifndef GRILLY_HIP_H
#define GRILLY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct grl_ctx grl_ctx;

typedef enum grl_status {
    GRL_OK = 0,
    GRL_ERR_ARG = -1,         /* null pointer, bad enum, non-positive size */
    GRL_ERR_SHAPE = -2,       /* shape the kernels do not cover (message says which) */
    GRL_ERR_HIP = -3,         /* a HIP runtime call failed */
    GRL_ERR_OOM = -4          /* device allocation failed */
} grl_status;

typedef enum grl_dtype { GRL_F32 = 0, GRL_BF16 = 1 } grl_dtype;

/* epilogue applied to (x.W^T + bias) inside the GEMM kernel, on the fp32 accumulator */
typedef enum grl_epilogue {
    GRL_EPI_NONE = 0,
    GRL_EPI_GELU = 1,   /* tanh GELU with the +-50 clamp rule of shaders/fused-linear-gelu.glsl:45-63 */
    GRL_EPI_SILU = 2,   /* s/(1+exp(-clamp(s,-88,88))), shaders/fused-linear-silu.glsl:43-48 */
    GRL_EPI_RELU = 3,   /* max(0,s), shaders/fused-linear-relu.glsl:63 */
    GRL_EPI_GCU = 4,    /* s*cos(s), shaders/fused-linear-gcu.glsl:44-46 */
    GRL_EPI_ROSWISH = 5 /* (s+alpha)*sigmoid(beta*s) - alpha/2, shaders/fused-linear-roswish.glsl:46-58 */
} grl_epilogue;

typedef enum grl_rope_style { GRL_ROPE_NONE = 0, GRL_ROPE_INTERLEAVED = 1, GRL_ROPE_HALF = 2 } grl_rope_style;

typedef struct grl_devinfo {
    char name[128];
    char arch[64];
    int32_t compute_units;
    int32_t clock_khz;
    int32_t lds_bytes_per_block;
    int32_t wavefront;
    int64_t hbm_bytes;
} grl_devinfo;

typedef struct grl_pool_stats {
    int64_t allocations;      /* hipMalloc calls made by the pool */
    int64_t hits;             /* grl_malloc calls served from a cached block */
    int64_t misses;           /* grl_malloc calls that had to allocate */
    int64_t bytes_in_use;
    int64_t bytes_cached;
    int64_t bytes_peak;
} grl_pool_stats;

/* ---- context / runtime --------------------------------------------------------
 * Replaces VulkanCore (backend/core.py:17-166 create, :423-439 cleanup) and
 * VulkanPipelines (backend/pipelines.py:97-130): one context = one device + one stream. */
grl_ctx*    grl_create(int device);
void        grl_destroy(grl_ctx* ctx);
const char* grl_last_error(void);
int         grl_device_info(grl_ctx* ctx, grl_devinfo* out);
/* the hipStream_t of the context, for callers that record their own events on it */
void*       grl_stream(grl_ctx* ctx);

/* Device buffers from a power-of-two bucketed caching pool.
 * Replaces VulkanCore._create_buffer (backend/core.py:304-335) and
 * BufferPool.acquire/release/get_stats (backend/buffer_pool.py:534-579, 627-640). */
void* grl_malloc(grl_ctx* ctx, size_t bytes);
int   grl_free(grl_ctx* ctx, void* ptr);
int   grl_pool_get_stats(grl_ctx* ctx, grl_pool_stats* out);
int   grl_pool_trim(grl_ctx* ctx);     /* return cached blocks to the driver */

/* Host <-> device copies, replacing _upload_buffer / _download_buffer (backend/core.py:345-360).  grl_h2d returns when
 * the host buffer has been consumed (the caller may reuse it at once); the transfer itself is ordered on the context
 * stream like a kernel launch, so later calls on this context see the data and grl_sync / grl_d2h wait for it.  A
 * consumer on another stream or context must grl_sync first.  grl_d2h blocks until the data is in the host buffer.
 * grl_sync replaces vkQueueWaitIdle (backend/core.py:418). */
int grl_h2d(grl_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes);
int grl_d2h(grl_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes);
int grl_d2d(grl_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes);
int grl_memset(grl_ctx* ctx, void* dst_dev, int byte, size_t bytes);
int grl_sync(grl_ctx* ctx);

/* HIP-event stopwatch on the context stream (there is no counterpart in the reference,
 * which times whole numpy->numpy calls with time.perf_counter).  A context holds one event pair: one timing
 * at a time; calls from several threads are serialised but share the pair, so concurrent timings overwrite
 * each other's start. */
int grl_timer_start(grl_ctx* ctx);
int grl_timer_stop(grl_ctx* ctx, float* elapsed_ms);   /* synchronises */
/* Lap events on the context stream (measurement aid, no counterpart in the reference): grl_timer_lap records event
 * `index` (0..255) behind whatever is enqueued so far, without waiting; grl_timer_lap_ms waits for event `to` and
 * returns the time between two recorded events.  A lap before and after each launch of a back-to-back sequence gives
 * per-launch durations (for medians) without host synchronisations between the launches. */
int grl_timer_lap(grl_ctx* ctx, int index);
int grl_timer_lap_ms(grl_ctx* ctx, int from, int to, float* elapsed_ms);
/* Lap trace: between grl_timer_lap_trace(ctx, first, NULL) and grl_timer_lap_trace(ctx, -1, &next) the encoder-layer entry
 * points (grl_bert_layer_fwd, grl_bert_layer_fwd_fused) record a lap at entry and after each kernel they launch, with
 * indices first+1, first+2, ... (lap `first` is recorded by the call that turns the trace on; marks beyond index 255 are
 * dropped).  `next` receives the index the next mark would have used, or -1 when no trace was on.  For timing the
 * launches inside a forward; one trace per context at a time. */
int grl_timer_lap_trace(grl_ctx* ctx, int first, int* next);
/* Matrix-core ceiling probe (measurement aid, no counterpart in the reference): every CU runs eight waves that issue
 * nothing but MFMAs on register-resident operands (kind 0: v_mfma_f32_32x32x16_bf16 in the GEMM kernels' operand order,
 * kind 1: v_mfma_f32_16x16x32_bf16; kinds 2, 3, 4: the 32x32x16 loop with one operand held for four instructions in a
 * row, with a serpentine walk, and with the same operand pair for every instruction)
 * for `iters` loop iterations, after one untimed warm-up launch.  `operands` points to 64 KiB of device memory whose
 * bits become the operand fragments (NULL: all-zero operands).  Returns the launch duration and the FLOPs it
 * executed: the rate the matrix cores sustain under the board's power limit for those operand bits. */
int grl_mfma_probe(grl_ctx* ctx, int kind, const void* operands, int iters, float* elapsed_ms, double* flops);
/* Shader-clock probe, a measurement aid with no counterpart in the reference: _begin starts a one-wave kernel on a
 * second stream of the context that runs for `millis` of wall time beside whatever the caller enqueues next; _end
 * waits for it and returns the average shader clock in GHz over that time (shader cycles over 100 MHz reference
 * ticks).  Peak MFMA rates are quoted at the nominal clock; under a power limit the GPU runs a loaded kernel below
 * it, and this is how the benchmark reads the clock its timed launches really ran at. */
int grl_clock_probe_begin(grl_ctx* ctx, float millis);
int grl_clock_probe_end(grl_ctx* ctx, float* ghz);

/* fp32 <-> bf16 conversion on the device (RNE).  No reference counterpart: the
 * reference is fp32 only. */
int grl_cast(grl_ctx* ctx, int src_dtype, int dst_dtype, int64_t n, const void* src, void* dst);

/* ---- GEMM family ---------------------------------------------------------------
 * C[m,n] = epi( sum_k A[m,k] * W[n,k] + bias[n] )      A (M,K), W (N,K), C (M,N)
 * Replaces VulkanFNN.linear (backend/fnn.py:1394-1496, shaders/fnn-linear.glsl:33-58),
 * VulkanFNN.fused_linear_gelu (backend/fnn.py:2022-2123, shaders/fused-linear-gelu.glsl:42-93),
 * VulkanFNN.fused_linear_silu (backend/fnn.py:2214-2303, shaders/fused-linear-silu.glsl:42-78)
 * and, with N = 3*H*D and packed [Wq;Wk;Wv], shaders/fused-qkv-projection.glsl:48-74.
 * in_dtype is the type of A and W, out_dtype the type of C; bias may be NULL. */
int grl_gemm_nt(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                const void* A, const void* W, const float* bias, void* C, int epilogue);
/* Which kernel grl_gemm_nt and its siblings launch for a problem whose operands are 16-byte aligned, as pure host
 * arithmetic (no device needed; no counterpart in the reference): 1 / 2 register-staged 256 x 256 / 128 x 128 tiles,
 * 3 / 4 direct-to-LDS 256 x 256 (persistent) / 128 x 128 tiles, 5 register-staged 64 x 64 tiles.  `dual` selects the
 * gated two-weight kernels, `compute_units` the CU count of the device (256 on MI355X).  Negative on bad arguments. */
int grl_gemm_plan(int dtype, int64_t M, int64_t N, int64_t K, int dual, int compute_units);

/* C = A.B with B (K,N) row-major.  Replaces VulkanFNN.gemm (backend/fnn.py:104-166,
 * shaders/gemm_mnk.glsl:35-88).  workspace must hold K*N elements of in_dtype (the
 * kernel transposes B once); pass NULL to let the context allocate it from its pool. */
int grl_gemm_nn(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                const void* A, const void* B, void* C, void* workspace);

/* C = A.B with B (K,N) row-major, like grl_gemm_nn, but allocating nothing: no hipMalloc / hipFree, no pool
 * request.  No counterpart in the reference; it is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid device allocation.  The transposed copy of B goes into
 * a static device array of grl_gemm_nn_noalloc_max_bytes() = 32 MiB that every GPU the library runs on holds
 * until the process ends (its address is looked up in grl_create); K*N*sizeof(in_dtype) beyond that returns
 * GRL_ERR_SHAPE.  All calls on one GPU share the array.  Host threads that call it on ONE context are safe: a lock
 * keeps each call's two launches (transpose into the array, GEMM out of it) adjacent on the context's stream,
 * which then orders the calls.  Calls on two contexts of the same GPU run on two streams and race on the
 * array: the caller must not overlap them.  Small products with a long K, whose K loop grl_gemm_nn shares out over
 * several workgroups through a pool buffer, keep their K loop whole here: results agree with grl_gemm_nn to the
 * last bits of the sums, not bit for bit. */
int grl_gemm_nn_noalloc(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                        const void* A, const void* B, void* C);
int64_t grl_gemm_nn_noalloc_max_bytes(void);

/* grl_gemm_nt with every epilogue of the reference's fused-linear family: additionally
 * GRL_EPI_RELU (VulkanFNN.fused_linear_relu, backend/fnn.py:2125-2212, shaders/fused-linear-relu.glsl:40-68),
 * GRL_EPI_GCU (fused_linear_gcu, backend/fnn.py:2307-2383, shaders/fused-linear-gcu.glsl:43-75) and
 * GRL_EPI_ROSWISH (fused_linear_roswish, backend/fnn.py:2385-2470, shaders/fused-linear-roswish.glsl:44-90)
 * with its two parameters; alpha and beta are ignored by the other epilogues. */
int grl_gemm_nt_act(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                    const void* A, const void* W, const float* bias, void* C, int epilogue,
                    float alpha, float beta);

/* C = A.W^T + bias + residual, the residual (M,N) of the output type; C may be the residual buffer itself.
 * One pass for what the reference does as a linear followed by VulkanFNN.residual
 * (backend/fnn.py:1950-2014, shaders/fnn-residual.glsl:25-34; the pair as the encoder recipes use it,
 * utils/vulkan_sentence_transformer.py:893, 945 and, in front of the LayerNorm, :1001-1004, :1023-1026). */
int grl_gemm_nt_res(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                    const void* A, const void* W, const float* bias, const void* residual, void* C);

/* out[m,n] = (x.Wg^T + bg)[m,n] * act((x.Wu^T + bu)[m,n]) with act = GRL_EPI_SILU (SwiGLU, below),
 * GRL_EPI_RELU (fused_reglu, backend/_glu_append.py:131-222, shaders/fused-reglu.glsl:42-75) or
 * GRL_EPI_GELU (fused_geglu, backend/_glu_append.py:224-315, shaders/fused-geglu.glsl:43-82: tanh GELU
 * without the clamp rule).  Biases and caches as for grl_swiglu_nt. */
int grl_glu_nt(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
               const void* x, const void* W_gate, const void* W_up,
               const float* b_gate, const float* b_up, void* out,
               float* gate_cache, float* up_cache, int activation);

/* out[m,n] = (x.Wg^T + bg)[m,n] * silu((x.Wu^T + bu)[m,n]),  silu(u) = u/(1+exp(-u)).
 * Replaces fused_swiglu (backend/_glu_append.py:8-129, shaders/fused-swiglu.glsl:43-79).
 * Biases are applied only when both are given, as in the reference (_glu_append.py:68).
 * gate_cache / up_cache (fp32, (M,N)) receive the pre-activations when non-NULL. */
int grl_swiglu_nt(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K,
                  const void* x, const void* W_gate, const void* W_up,
                  const float* b_gate, const float* b_up, void* out,
                  float* gate_cache, float* up_cache);

/* ---- attention -------------------------------------------------------------------
 * O[b,i,h,:] = sum_j softmax_j( scale*<Q'[b,i,h],K'[b,j,h]> + (mask[b,j]-1)*1e9 ) V[b,j,h,:]
 * with Q',K' optionally rotated (RoPE) and, if causal, keys j>i excluded.
 * Layout of Q,K,V,O: (B,S,H,D).  mask: fp32 (B,S), 1 keep / 0 drop, or NULL; any other value enters through the
 * same bias (0.5 still drops, 1+2^-23 adds 119 to the key's scores), and a row whose visible keys are all dropped
 * comes out as the mean of those keys' values (every score is rounded to the same -1e9, as in the shader).
 * Replaces VulkanAttention.flash_attention2 (backend/attention.py:361-597; contract in
 * its docstring :374-395; constants of shaders/flash-attention2.glsl:95,152,214) and
 * shaders/flash-attention2-rope.glsl:73-148 (interleaved pairs, theta =
 * pos*base^(-2p/D)/scaling); causal rule of shaders/attention-mask.glsl:42-46.
 * Any head dim D from 1 to 1024 (the reference reshapes with whatever head_dim it is given,
 * backend/attention.py:403-410): 32, 64 and 128 with 16-byte granular operands run the MFMA kernels directly,
 * other head dims up to 128 (or operands that are not 16-byte granular) run them on zero-padded copies taken
 * from the pool, larger ones a one-wave-per-query kernel; RoPE needs an even D up to 128.
 * GRL_ROPE_HALF uses the (d, d+D/2) pairing of shaders/rope.glsl:74-125 and, on the direct path, a workspace of
 * 2*B*S*H*D elements (NULL = pool).  The cos/sin table of the rotation is built once per (D, base, scaling,
 * pairing) and kept on the context. */
int grl_fa2_fwd(grl_ctx* ctx, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                const void* Q, const void* K, const void* V, const float* mask, void* O,
                float scale, int causal, int rope, float rope_base, float rope_scaling,
                void* workspace);

/* Same as grl_fa2_fwd with explicit position strides (elements between consecutive sequence
 * positions of one batch entry), so Q, K and V can be the three column blocks of the packed
 * (B*S, 3*H*D) output of the fused QKV projection (shaders/fused-qkv-projection.glsl:58-70)
 * without a split copy.  Both RoPE pairings are offered; rotate-half takes its workspace (fp32: rotated copies of Q and
 * K, bf16: the rotated K) from the pool.  Strides of at least H*D elements; operands that are not 16-byte granular
 * (base addresses or strides) run on dense copies from the pool. */
int grl_fa2_fwd_strided(grl_ctx* ctx, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                        const void* Q, const void* K, const void* V, const float* mask, void* O,
                        int64_t q_stride, int64_t k_stride, int64_t v_stride, int64_t o_stride,
                        float scale, int causal, int rope, float rope_base, float rope_scaling);

/* y = rotate(x) for x (B,S,H,D); position_ids int32 (B,S) or NULL for 0..S-1.
 * Replaces VulkanAttention.apply_rope (backend/attention.py:599-676, _rope_cpu :795-835,
 * shaders/rope.glsl:74-125) for style GRL_ROPE_HALF; GRL_ROPE_INTERLEAVED follows
 * shaders/flash-attention2-rope.glsl:84-90,122-137. */
int grl_rope(grl_ctx* ctx, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
             const void* x, const int32_t* position_ids, void* y,
             int style, float rope_base, float rope_scaling);

/* ---- bandwidth-bound row / element kernels ------------------------------------------
 * y = gamma*(t-mean)/sqrt(var+eps)+beta per row of F features, t = x (+ residual if given),
 * biased variance, two-pass statistics in fp32.
 * Replaces VulkanFNN.layernorm (backend/fnn.py:1285-1389, shaders/fnn-layernorm.glsl:44-103);
 * the optional residual folds VulkanFNN.residual (backend/fnn.py:1950-2014) into the same
 * pass, which is how the encoder uses the pair (utils/vulkan_sentence_transformer.py:1004,1026).
 * In-place use is allowed: y may be x or residual (each element is read and written by the same lane).
 * x and residual may also be the same buffer. */
int grl_layernorm(grl_ctx* ctx, int dtype, int64_t rows, int64_t F, const void* x,
                  const void* residual, const float* gamma, const float* beta, float eps, void* y);

/* ---- Linear(LayerNorm(x)) without forming the normalised rows --------------------------
 * Replaces the shader shaders/fused-layernorm-linear.glsl:67-128 (per-row mean / variance, then the GEMM on the
 * normalised row inside one dispatch).  Here the normalisation moves into the GEMM epilogue:
 *     sum_k LN(x)[m,k] W[n,k] = rstd_m * (sum_k x[m,k] Ws[n,k] - mean_m * c[n]) + b'[n]
 * with Ws[n,k] = gamma[k] W[n,k], c[n] = sum_k Ws[n,k], b'[n] = bias[n] + sum_k beta[k] W[n,k].
 * grl_ln_fold builds Ws (storage type), c and b' once per weight; grl_ln_stats writes {rstd, rstd*mean} per row
 * (one read of x, 8 bytes out per row); grl_ln_gemm_nt runs grl_ln_stats into `stats` (2*M floats, 16-byte aligned,
 * caller-owned) and then the GEMM on the raw x.  grl_ln_glu_nt is the gated form act(up)*gate of grl_glu_nt on
 * LN(x), both weights folded with the same gamma / beta.  Statistics as grl_layernorm (biased variance, two passes). */
int grl_ln_fold(grl_ctx* ctx, int dtype, int64_t N, int64_t K, const void* W, const float* gamma, const float* beta,
                const float* bias /* (N) or NULL */, void* W_scaled, float* colsum, float* bias_folded);
int grl_ln_stats(grl_ctx* ctx, int dtype, int64_t rows, int64_t F, const void* x, float eps, float* stats);
int grl_ln_gemm_nt(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                   const void* W_scaled, const float* colsum, const float* bias_folded /* (N) or NULL */, float eps,
                   float* stats, void* out);
int grl_ln_glu_nt(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                  const void* Wg_scaled, const void* Wu_scaled, const float* colsum_gate, const float* colsum_up,
                  const float* bias_gate_folded, const float* bias_up_folded, float eps, float* stats,
                  void* out, int activation);
/* grl_ln_glu_nt with the row statistics given ({1/sd, mean/sd} per row of x, e.g. written by grl_gemm_nt_resln when it
 * produced x): no pass over x in front of the GEMM. */
int grl_ln_glu_nt_stats(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                        const void* Wg_scaled, const void* Wu_scaled, const float* colsum_gate, const float* colsum_up,
                        const float* bias_gate_folded, const float* bias_up_folded, const float* stats,
                        void* out, int activation);
/* grl_ln_gemm_nt with the row statistics given ({1/sd, mean/sd} per row of x, as grl_ln_stats or grl_gemm_nt_resln
 * write them) and a choice of epilogue: GRL_EPI_NONE or GRL_EPI_GELU (out = gelu(LN(x).W^T + b), the first half of the
 * feed-forward block behind a LayerNorm, utils/vulkan_sentence_transformer.py:1004-1012). */
int grl_ln_gemm_nt_stats(grl_ctx* ctx, int in_dtype, int out_dtype, int64_t M, int64_t N, int64_t K, const void* x,
                         const void* W_scaled, const float* colsum, const float* bias_folded, const float* stats,
                         void* out, int epilogue);
/* C = A.W^T + bias + LayerNorm(R; r_gamma, r_beta), and stats_out = {1/sd, mean/sd} of every row of C (with eps).
 * The post-LN sub-block "x + f(x)" where x is itself the output of a LayerNorm that was never written out: R holds the
 * raw rows in front of that LayerNorm, r_stats their {1/sd, mean/sd}; the GEMM epilogue re-forms x from them, adds it,
 * and reduces each output row's sum and sum of squares per column tile, which a small merge kernel turns into the
 * statistics the NEXT LayerNorm-folded GEMM (grl_ln_gemm_nt_stats) reads.  Together the two entry points run the
 * reference's linear -> add -> layer_norm -> linear chain (utils/vulkan_sentence_transformer.py:996-1026) without a
 * LayerNorm pass over HBM.  C may be R (in place).  A, W, R, C of `dtype`; only for problems the direct-to-LDS kernels
 * take: K a multiple of 64 (bf16) / 32 (fp32), N a multiple of 8 / 4, 16-byte aligned pointers, else GRL_ERR_SHAPE.
 * workspace: grl_gemm_nt_resln_workspace(M, N) bytes, 16-byte aligned. */
int64_t grl_gemm_nt_resln_workspace(int64_t M, int64_t N);
int grl_gemm_nt_resln(grl_ctx* ctx, int dtype, int64_t M, int64_t N, int64_t K, const void* A, const void* W,
                      const float* bias, const void* R, const float* r_stats, const float* r_gamma, const float* r_beta,
                      void* C, float eps, float* stats_out, void* workspace);

/* out = a + b.  Replaces VulkanFNN.residual (shaders/fnn-residual.glsl:25-34).
 * grl_add, grl_gelu, grl_silu and grl_relu may run in place (out == a, out == b, y == x).
 * Every other entry point of this header needs its outputs distinct from its inputs unless its own
 * comment says otherwise (grl_gemm_nt_res, grl_gemm_nt_resln: C may be the residual; grl_bert_layer_fwd, grl_bert_layer_fwd_fused: x / r is
 * updated in place). */
int grl_add(grl_ctx* ctx, int dtype, int64_t n, const void* a, const void* b, void* out);
/* Replaces VulkanFNN.activation_gelu (backend/fnn.py:285-342, shaders/activation-gelu.glsl:23-53). */
int grl_gelu(grl_ctx* ctx, int dtype, int64_t n, const void* x, void* y);
/* Replaces VulkanFNN.activation_silu (backend/fnn.py:344-391): x*sigmoid(x). */
int grl_silu(grl_ctx* ctx, int dtype, int64_t n, const void* x, void* y);
/* Replaces VulkanFNN.activation_relu (backend/fnn.py:232-283): max(0,x). */
int grl_relu(grl_ctx* ctx, int dtype, int64_t n, const void* x, void* y);
/* Replaces VulkanFNN.activation_gcu (backend/fnn.py:393-440, shaders/activation-gcu.glsl:29-31): x*cos(x). */
int grl_gcu(grl_ctx* ctx, int dtype, int64_t n, const void* x, void* y);
/* Replaces VulkanFNN.activation_roswish (backend/fnn.py:442-497, shaders/activation-roswish.glsl:30-46):
 * (x+alpha)*sigmoid(beta*x) - alpha/2. */
int grl_roswish(grl_ctx* ctx, int dtype, int64_t n, const void* x, void* y, float alpha, float beta);
/* Softmax over the last dimension of x (rows, F).  Replaces VulkanFNN.activation_softmax
 * (backend/fnn.py:574-700, shaders/activation-softmax.glsl:38-99: max from -1e10, sum of exp(x-max), quotient). */
int grl_softmax(grl_ctx* ctx, int dtype, int64_t rows, int64_t F, const void* x, void* y);
/* x (rows, 2h) -> y (rows, h): x1*(x2*sigmoid(x2)), x1 first half.
 * Replaces VulkanFNN.activation_swiglu (backend/fnn.py:499-572, shaders/activation-swiglu.glsl:21-52). */
int grl_swiglu_act(grl_ctx* ctx, int dtype, int64_t rows, int64_t h, const void* x, void* y);

/* ---- encoder pre/post steps ------------------------------------------------------------
 * x[b,s,:] = tok_emb[ids[b,s]] + pos_emb[s] + type_emb[0]   (tables fp32, x of `dtype`).
 * pos_emb and type_emb may each be NULL (a model without that table: the rotary-position
 * branch of encode adds neither, utils/vulkan_sentence_transformer.py:1148-1155).
 * Replaces the embedding steps of VulkanSentenceTransformer
 * (utils/vulkan_sentence_transformer.py:563-707). */
int grl_embed(grl_ctx* ctx, int dtype, int64_t B, int64_t S, int64_t F, int64_t vocab,
              const int32_t* ids, const float* tok_emb, const float* pos_emb,
              const float* type_emb, void* x);

/* grl_embed followed by grl_layernorm on the gathered rows, in one pass over them (the embedding LayerNorm of the
 * encoders: utils/vulkan_sentence_transformer.py:729-736 after :563-707).  The gathered row is rounded to the storage
 * type before it is normalised, as the two calls would store it; feature counts the fused kernel does not take
 * (not a multiple of 4, above 2048, unaligned tables) run the two kernels one after the other. */
int grl_embed_layernorm(grl_ctx* ctx, int dtype, int64_t B, int64_t S, int64_t F, int64_t vocab,
                        const int32_t* ids, const float* tok_emb, const float* pos_emb, const float* type_emb,
                        const float* gamma, const float* beta, float eps, void* x);
/* out[b,:] = sum_s mask[b,s]*x[b,s,:] / max(sum_s mask[b,s], 1e-9), optionally L2-normalised
 * (x / max(||x||, 1e-12)); out fp32 (B,F).
 * Replaces mean pooling + normalise of encode (utils/vulkan_sentence_transformer.py:1177-1201). */
int grl_mean_pool(grl_ctx* ctx, int dtype, int64_t B, int64_t S, int64_t F, const void* x,
                  const float* mask, float* out, int l2_normalize);

/* ---- one post-LN BERT encoder layer, device resident ----------------------------------------
 * x <- LN(x + Wo.Attn(QKV(x); mask) + bo; g1,b1,eps); x <- LN(x + W2.gelu(W1.x+b1)+b2; g2,b2,eps)
 * Replaces VulkanSentenceTransformer._forward_layer, BERT branch
 * (utils/vulkan_sentence_transformer.py:972-1035) with the fused QKV projection.
 * Weights are (out,in) matrices of `dtype`; biases and LN parameters fp32.
 * workspace: at least grl_bert_layer_workspace(...) bytes. */
typedef struct grl_bert_layer {
    const void*  w_qkv;  const float* b_qkv;     /* (3*H*D, d_model), (3*H*D) */
    const void*  w_o;    const float* b_o;       /* (d_model, H*D) */
    const float* ln1_g;  const float* ln1_b;
    const void*  w_ff1;  const float* b_ff1;     /* (d_ff, d_model) */
    const void*  w_ff2;  const float* b_ff2;     /* (d_model, d_ff) */
    const float* ln2_g;  const float* ln2_b;
} grl_bert_layer;

int64_t grl_bert_layer_workspace(int dtype, int64_t B, int64_t S, int64_t H, int64_t D, int64_t d_ff);
int grl_bert_layer_fwd(grl_ctx* ctx, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                       int64_t d_ff, const grl_bert_layer* w, const float* mask, float eps,
                       void* x, void* workspace);

/* The same layer with both LayerNorms folded into the GEMMs around them: no LayerNorm pass over HBM.  The residual
 * stream travels as RAW rows r plus their statistics: on entry r holds the rows whose LayerNorm (in_g, in_b, statistics
 * in `stats`) is the layer's input x; on return r holds x1 + FFN(x1) (x1 = LN(x + attention block; ln1)) and `stats`
 * its statistics, so that the layer's output LN(r; ln2) is formed by the next layer (whose in_g / in_b are this
 * layer's ln2 parameters) or by one grl_layernorm after the last layer.
 *   qkv = LN(r).Wqkv^T          grl_ln_gemm_nt_stats on r with the weight folded by grl_ln_fold(in_g, in_b)
 *   r   = attn.Wo^T + LN(r)     grl_gemm_nt_resln (in place), statistics of the new r out
 *   ff  = gelu(LN(r; ln1).W1^T) grl_ln_gemm_nt_stats, weight folded with ln1
 *   r   = ff.W2^T + LN(r; ln1)  grl_gemm_nt_resln (in place)
 * Same recipe as grl_bert_layer_fwd (utils/vulkan_sentence_transformer.py:972-1035); needs d_model and d_ff multiples
 * of 64 (bf16) / 32 (fp32), else GRL_ERR_SHAPE.  stats: (B*S, 2) floats, 16-byte aligned. */
typedef struct grl_bert_layer_fused {
    const void*  ws_qkv; const float* c_qkv;  const float* bf_qkv;   /* grl_ln_fold of (w_qkv, b_qkv) with in_g, in_b */
    const float* in_g;   const float* in_b;                           /* the LayerNorm that turns r into the layer input */
    const void*  w_o;    const float* b_o;
    const float* ln1_g;  const float* ln1_b;
    const void*  ws_ff1; const float* c_ff1;  const float* bf_ff1;   /* grl_ln_fold of (w_ff1, b_ff1) with ln1_g, ln1_b */
    const void*  w_ff2;  const float* b_ff2;
} grl_bert_layer_fused;

int64_t grl_bert_layer_fused_workspace(int dtype, int64_t B, int64_t S, int64_t H, int64_t D, int64_t d_ff);
int grl_bert_layer_fwd_fused(grl_ctx* ctx, int dtype, int64_t B, int64_t S, int64_t H, int64_t D,
                             int64_t d_ff, const grl_bert_layer_fused* w, const float* mask, float eps,
                             void* r, float* stats, void* workspace);

#ifdef __cplusplus
}
#endif
#endif /* GRILLY_HIP_H */
