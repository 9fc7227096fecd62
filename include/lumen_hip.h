/*
 * lumen_hip.h -- C ABI of liblumen_hip.so: Lumen's batch-1 inference path on
 * one AMD Instinct MI355X (gfx950), hand-written HIP kernels.
 *
 * The reference (chen-197/Lumen) is pure Rust with no FFI seam; its operator
 * API is its public Rust function surface.  Each entry point below replaces
 * one of those functions and cites it (paths relative to the reference
 * checkout).  A Rust `extern "C"` block binding these symbols is all the
 * reference needs to route its hot path here.
 *
 * Conventions
 *  - every function returns an int status (LUMEN_OK == 0); nothing throws or
 *    aborts across the boundary.  Status codes 1..5 map one-to-one to the
 *    reference's panics.  lumen_last_error() gives the message of the last
 *    failure on the calling thread.
 *  - pointers named *_dev are device pointers (from lumen_malloc or any HIP
 *    allocation, 16-byte aligned); *_host are host pointers, borrowed for the
 *    duration of the call only.
 *  - a lumen_ctx owns one HIP stream; all work of its objects is enqueued on
 *    it in call order.  Functions that return data to the host synchronise;
 *    the others only enqueue.  A ctx and its objects are not thread-safe.
 *  - linear weights are [N, K] row-major = [out_features, in_features]
 *    (src/layers/basic/linear.rs:8), never transposed.
 */
#ifndef LUMEN_HIP_H
#define LUMEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ status */
#define LUMEN_OK 0
#define LUMEN_ERR_SHAPE 1        /* src/ops/matmul.rs:24-38 (RHS not 2-D, K mismatch)            */
#define LUMEN_ERR_KV_OVERFLOW 2  /* src/layers/attention/self_attention.rs:144-149, 341-346      */
#define LUMEN_ERR_ROPE_RANGE 3   /* src/layers/attention/encoding.rs:63-68, 176-181, 209-214     */
#define LUMEN_ERR_EMBED_OOB 4    /* src/layers/basic/embedding.rs:55                             */
#define LUMEN_ERR_CACHE_COUNT 5  /* src/models/llama.rs:182-188                                  */
#define LUMEN_ERR_INVALID 6      /* null pointer, bad enum, unknown parameter name               */
#define LUMEN_ERR_HIP 7          /* a HIP runtime call failed                                    */
#define LUMEN_ERR_NO_DEVICE 8    /* no usable gfx950 device                                      */
#define LUMEN_ERR_UNSUPPORTED 9  /* shape outside what the kernels are built for                 */

#define LUMEN_DTYPE_F32 0
#define LUMEN_DTYPE_BF16 1

typedef struct lumen_ctx lumen_ctx;
typedef struct lumen_rope lumen_rope;
typedef struct lumen_kv_cache lumen_kv_cache;
typedef struct lumen_llama lumen_llama;

const char *lumen_last_error(void);
const char *lumen_version(void);

/* ----------------------------------------------------------------- context */
int lumen_ctx_create(int device, lumen_ctx **out);
int lumen_ctx_destroy(lumen_ctx *ctx);
/* run on a caller-owned hipStream_t instead of the ctx's own (NULL restores it) */
int lumen_ctx_set_stream(lumen_ctx *ctx, void *hip_stream);
int lumen_ctx_synchronize(lumen_ctx *ctx);
/* HIP-event stopwatch on the ctx stream: start enqueues an event, stop
 * enqueues a second one, waits for it and returns the elapsed milliseconds */
/* compute units of the context's device (what the launchers size their grids by) */
int lumen_ctx_num_cus(const lumen_ctx *ctx, int *num_cus_out);
int lumen_timer_start(lumen_ctx *ctx);
int lumen_timer_stop(lumen_ctx *ctx, float *ms_out);

/* device memory: stands in for the storage behind the reference's Tensor
 * (src/autograd.rs:53-64, ArcArray<f32>) */
int lumen_malloc(lumen_ctx *ctx, size_t bytes, void **dev_out);
int lumen_free(lumen_ctx *ctx, void *dev);
int lumen_upload(lumen_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
int lumen_download(lumen_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
/* device to device, in stream order (e.g. laying w_q | w_k | w_v out as one matrix for lumen_qkv_rope_append_f32) */
int lumen_copy_d2d(lumen_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes);

/* --------------------------------------------------------------------- ops */
/* ops::matmul::matmul forward, src/ops/matmul.rs:10-99.  A [M, K_a] @ W[N, K_w]^T
 * -> C [M, N].  K_a != K_w -> LUMEN_ERR_SHAPE (:33-38).  M == 1 takes the
 * memory-bound GEMV (:42-69), M > 1 the GEMM branch (:70-92): two rows stream W
 * through the vector ALU, 3-32 rows through the f32 matrix instruction (both
 * bound by the weights), more rows run on the bf16 matrix cores with every
 * f32 value taken as three bf16 parts (f32 accuracy). */
int lumen_matmul_f32(lumen_ctx *ctx, const float *A_dev, const float *W_dev, float *C_dev,
                     int M, int N, int K_a, int K_w);
/* the two branches on their own.  The GEMM splits K over workgroups when its tile grid
 * alone would not fill the chip; the partial tiles go to a workspace of the ctx (256 MiB at
 * most) that grows, with a stream synchronisation and a hipMalloc, the first time a call
 * needs more of it.  Results do not depend on scheduling (splits are added in index order). */
int lumen_gemv_f32(lumen_ctx *ctx, const float *W_dev, const float *x_dev, float *y_dev, int N, int K);
int lumen_gemm_f32(lumen_ctx *ctx, const float *A_dev, const float *W_dev, float *C_dev,
                   int M, int N, int K);
/* The fused form of the decoder layer's leaves for one token (M == 1), one launch each: y = epilogue(W rmsnorm(x)).
 * W [N, K] f32, or bf16 bits with w_bf16 = 1.  norm_w [K] not null: x is RMS-normalised first, (x * inv_rms) * g
 * with eps (RMSNorm::forward, src/layers/norm/rms_norm.rs:24-62, as applied in src/models/llama.rs:107, :113, :202);
 * norm_w null: x as it is.  Epilogues:
 *   STORE     y [N] = W x                                        (Linear::forward, src/ops/matmul.rs:42-69)
 *   RESIDUAL  y [N] = residual [N] + W x                         (src/models/llama.rs:110, :115)
 *   SWIGLU    W holds gate_proj and up_proj row-interleaved (row 2i = gate_i, row 2i + 1 = up_i, N = 2 I; build it
 *             once with lumen_interleave_rows): y [N / 2] = silu(gate) * up   (LlamaMLP::forward, llama.rs:59-65)
 * K must be a multiple of 4 (8 for bf16) and at most 16384, operands 16-byte aligned -> else LUMEN_ERR_UNSUPPORTED.
 * A decoder layer is five launches with these: lumen_qkv_rope_append_f32, lumen_attn_decode_prerotated_f32,
 * RESIDUAL (o_proj), RMSNorm + SWIGLU (gate|up), RESIDUAL (down); the model-level step (lumen_llama_forward) needs
 * three on short caches. */
#define LUMEN_GEMV_EPI_STORE 0
#define LUMEN_GEMV_EPI_RESIDUAL 1
#define LUMEN_GEMV_EPI_SWIGLU 2
#define LUMEN_GEMV_EPI_ARGMAX 3   /* model-internal (lm_head + greedy pick); named here for lumen_gemv_kernel_name */
#define LUMEN_GEMV_EPI_ROPE_QKV 4 /* what lumen_qkv_rope_append_f32 launches */
int lumen_gemv_fused_f32(lumen_ctx *ctx, const void *W_dev, int w_bf16, const float *x_dev, float *y_dev, int N, int K,
                         const float *norm_w_dev, float eps, int epilogue, const float *residual_dev);
/* out row 2i = a row i, out row 2i + 1 = b row i (rows of row_bytes bytes each, device memory, no overlap) */
int lumen_interleave_rows(lumen_ctx *ctx, const void *a_dev, const void *b_dev, void *out_dev, int rows, size_t row_bytes);
/* Name of the kernel instance -- template arguments as a profiler prints them -- that the fused product launches
 * for W [N, K] on a device with num_cus compute units (MI355X: 256), aligned operands.  Host only: no GPU needed.
 * The launcher and this function read the same decision. */
int lumen_gemv_kernel_name(int num_cus, int N, int K, int w_bf16, int rmsnorm, int epilogue, char *buf, int buf_len);
/* same products with W stored as bf16 bits and widened on load, f32 accumulate:
 * the device-side form of the reference's load-time upcast, src/loader.rs:50-64 */
int lumen_gemv_bf16w(lumen_ctx *ctx, const uint16_t *W_dev, const float *x_dev, float *y_dev, int N, int K);
int lumen_gemm_bf16w(lumen_ctx *ctx, const float *A_dev, const uint16_t *W_dev, float *C_dev,
                     int M, int N, int K);

/* measurement aid (no reference counterpart): iters GEMVs back to back on the ctx
 * stream, launch i using the weight matrix at W_base + (i % ncopies) * stride_elems
 * elements, so that each launch streams from HBM and not from a cache; ms_out is the
 * HIP-event time of the whole run. */
int lumen_gemv_bench(lumen_ctx *ctx, const void *W_base_dev, size_t stride_elems, int ncopies,
                     int w_bf16, const float *x_dev, float *y_dev, int N, int K, int iters,
                     float *ms_out);

/* RMSNorm::forward, src/layers/norm/rms_norm.rs:24-62.  x [rows, dim], w [dim] */
int lumen_rmsnorm_f32(lumen_ctx *ctx, const float *x_dev, const float *w_dev, float *out_dev,
                      int rows, int dim, float eps);
/* SiLU::forward, src/layers/activation.rs:139-146 */
int lumen_silu_f32(lumen_ctx *ctx, const float *x_dev, float *out_dev, size_t n);
/* plain device copy out[i] = x[i] (Tensor::detach / to_owned, src/autograd.rs:262-266) */
int lumen_copy_f32(lumen_ctx *ctx, const float *x_dev, float *out_dev, size_t n);
/* Tensor + Tensor and Tensor * Tensor, same shape, src/ops/arithmetic.rs:48-51, 105-108 */
int lumen_add_f32(lumen_ctx *ctx, const float *a_dev, const float *b_dev, float *out_dev, size_t n);
int lumen_mul_f32(lumen_ctx *ctx, const float *a_dev, const float *b_dev, float *out_dev, size_t n);
/* silu(gate) * up in one pass: the three elementwise ops of LlamaMLP::forward,
 * src/models/llama.rs:60-63 */
int lumen_swiglu_f32(lumen_ctx *ctx, const float *gate_dev, const float *up_dev, float *out_dev, size_t n);
/* Embedding::forward, src/layers/basic/embedding.rs:21-57.  ids are f32 on
 * the host like the reference's (src/main.rs:143-152), cast as `as usize`;
 * idx >= vocab -> LUMEN_ERR_EMBED_OOB.  out [n_ids, dim] */
int lumen_embedding_f32(lumen_ctx *ctx, const float *W_dev, const float *ids_host, int n_ids,
                        int vocab, int dim, float *out_dev);
/* greedy pick, lowest index on ties (the reference samples top-p from an
 * unseeded RNG, src/main.rs:74-137; greedy is this build's deterministic stand-in) */
int lumen_argmax_f32(lumen_ctx *ctx, const float *x_dev, int n, int *index_host_out);

/* ------------------------------------------------------------------- RoPE */
/* RotaryEmbedding::new + precompute_freqs_cis, src/layers/attention/encoding.rs:17-54.
 * Tables are computed on the host with the reference's exact f32 formula and
 * uploaded once: [max_seq, dim] cos and sin. */
int lumen_rope_create(lumen_ctx *ctx, int dim, int max_seq, float theta, lumen_rope **out);
int lumen_rope_destroy(lumen_rope *rope);
int lumen_rope_tables_download(lumen_rope *rope, float *cos_host, float *sin_host);
/* RotaryEmbedding::forward, encoding.rs:56-123.  x, out [B, H, S, D]; offset + S > max_seq
 * -> LUMEN_ERR_ROPE_RANGE (:62-68) */
int lumen_rope_forward_f32(lumen_rope *rope, const float *x_dev, float *out_dev,
                           int b, int h, int s, int d, int offset);
/* RotaryEmbedding::rope_1token_copy, encoding.rs:173-204.  src, dst [D] */
int lumen_rope_1token_copy_f32(lumen_rope *rope, const float *src_dev, float *dst_dev, int d, int pos);

/* --------------------------------------------------------------- KV cache */
/* KVCacheInner, src/layers/attention/self_attention.rs:24-44: k, v
 * [B, H_kv, max_seq, D] f32 zero-initialised in HBM, plus len.  Allocated
 * once; nothing is allocated per token. */
int lumen_kv_cache_create(lumen_ctx *ctx, int b, int h_kv, int max_seq, int d, lumen_kv_cache **out);
int lumen_kv_cache_destroy(lumen_kv_cache *cache);
int lumen_kv_cache_reset(lumen_kv_cache *cache);               /* :41-43, len = 0, data kept */
int lumen_kv_cache_len(const lumen_kv_cache *cache, int *len_out);
/* len is a public field of the reference's cache (:28): a caller that has filled rows itself
 * (lumen_kv_cache_update, or through lumen_kv_cache_ptrs) says how many are valid; outside
 * [0, max_seq] -> LUMEN_ERR_KV_OVERFLOW */
int lumen_kv_cache_set_len(lumen_kv_cache *cache, int len);
int lumen_kv_cache_ptrs(const lumen_kv_cache *cache, float **k_dev_out, float **v_dev_out);
/* legacy LlamaKVCache::update / get_view, src/kv_cache.rs:31-59: k, v
 * [B, H_kv, S, D] written at start_pos (overflow -> LUMEN_ERR_KV_OVERFLOW);
 * get_view copies the first current_len positions out, [B, H_kv, current_len, D] */
int lumen_kv_cache_update(lumen_kv_cache *cache, const float *k_dev, const float *v_dev, int s, int start_pos);
int lumen_kv_cache_get_view(const lumen_kv_cache *cache, int current_len, float *k_out_dev, float *v_out_dev);

/* -------------------------------------------------------------- attention */
/* SelfAttention::forward decode core, S == 1, self_attention.rs:125-297:
 * q3 [B, H, D], k3/v3 [B, H_kv, D] un-rotated projections.  Writes RoPE(k)
 * and v into the cache at position len, sets len += 1, rotates q, runs the
 * online-softmax GQA attention over the cache, out [B, 1, H, D]. */
int lumen_attn_decode_f32(lumen_kv_cache *cache, lumen_rope *rope, const float *q3_dev,
                          const float *k3_dev, const float *v3_dev, float *out_dev,
                          int h, float scale, int causal);
/* The fused decode step of SelfAttention::forward (S == 1, batch 1) as two operators.
 * lumen_qkv_rope_append_f32: RMSNorm (norm_w null: none) + the q, k, v projections as ONE product -- Wqkv
 * [(n_head + 2 n_kv_head) * head_dim, K] = the rows of w_q, w_k, w_v one after the other, f32 or bf16 bits -- +
 * rotation of q and k at position cache.len + write of the rotated k and the raw v to cache row cache.len
 * (src/layers/attention/self_attention.rs:106-108, :161-176, :220-227; input norm: src/models/llama.rs:107).
 * q_rot_out [n_head * head_dim] is the rotated query.  The cache length does not advance.  Errors as
 * lumen_attn_decode_f32 (KV overflow, RoPE range, shapes); the first call on a cache allocates 4 bytes.
 * lumen_attn_decode_prerotated_f32: attention of that query over cache rows [0, cache.len] -- the appended row
 * included -- (self_attention.rs:183-297); out [n_head * head_dim]; the cache length advances by one. */
int lumen_qkv_rope_append_f32(lumen_kv_cache *cache, lumen_rope *rope, const void *Wqkv_dev, int w_bf16,
                              const float *x_dev, int K, const float *norm_w_dev, float eps, float *q_rot_out_dev,
                              int n_head);
int lumen_attn_decode_prerotated_f32(lumen_kv_cache *cache, const float *q_rot_dev, float *out_dev, int n_head,
                                     float scale);
/* The same decode step for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments,
 * same results, bit for bit, as lumen_attn_decode_f32, but the scratch that the slices of a long cache need
 * (per query head and slice a partial state of head_dim + 2 values, each an 8-byte word {value, tag of the launch})
 * comes from a fixed 4 MiB array inside the library's device image instead of a hipMalloc at the first call:
 * this entry point calls no allocator.  The launch count the tags are made of sits in the same array and is
 * advanced by a one-thread kernel in front of the launch, so a call recorded into a graph is sound at every replay.
 * Partial states beyond the array (batch x heads x slices x (head_dim + 2) x 8 bytes > 4 MiB - 256 bytes; slices =
 * ceil(max_seq / (16384 / head_dim)) rounded up to a power of two, 64 at most) -> LUMEN_ERR_UNSUPPORTED.  All calls
 * on one GPU share that GPU's array: calls that overlap in time on one GPU (two contexts, two streams) race; calls
 * in stream order do not.
 * Both entry points merge the slices inside the launch: the workgroup of a head's last slice waits (bounded) for
 * the others' states; a wait that runs out is reported by the next lumen_ctx_synchronize / lumen_download on the
 * context as LUMEN_ERR_HIP. */
int lumen_attn_decode_static_f32(lumen_kv_cache *cache, lumen_rope *rope, const float *q3_dev,
                                 const float *k3_dev, const float *v3_dev, float *out_dev,
                                 int h, float scale, int causal);
/* SelfAttention::forward prefill core, S > 1, self_attention.rs:308-419 with
 * gqa_attention_no_repeat_bshd_view :519-641 and softmax_inplace_view :643-678:
 * q [B, S, H, D], k/v [B, S, H_kv, D] un-rotated; appends S positions to the
 * cache (which may already hold past_len > 0), out [B, S, H, D]. */
int lumen_attn_prefill_f32(lumen_kv_cache *cache, lumen_rope *rope, const float *q_dev,
                           const float *k_dev, const float *v_dev, float *out_dev,
                           int s, int h, float scale, int causal);

/* ------------------------------------------------------------------ model */
/* LlamaConfig, src/models/llama.rs:11-37, plus what the other benchmark
 * shapes need and the reference lacks (head_dim, qk_norm, tie_embeddings,
 * weight_dtype). */
typedef struct {
    int vocab_size, hidden_size, intermediate_size, num_hidden_layers;
    int num_attention_heads, num_key_value_heads;
    float rms_norm_eps;
    int max_seq_len;
    float rope_theta;
    int head_dim;        /* 0 => hidden_size / num_attention_heads (llama.rs:162) */
    int qk_norm;         /* per-head RMSNorm on q and k before RoPE               */
    int tie_embeddings;  /* lm_head shares model.embed_tokens.weight              */
    int weight_dtype;    /* LUMEN_DTYPE_F32, or LUMEN_DTYPE_BF16 for the linear weights */
} lumen_llama_config;

/* LlamaModel::new + init_kv_caches(1), llama.rs:138-169: allocates weights,
 * the static KV caches of all layers and every activation buffer once. */
int lumen_llama_create(lumen_ctx *ctx, const lumen_llama_config *cfg, lumen_llama **out);
int lumen_llama_destroy(lumen_llama *model);
/* ModelLoader::load_llama_weights for one tensor, src/loader.rs:23-68, by its
 * HF name (LlamaModel::named_parameters, llama.rs:218-279).  dtype f32 or
 * bf16 bits (widened like loader.rs:58 when the model stores f32); shape must
 * match -> LUMEN_ERR_SHAPE; unknown name -> LUMEN_ERR_INVALID. */
int lumen_llama_set_param(lumen_llama *model, const char *name, const void *data_host,
                          int dtype, const int64_t *shape, int ndim);
/* ModelLoader::load_llama_weights, src/loader.rs:10-80: maps a .safetensors file and
 * sets every parameter of the model that the file holds (F32 or BF16, :32-66);
 * a parameter the file lacks is counted in *n_missing_out and left as it is (the
 * reference's warning, :69-74); another dtype -> LUMEN_ERR_INVALID (:67); an element
 * count that differs from the parameter's -> LUMEN_ERR_SHAPE (:44-46).  Counters may be NULL. */
int lumen_llama_load_safetensors(lumen_llama *model, const char *path, int *n_loaded_out, int *n_missing_out);
/* the header lookup behind it (SafeTensors::deserialize + tensor(name), loader.rs:18, :24), host only:
 * dtype (LUMEN_DTYPE_* or -1 for any other), shape (ndim_inout: room in, dimensions out) and the
 * byte range of one tensor relative to the end of the header; not in the file -> LUMEN_ERR_INVALID. */
int lumen_safetensors_find(const char *path, const char *name, int *dtype_out, int64_t *shape_out,
                           int *ndim_inout, uint64_t *begin_out, uint64_t *end_out);
/* LlamaModel::forward, llama.rs:181-206: ids_host [S] as f32 (main.rs:143-152);
 * S == 1 takes the decode path, S > 1 prefill (appending to the live cache).
 * logits_host receives [S, V] when all_rows != 0 (what the reference computes)
 * or just the last position [V] (what its caller keeps, main.rs:155-163). */
int lumen_llama_forward(lumen_llama *model, const float *ids_host, int s, float *logits_host, int all_rows);
/* the generation loop of src/main.rs:340-378 with greedy picks: feeds
 * first_id, then each argmax, for n steps, without leaving the GPU.
 * ids_out_host [n] receives the picks; logits_out_host [n, V] is optional. */
int lumen_llama_decode_greedy(lumen_llama *model, int first_id, int n, int32_t *ids_out_host,
                              float *logits_out_host);
/* sample_top_p, src/main.rs:74-137 (host code there and here): repetition penalty over the
 * recent tokens, temperature, softmax, nucleus of mass top_p, inverse-CDF pick.  The uniform
 * draw r in [0,1) is an argument; the reference takes it from an unseeded generator (:69-72). */
int lumen_sample_top_p_f32(const float *logits_host, int n, float temperature, float top_p,
                           float repetition_penalty, const int32_t *recent_tokens, int n_recent,
                           float r, int32_t *index_out);
/* the seeded stand-in for rand01 (main.rs:69-72): splitmix64, 24 random bits -> [0,1) */
float lumen_rand01(uint64_t *state);
typedef struct lumen_sampling {
    float temperature, top_p, repetition_penalty; /* main.rs:223-225: 0.8, 0.9, 1.05 there */
    int recent_window;                            /* tokens the penalty looks back over, :226 (96) */
    int max_gen;                                  /* tokens per turn at most, :227 (200) */
    uint64_t seed;                                /* start of the lumen_rand01 stream of this turn */
} lumen_sampling;
/* one turn of the chat loop, src/main.rs:325-378, without the tokenizer: prefill the turn's new
 * tokens into the live cache, then sample / feed back until a stop id, max_gen, out_cap or the end
 * of the cache (len + 2 >= max_seq).  history = tokens already in the cache (the penalty window
 * reaches into them).  len + n_new + 8 >= max_seq -> LUMEN_ERR_KV_OVERFLOW: the caller resets and
 * starts a first turn, as the reference does at :266-270.  Stops on generated text (:364-366)
 * need the tokenizer and stay with the caller. */
int lumen_llama_generate_turn(lumen_llama *model, const int32_t *new_tokens, int n_new,
                              const int32_t *history, int n_history, const lumen_sampling *sampling,
                              const int32_t *stop_ids, int n_stop, int32_t *out_ids, int out_cap, int *n_out);
int lumen_llama_get_config(const lumen_llama *model, lumen_llama_config *cfg_out);
/* measurement aid (no reference counterpart): n greedy steps launched kernel by
 * kernel, every launch bracketed by HIP events on the ctx stream.  Classes:
 * 0 embedding, 1 norm+q|k|v GEMV, 2 decode attention, 3 o_proj GEMV, 4 norm+gate|up
 * GEMV, 5 down GEMV, 6 norm+lm_head GEMV, 7 argmax, 8 decode attention + o_proj in one launch
 * (short caches), 9 gate|up + down in one launch (narrow models).  ms_sum_out / count_out [n_classes >= 10]. */
int lumen_llama_decode_profile(lumen_llama *model, int first_id, int n, double *ms_sum_out,
                               int *count_out, int n_classes);
/* how S == 1 steps are issued (no reference counterpart; the results are the same):
 * GRAPH (default): one captured HIP graph replay per token (5 kernels per layer);
 * EAGER: the same kernels launched one by one (for kernel tracing tools);
 * PERSISTENT: one cooperative kernel for all layers of all requested steps -- switched
 * off in this build, lumen_llama_set_decode_mode returns LUMEN_ERR_UNSUPPORTED for it. */
#define LUMEN_DECODE_EAGER 0
#define LUMEN_DECODE_GRAPH 1
#define LUMEN_DECODE_PERSISTENT 2
int lumen_llama_set_decode_mode(lumen_llama *model, int mode);
/* name of the kernel instance the last lumen_llama_decode_profile launched for a class ("" if none) */
int lumen_llama_profile_kernel_name(const lumen_llama *model, int kernel_class, char *buf, int buf_len);
/* Where the shape allows (head_dim 64 or 128, n_head * head_dim a multiple of 512 and at most 4096 values of f32 /
 * 8192 of bf16 weights per row) and the cache is not too long (up to 16 trips of rows: 4096 rows for head_dim 64, 2048
 * for 128), decode attention and the o_proj product of a layer are ONE launch: attention workgroups hand their
 * output to resident o_proj workgroups, whose weights are already in registers, through tagged 8-byte words (no
 * reference counterpart; same results as the launches it replaces).  Form 2 puts the RMSNorm + q|k|v + RoPE product
 * in front in the same launch, handing q and the new key / value to the attention workgroups the same way: it needs
 * two q|k|v weight rows to fit a wavefront's registers (hidden 512, 1024 or 2048 in f32, twice that in bf16) and
 * n_head * head_dim == hidden (head_dim 128: also 2 * hidden); q/k-norm models (head_dim 128) are served by form 2
 * only (norm and rotation then happen in the attention workgroups).  Caches of more than two trips of rows are cut
 * into slices taken by several attention workgroups per head in parallel and folded by a further set of workgroups.
 * lumen_llama_create switches the chain on where every role is at most one workgroup per compute unit (models up to
 * ~2048 wide; wider products stream better as launches of their own).  This call picks the form (enable 0: separate
 * launches, 1: attention + o_proj, 2: q|k|v + attention + o_proj) and sets its waits:
 * spin_limit = polls after which a waiting
 * workgroup gives up -- the call that finds a wait given up returns LUMEN_ERR_HIP, its results are invalid, every
 * wavefront still exits -- and the timing of the o_proj workgroups: pre_sleep, their weight requests go out that
 * many tenths of a microsecond after the workgroup's start; poll_delay, their first poll follows that many tenths
 * later; poll_gap, pause between polls in units of 256 clocks (kept per form; the call sets those of the form in
 * use after it).  A negative argument leaves that setting as it is.  Limits (beyond them LUMEN_ERR_INVALID):
 * spin_limit <= 2^22, pre_sleep and poll_delay <= 1000 (100 us), poll_gap <= 16 -- so a wait that cannot end costs
 * about 10 s at the very worst (a few seconds with the defaults) before its workgroup flags it and exits.
 * A single-token lumen_llama_forward without a logits pointer does not synchronise: a wait given up inside it is
 * reported by the next call that does (forward with logits, decode_greedy, decode_profile).
 * enable = 1 or 2 on a shape that form does not cover -> LUMEN_ERR_UNSUPPORTED. */
int lumen_llama_set_handover(lumen_llama *model, int enable, int64_t spin_limit, int pre_sleep, int poll_delay, int poll_gap);
int lumen_llama_get_decode_mode(const lumen_llama *model, int *mode_out);
int lumen_llama_reset(lumen_llama *model);                      /* reset_kv_caches, llama.rs:172-176 */
int lumen_llama_kv_len(const lumen_llama *model, int *len_out);
/* len of every layer's cache at once (a public field of the reference's KVCacheInner, self_attention.rs:28): go
 * back to an earlier length -- the rows beyond it are overwritten by the steps that follow -- e.g. to decode the
 * same positions again, or say how many rows of caches filled with lumen_llama_cache_upload are valid.
 * Outside [0, max_seq_len] -> LUMEN_ERR_KV_OVERFLOW. */
int lumen_llama_set_kv_len(lumen_llama *model, int len);
int lumen_llama_cache_download(lumen_llama *model, int layer, float *k_host, float *v_host);
/* the other direction: a layer's cache rows from host memory, k and v [1, H_kv, max_seq, D] (k, v and len are public
 * fields of the reference's KVCacheInner, self_attention.rs:24-31: a caller may fill a cache itself and then say
 * how many rows are valid with lumen_llama_set_kv_len) */
int lumen_llama_cache_upload(lumen_llama *model, int layer, const float *k_host, const float *v_host);
/* bytes of weights + KV prefix one decode step at cache length len must read */
int lumen_llama_decode_bytes(const lumen_llama *model, int len, double *bytes_out);

/* ---- layer level: LlamaDecoderLayer::forward_infer for ONE token (src/models/llama.rs:104-116) as one operator.
 * y = h + down(silu(gate(n2)) * up(n2)), h = x + o_proj(attention(q|k|v(n1))), n1 = RMSNorm(x), n2 = RMSNorm(h), with
 * RoPE and the append of the new row to `cache` -- the launches of the model-level decode step: three per layer
 * (q|k|v + attention + o_proj chained in one, gate|up, down), two where gate|up + down chain as well, five where no
 * chain covers the shape; the cache length advances by one.
 * lumen_decoder_layer holds what such a step needs besides weights and cache (activations, RoPE tables, the words
 * values travel in between workgroups, the position counter in device memory); one handle serves every layer of a
 * stack that is called layer by layer.  cfg: hidden_size, intermediate_size, num_attention_heads,
 * num_key_value_heads, head_dim, qk_norm, rms_norm_eps, max_seq_len, rope_theta, weight_dtype (vocab_size,
 * num_hidden_layers and tie_embeddings are ignored).  Weights as the model keeps them: wqkv [(n_head + 2 n_kv_head) *
 * head_dim, hidden] = the rows of w_q, w_k, w_v one after the other; wo [hidden, n_head * head_dim]; wgu
 * [2 * intermediate, hidden] = gate / up rows interleaved (lumen_interleave_rows); wdown [hidden, intermediate]; f32 or
 * bf16 bits by cfg.weight_dtype; norm gains f32, q_norm / k_norm [head_dim] exactly when cfg.qk_norm.
 * x, y [hidden] f32 (may be the same array).  cache: batch 1, n_kv_head x max_seq_len x head_dim.
 * Every call is a set of launches of its own whose arguments carry the call's tag: not for replay from a recorded
 * graph (lumen_llama_* records its steps itself).  A wait inside a chained launch that runs out is reported by the
 * next lumen_ctx_synchronize / lumen_download on the context.  Errors: KV overflow like lumen_attn_decode_f32. */
typedef struct lumen_decoder_layer lumen_decoder_layer;
int lumen_decoder_layer_create(lumen_ctx *ctx, const lumen_llama_config *cfg, lumen_decoder_layer **out);
int lumen_decoder_layer_destroy(lumen_decoder_layer *layer);
int lumen_decoder_layer_decode_f32(lumen_decoder_layer *layer, lumen_kv_cache *cache, const void *wqkv_dev,
                                   const void *wo_dev, const void *wgu_dev, const void *wdown_dev,
                                   const float *input_norm_dev, const float *post_norm_dev, const float *q_norm_dev,
                                   const float *k_norm_dev, const float *x_dev, float *y_dev);

#ifdef __cplusplus
}
#endif
#endif
