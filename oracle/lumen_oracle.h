/*
 * lumen_oracle.h -- CPU restatement of Lumen's batch-1 inference path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP path is
 * compared against and the "port" CPU baseline that the benchmark times
 * beside the GPU.  Nothing in the shipped library links, loads or calls it.
 *
 * Every function restates one piece of the reference (chen-197/Lumen,
 * pure Rust, f32, CPU) in plain C with the same f32 operation order wherever
 * the reference's order is defined by its own source.  The file:line cited at
 * each function is relative to the reference checkout.
 *
 * Build: see oracle/Makefile (gcc -O3 -ffp-contract=off -fno-fast-math
 * -fopenmp).  -ffp-contract=off matters: rustc never contracts `a*b+c` into
 * an FMA, and it never reassociates a float reduction, so the sequential sums
 * below must stay sequential mul-then-add.
 *
 * Pinning status (what independent evidence checks each function; the
 * reference ships no tests, fixtures or golden vectors of its own):
 *   lo_gemv_f32, lo_rmsnorm_f32, lo_rope_table, lo_rope_forward,
 *   lo_rope_1token_copy, lo_silu_f32, lo_add_f32, lo_mul_f32, lo_embedding_f32,
 *   lo_attn_decode_f32, lo_attn_prefill_f32, lo_llama_forward (Llama shape):
 *     pinned by fp64 closed forms, algebraic invariants, brute force and
 *     torch / HF-transformers (config-only, random-init) cross-checks in
 *     tests/test_oracle_*.py.
 *   lo_sample_top_p: pinned in tests/test_sampler.py by the definition of
 *     nucleus sampling (share of a swept draw per token = renormalised fp64
 *     softmax over the shortest prefix reaching top_p, ties in index order,
 *     penalty and temperature special cases).
 *   lo_gemm_f32 and the two GEMMs inside lo_attn_prefill_f32: the reference
 *     calls matrixmultiply::sgemm (transitive dependency of ndarray 0.15,
 *     version not locked, source not in the reference tree); its accumulation
 *     order is implementation-defined, so bit order is PARITY UNPINNED and
 *     only value agreement within fp32 tolerance is claimed.
 *   Extensions with no reference counterpart (decoupled head_dim, per-head
 *     q/k RMSNorm, tied embeddings, bf16-stored weights, greedy argmax):
 *     pinned only by the HF Qwen3 / closed-form cross-checks; labelled
 *     "reference-extrapolated".
 */
#ifndef LUMEN_ORACLE_H
#define LUMEN_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes; each maps to one panic of the reference */
#define LO_OK 0
#define LO_ERR_SHAPE 1        /* matmul.rs:24-38 K mismatch / RHS not 2-D          */
#define LO_ERR_KV_OVERFLOW 2  /* self_attention.rs:144-149, 341-346                */
#define LO_ERR_ROPE_RANGE 3   /* encoding.rs:63-68, 176-181, 209-214               */
#define LO_ERR_EMBED_OOB 4    /* embedding.rs:55                                   */
#define LO_ERR_CACHE_COUNT 5  /* llama.rs:182-188                                  */

void lo_set_threads(int n);
int lo_get_threads(void);

/* ops ------------------------------------------------------------------- */
void lo_gemv_f32(const float *W, const float *x, float *y, int N, int K);
void lo_gemm_f32(const float *A, const float *W, float *C, int M, int N, int K);
int lo_matmul_f32(const float *A, const float *W, float *C, int M, int N, int K_a, int K_w);
void lo_rmsnorm_f32(const float *x, const float *w, float *out, int rows, int dim, float eps);
void lo_rope_table(float *cos_t, float *sin_t, int dim, int max_seq, float theta);
int lo_rope_forward(const float *x, float *out, const float *cos_t, const float *sin_t,
                    int b, int h, int s, int d, int offset, int max_seq);
int lo_rope_1token_copy(const float *src, float *dst, const float *cos_t, const float *sin_t,
                        int d, int pos, int max_seq);
void lo_silu_f32(const float *x, float *out, long n);
void lo_add_f32(const float *a, const float *b, float *out, long n);
void lo_mul_f32(const float *a, const float *b, float *out, long n);
int lo_embedding_f32(const float *W, const float *ids, int n_ids, int vocab, int dim, float *out);
void lo_bf16_to_f32(const uint16_t *src, float *dst, long n);
void lo_f32_to_bf16_rne(const float *src, uint16_t *dst, long n);
int lo_argmax_f32(const float *x, int n);
/* sample_top_p, src/main.rs:74-137, with the uniform draw r supplied by the caller */
int lo_sample_top_p(const float *logits, int n, float temperature, float top_p, float repetition_penalty,
                    const int *recent, int n_recent, float r);

/* static KV cache: k, v are [B, H_kv, max_seq, D] (self_attention.rs:24-44) */
typedef struct {
    float *k;
    float *v;
    int b, h_kv, max_seq, d;
    int len;
} lo_kv_cache;

lo_kv_cache *lo_kv_cache_new(int b, int h_kv, int max_seq, int d);
void lo_kv_cache_reset(lo_kv_cache *c);
void lo_kv_cache_free(lo_kv_cache *c);

/* decode attention core, S == 1 (self_attention.rs:125-297): q3 [B,H,D],
 * k3/v3 [B,H_kv,D] un-rotated projections; writes RoPE(k), v into the cache
 * at cache->len, bumps len, returns out [B,1,H,D]. */
int lo_attn_decode_f32(lo_kv_cache *c, const float *q3, const float *k3, const float *v3,
                       float *out, int h, const float *cos_t, const float *sin_t,
                       int rope_max_seq, float scale, int causal);

/* prefill attention core, S > 1 (self_attention.rs:308-419, 519-678): q [B,S,H,D],
 * k/v [B,S,H_kv,D] un-rotated projections; out [B,S,H,D]. */
int lo_attn_prefill_f32(lo_kv_cache *c, const float *q, const float *k, const float *v,
                        float *out, int s, int h, const float *cos_t, const float *sin_t,
                        int rope_max_seq, float scale, int causal);

/* model ------------------------------------------------------------------ */
typedef struct {
    int vocab_size, hidden_size, intermediate_size, num_hidden_layers;
    int num_attention_heads, num_key_value_heads;
    float rms_norm_eps;
    int max_seq_len;
    float rope_theta;
    /* extensions (no reference counterpart) */
    int head_dim;        /* 0 => hidden_size / num_attention_heads (llama.rs:162) */
    int qk_norm;         /* per-head RMSNorm on q and k before RoPE               */
    int tie_embeddings;  /* lm_head shares embed_tokens                           */
} lo_llama_config;

typedef struct {
    const float *wq, *wk, *wv, *wo;       /* [out,in]                        */
    const float *w_gate, *w_up, *w_down;  /* [I,H] [I,H] [H,I]               */
    const float *input_norm, *post_norm;  /* [H]                              */
    const float *q_norm, *k_norm;         /* [D] or NULL                      */
} lo_llama_layer;

typedef struct lo_llama lo_llama;

lo_llama *lo_llama_new(const lo_llama_config *cfg);
void lo_llama_free(lo_llama *m);
/* borrowed pointers; must outlive the model */
void lo_llama_set_globals(lo_llama *m, const float *embed, const float *final_norm,
                          const float *lm_head);
void lo_llama_set_layer(lo_llama *m, int layer, const lo_llama_layer *w);
void lo_llama_reset(lo_llama *m);
int lo_llama_kv_len(const lo_llama *m);
const float *lo_llama_cache_k(const lo_llama *m, int layer);
const float *lo_llama_cache_v(const lo_llama *m, int layer);
/* fills a layer's cache with rows computed elsewhere (k, v [1, Hkv, max_seq, D], rows [0, len)) and sets its length */
int lo_llama_set_kv(lo_llama *m, int layer, const float *k, const float *v, int len);
/* ids as f32 like the reference (main.rs:143-152); logits [S, V] for all
 * positions (llama.rs:205) */
int lo_llama_forward(lo_llama *m, const float *ids, int s, float *logits);

#ifdef __cplusplus
}
#endif
#endif
