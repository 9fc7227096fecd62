/*
 * lumen_oracle.c -- CPU restatement of Lumen's batch-1 inference path.
 * TEST INFRASTRUCTURE ONLY (checker + reported CPU baseline); see
 * lumen_oracle.h for scope, build flags and pinning status.
 *
 * Parallelism mirrors the reference: one rayon task per output row / head
 * becomes one OpenMP iteration; no reduction is ever split across threads, so
 * results do not depend on the thread count.
 */
#include "lumen_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <omp.h>

static int g_threads = 0;

void lo_set_threads(int n) {
    g_threads = n;
    if (n > 0) omp_set_num_threads(n);
}

int lo_get_threads(void) { return g_threads > 0 ? g_threads : omp_get_max_threads(); }

/* ------------------------------------------------------------------------
 * matmul, M == 1 branch.  src/ops/matmul.rs:42-69
 * One task per output n; strict sequential f32 sum over k, `sum += w * x`
 * (matmul.rs:62-65).  W is [N,K] row-major ([out,in], linear.rs:8).
 * ---------------------------------------------------------------------- */
void lo_gemv_f32(const float *W, const float *x, float *y, int N, int K) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const float *row = W + (size_t)n * K;
        float sum = 0.0f;
        for (int k = 0; k < K; ++k) sum += row[k] * x[k];
        y[n] = sum;
    }
}

/* ------------------------------------------------------------------------
 * matmul, M > 1 branch.  src/ops/matmul.rs:70-92
 * The reference hands this to ndarray::linalg::general_mat_mul ->
 * matrixmultiply::sgemm whose accumulation order is implementation-defined
 * (PARITY UNPINNED for bit order).  Restated as C[m,n] = sum_k A[m,k] W[n,k]
 * with eight interleaved partial sums per dot product so that gcc can
 * vectorise without reassociating; tests hold it to lo_gemv_f32 row by row
 * within fp32 tolerance and to an fp64 shadow.
 * ---------------------------------------------------------------------- */
static inline float dot8(const float *a, const float *b, int K) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    int k = 0;
    for (; k + 8 <= K; k += 8)
        for (int l = 0; l < 8; ++l) acc[l] += a[k + l] * b[k + l];
    float tail = 0.0f;
    for (; k < K; ++k) tail += a[k] * b[k];
    return (((acc[0] + acc[4]) + (acc[1] + acc[5])) + ((acc[2] + acc[6]) + (acc[3] + acc[7]))) + tail;
}

void lo_gemm_f32(const float *A, const float *W, float *C, int M, int N, int K) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const float *w = W + (size_t)n * K;
        for (int m = 0; m < M; ++m) C[(size_t)m * N + n] = dot8(A + (size_t)m * K, w, K);
    }
}

/* shape checks + M dispatch of matmul().  src/ops/matmul.rs:24-42 */
int lo_matmul_f32(const float *A, const float *W, float *C, int M, int N, int K_a, int K_w) {
    if (K_a != K_w) return LO_ERR_SHAPE;
    if (M == 1)
        lo_gemv_f32(W, A, C, N, K_a);
    else
        lo_gemm_f32(A, W, C, M, N, K_a);
    return LO_OK;
}

/* ------------------------------------------------------------------------
 * RMSNorm forward.  src/layers/norm/rms_norm.rs:45-58
 * sum_sq: sequential fold (:49); rms = sqrt(sum_sq/dim + eps) (:51);
 * inv = 1/rms (:52); out = (x * inv) * w (:56).
 * ---------------------------------------------------------------------- */
void lo_rmsnorm_f32(const float *x, const float *w, float *out, int rows, int dim, float eps) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        const float *xr = x + (size_t)r * dim;
        float *o = out + (size_t)r * dim;
        float sum_sq = 0.0f;
        for (int i = 0; i < dim; ++i) sum_sq = sum_sq + xr[i] * xr[i];
        float rms = sqrtf(sum_sq / (float)dim + eps);
        float inv_rms = 1.0f / rms;
        for (int i = 0; i < dim; ++i) o[i] = xr[i] * inv_rms * w[i];
    }
}

/* ------------------------------------------------------------------------
 * RoPE tables.  src/layers/attention/encoding.rs:29-54
 * freq = 1 / theta.powf(2j/dim) (:41), val = pos * freq (:42), cos/sin in
 * f32 (:44-45), duplicated into both halves (:47-50).  Tables are
 * [max_seq, dim].
 * ---------------------------------------------------------------------- */
void lo_rope_table(float *cos_t, float *sin_t, int dim, int max_seq, float theta) {
    int half_d = dim / 2;
    for (int i = 0; i < max_seq; ++i) {
        float pos = (float)i;
        for (int j = 0; j < half_d; ++j) {
            float freq = 1.0f / powf(theta, ((float)j * 2.0f) / (float)dim);
            float val = pos * freq;
            float c = cosf(val);
            float s = sinf(val);
            cos_t[(size_t)i * dim + j] = c;
            cos_t[(size_t)i * dim + j + half_d] = c;
            sin_t[(size_t)i * dim + j] = s;
            sin_t[(size_t)i * dim + j + half_d] = s;
        }
    }
}

/* ------------------------------------------------------------------------
 * RotaryEmbedding::forward on [B,H,S,D] with position offset.
 * src/layers/attention/encoding.rs:56-123 (range check :62-68, rotation
 * :103-116: out[j] = x1*c - x2*s; out[j+half] = x2*c + x1*s).
 * ---------------------------------------------------------------------- */
int lo_rope_forward(const float *x, float *out, const float *cos_t, const float *sin_t,
                    int b, int h, int s, int d, int offset, int max_seq) {
    if (offset + s > max_seq) return LO_ERR_ROPE_RANGE;
    int half = d / 2;
    for (int bb = 0; bb < b; ++bb)
        for (int hh = 0; hh < h; ++hh)
            for (int ss = 0; ss < s; ++ss) {
                const float *xr = x + (((size_t)bb * h + hh) * s + ss) * d;
                float *o = out + (((size_t)bb * h + hh) * s + ss) * d;
                const float *cr = cos_t + (size_t)(offset + ss) * d;
                const float *sr = sin_t + (size_t)(offset + ss) * d;
                for (int j = 0; j < half; ++j) {
                    float x1 = xr[j], x2 = xr[j + half];
                    float c = cr[j], sv = sr[j];
                    o[j] = x1 * c - x2 * sv;
                    o[j + half] = x2 * c + x1 * sv;
                }
            }
    return LO_OK;
}

/* rope_1token_copy.  src/layers/attention/encoding.rs:173-204 */
int lo_rope_1token_copy(const float *src, float *dst, const float *cos_t, const float *sin_t,
                        int d, int pos, int max_seq) {
    if (pos >= max_seq) return LO_ERR_ROPE_RANGE;
    const float *cr = cos_t + (size_t)pos * d;
    const float *sr = sin_t + (size_t)pos * d;
    int half = d / 2;
    for (int j = 0; j < half; ++j) {
        float x1 = src[j], x2 = src[j + half];
        float c = cr[j], sv = sr[j];
        dst[j] = x1 * c - x2 * sv;
        dst[j + half] = x2 * c + x1 * sv;
    }
    return LO_OK;
}

/* SiLU forward.  src/layers/activation.rs:143-146: sig = 1/(1+exp(-x)); x*sig */
void lo_silu_f32(const float *x, float *out, long n) {
#pragma omp parallel for schedule(static)
    for (long i = 0; i < n; ++i) {
        float sig = 1.0f / (1.0f + expf(-x[i]));
        out[i] = x[i] * sig;
    }
}

/* Tensor + Tensor, same shape.  src/ops/arithmetic.rs:48-51 */
void lo_add_f32(const float *a, const float *b, float *out, long n) {
    for (long i = 0; i < n; ++i) out[i] = a[i] + b[i];
}

/* Tensor * Tensor, same shape.  src/ops/arithmetic.rs:105-108 */
void lo_mul_f32(const float *a, const float *b, float *out, long n) {
    for (long i = 0; i < n; ++i) out[i] = a[i] * b[i];
}

/* Embedding forward.  src/layers/basic/embedding.rs:47-57: ids are f32, cast
 * `as usize` (saturating: negative / NaN -> 0), idx >= vocab panics (:55). */
int lo_embedding_f32(const float *W, const float *ids, int n_ids, int vocab, int dim, float *out) {
    for (int t = 0; t < n_ids; ++t) {
        float f = ids[t];
        size_t idx = (f > 0.0f) ? (f >= 1.8446744e19f ? (size_t)-1 : (size_t)f) : 0; /* NaN -> 0 */
        if (idx >= (size_t)vocab) return LO_ERR_EMBED_OOB;
        memcpy(out + (size_t)t * dim, W + idx * dim, sizeof(float) * (size_t)dim);
    }
    return LO_OK;
}

/* bf16 -> f32 exact widening.  src/loader.rs:58 (half::bf16::to_f32) */
void lo_bf16_to_f32(const uint16_t *src, float *dst, long n) {
    for (long i = 0; i < n; ++i) {
        uint32_t u = (uint32_t)src[i] << 16;
        memcpy(dst + i, &u, 4);
    }
}

/* f32 -> bf16 round-to-nearest-even (test-input preparation for the
 * bf16-weight configuration; no reference counterpart). */
void lo_f32_to_bf16_rne(const float *src, uint16_t *dst, long n) {
    for (long i = 0; i < n; ++i) {
        uint32_t u;
        memcpy(&u, src + i, 4);
        if ((u & 0x7fffffffu) > 0x7f800000u) {
            dst[i] = (uint16_t)((u >> 16) | 0x40);
        } else {
            u += 0x7fffu + ((u >> 16) & 1u);
            dst[i] = (uint16_t)(u >> 16);
        }
    }
}

/* greedy pick: first index of the maximum (no reference counterpart; the
 * reference samples top-p with an unseeded RNG, main.rs:74-137). */
int lo_argmax_f32(const float *x, int n) {
    int best = 0;
    for (int i = 1; i < n; ++i)
        if (x[i] > x[best]) best = i;
    return best;
}

/* sample_top_p, src/main.rs:74-137, with the uniform draw r passed in (the
 * reference takes it from an unseeded generator, :69-72).  Steps as written
 * there: logits of the recent tokens divided by the penalty (also negative
 * ones, :84-89), division by max(temperature, 1e-5), softmax with divisor
 * (sum + 1e-9) in f32 (:100-110), indices sorted by probability descending --
 * a stable sort, equal probabilities stay in index order (:113-114) --
 * nucleus = shortest prefix whose running f32 sum reaches
 * clamp(top_p, 0, 1).max(1e-6) (:116-126), then the first index whose running
 * sum of p / cumulative reaches r, else the nucleus' last (:129-137).
 * Returns -1 when n <= 0. */
int lo_sample_top_p(const float *logits, int n, float temperature, float top_p, float repetition_penalty,
                    const int *recent, int n_recent, float r) {
    if (n <= 0) return -1;
    float *adj = (float *)malloc(sizeof(float) * (size_t)n);
    int *idx = (int *)malloc(sizeof(int) * (size_t)n);
    int *tmp = (int *)malloc(sizeof(int) * (size_t)n);
    memcpy(adj, logits, sizeof(float) * (size_t)n);
    if (repetition_penalty > 1.0f)
        for (int i = 0; i < n_recent; ++i)
            if (recent[i] >= 0 && recent[i] < n) adj[recent[i]] /= repetition_penalty;
    const float temp = temperature > 1e-5f ? temperature : 1e-5f;
    for (int i = 0; i < n; ++i) adj[i] /= temp;
    float maxv = -INFINITY;
    for (int i = 0; i < n; ++i)
        if (adj[i] > maxv) maxv = adj[i];
    float sum = 0.f;
    for (int i = 0; i < n; ++i) {
        adj[i] = expf(adj[i] - maxv);
        sum += adj[i];
    }
    const float inv = 1.0f / (sum + 1e-9f);
    for (int i = 0; i < n; ++i) adj[i] *= inv;
    /* bottom-up merge sort, descending by probability, stable */
    for (int i = 0; i < n; ++i) idx[i] = i;
    for (int w = 1; w < n; w *= 2) {
        for (int lo = 0; lo < n; lo += 2 * w) {
            int mid = lo + w < n ? lo + w : n, hi = lo + 2 * w < n ? lo + 2 * w : n;
            int a = lo, b = mid, o = lo;
            while (a < mid && b < hi) tmp[o++] = (adj[idx[b]] > adj[idx[a]]) ? idx[b++] : idx[a++];
            while (a < mid) tmp[o++] = idx[a++];
            while (b < hi) tmp[o++] = idx[b++];
        }
        int *sw = idx;
        idx = tmp;
        tmp = sw;
    }
    float target = top_p < 0.f ? 0.f : (top_p > 1.f ? 1.f : top_p);
    if (target < 1e-6f) target = 1e-6f;
    float cumulative = 0.f;
    int cut = 0;
    for (int k = 0; k < n; ++k) {
        cumulative += adj[idx[k]];
        cut = k + 1;
        if (cumulative >= target) break;
    }
    if (cut < 1) cut = 1;
    float acc = 0.f;
    int pick = idx[cut - 1];
    for (int k = 0; k < cut; ++k) {
        acc += adj[idx[k]] / cumulative;
        if (r <= acc) {
            pick = idx[k];
            break;
        }
    }
    free(adj);
    free(idx);
    free(tmp);
    return pick;
}

/* ------------------------------------------------------------------------
 * KVCacheInner.  src/layers/attention/self_attention.rs:24-44
 * ---------------------------------------------------------------------- */
lo_kv_cache *lo_kv_cache_new(int b, int h_kv, int max_seq, int d) {
    lo_kv_cache *c = (lo_kv_cache *)calloc(1, sizeof(*c));
    size_t n = (size_t)b * h_kv * max_seq * d;
    c->k = (float *)calloc(n, sizeof(float));
    c->v = (float *)calloc(n, sizeof(float));
    c->b = b;
    c->h_kv = h_kv;
    c->max_seq = max_seq;
    c->d = d;
    c->len = 0;
    return c;
}

void lo_kv_cache_reset(lo_kv_cache *c) { c->len = 0; } /* :41-43: no zeroing */

void lo_kv_cache_free(lo_kv_cache *c) {
    if (!c) return;
    free(c->k);
    free(c->v);
    free(c);
}

/* ------------------------------------------------------------------------
 * Decode attention, S == 1.  src/layers/attention/self_attention.rs:125-297
 *   :141-180  RoPE(k) -> cache.k[b,hk,past_len,:], memcpy v, len = past_len+1
 *   :199-293  one task per (b, hq): hk = hq / n_rep (:205); RoPE(q) (:220-227);
 *             branchy online softmax over j (:255-285); out = ctx/(l+1e-9) (:287-290)
 * ---------------------------------------------------------------------- */
int lo_attn_decode_f32(lo_kv_cache *c, const float *q3, const float *k3, const float *v3,
                       float *out, int h, const float *cos_t, const float *sin_t,
                       int rope_max_seq, float scale, int causal) {
    const int b = c->b, h_kv = c->h_kv, d = c->d, max_seq = c->max_seq;
    const int n_rep = h / h_kv;
    const int past_len = c->len;
    const int new_len = past_len + 1;
    if (new_len > max_seq) return LO_ERR_KV_OVERFLOW;
    if (past_len >= rope_max_seq) return LO_ERR_ROPE_RANGE;

    for (int bb = 0; bb < b; ++bb)
        for (int hk = 0; hk < h_kv; ++hk) {
            const float *src_k = k3 + ((size_t)bb * h_kv + hk) * d;
            const float *src_v = v3 + ((size_t)bb * h_kv + hk) * d;
            float *dst_k = c->k + (((size_t)bb * h_kv + hk) * max_seq + past_len) * d;
            float *dst_v = c->v + (((size_t)bb * h_kv + hk) * max_seq + past_len) * d;
            lo_rope_1token_copy(src_k, dst_k, cos_t, sin_t, d, past_len, rope_max_seq);
            memcpy(dst_v, src_v, sizeof(float) * (size_t)d);
        }
    c->len = new_len;

    const int total_len = past_len + 1;
    const int half_d = d / 2;
    const float *cos_row = cos_t + (size_t)past_len * d; /* cos_sin_row_vec, encoding.rs:208-229 */
    const float *sin_row = sin_t + (size_t)past_len * d;

#pragma omp parallel for schedule(static)
    for (int row = 0; row < b * h; ++row) {
        int bb = row / h, hh = row % h, hk = hh / n_rep;
        float qbuf[512];
        float ctx[512];
        float *qb = d <= 512 ? qbuf : (float *)malloc(sizeof(float) * (size_t)d);
        float *cx = d <= 512 ? ctx : (float *)malloc(sizeof(float) * (size_t)d);
        const float *q_src = q3 + ((size_t)bb * h + hh) * d;
        for (int j = 0; j < half_d; ++j) {
            float x1 = q_src[j], x2 = q_src[j + half_d];
            float cc = cos_row[j], s_val = sin_row[j];
            qb[j] = x1 * cc - x2 * s_val;
            qb[j + half_d] = x1 * s_val + x2 * cc;
        }
        const float *k_sl = c->k + ((size_t)bb * h_kv + hk) * max_seq * d;
        const float *v_sl = c->v + ((size_t)bb * h_kv + hk) * max_seq * d;
        for (int i = 0; i < d; ++i) cx[i] = 0.0f;
        float m = -INFINITY, l = 0.0f;
        for (int j = 0; j < total_len; ++j) {
            if (causal && j > past_len) break;
            const float *k_row = k_sl + (size_t)j * d;
            float dot = 0.0f;
            for (int i = 0; i < d; ++i) dot += qb[i] * k_row[i];
            float score = dot * scale;
            const float *v_row = v_sl + (size_t)j * d;
            if (score > m) {
                float s = expf(m - score);
                for (int i = 0; i < d; ++i) cx[i] *= s;
                l *= s;
                m = score;
                for (int i = 0; i < d; ++i) cx[i] += v_row[i];
                l += 1.0f;
            } else {
                float w = expf(score - m);
                for (int i = 0; i < d; ++i) cx[i] += w * v_row[i];
                l += w;
            }
        }
        float inv = 1.0f / (l + 1e-9f);
        float *out_row = out + (size_t)row * d;
        for (int i = 0; i < d; ++i) out_row[i] = cx[i] * inv;
        if (d > 512) {
            free(qb);
            free(cx);
        }
    }
    return LO_OK;
}

/* ------------------------------------------------------------------------
 * Prefill attention, S > 1.  src/layers/attention/self_attention.rs:308-419
 *   :334-335  RoPE(q), RoPE(k) with offset past_len (encoding.rs:56-123)
 *   :397-402  cache[.., past_len..new_len, ..] = k_rot / v; len = new_len
 *   :519-641  gqa_attention_no_repeat_bshd_view, S>1 branch :603-637:
 *             scores = Q K^T (sgemm), softmax_inplace_view (:643-678: *scale,
 *             j > past_len+i -> -inf, max, exp, 1/(sum+1e-9)), ctx = P V (sgemm)
 * The two sgemm calls have implementation-defined order (PARITY UNPINNED for
 * bits).  Masked entries become exp(-inf) = 0 and add exactly 0 to ctx, so
 * skipping them is value-identical; one score row is live at a time instead
 * of the reference's S*L buffer.
 * ---------------------------------------------------------------------- */
int lo_attn_prefill_f32(lo_kv_cache *c, const float *q, const float *k, const float *v,
                        float *out, int s, int h, const float *cos_t, const float *sin_t,
                        int rope_max_seq, float scale, int causal) {
    const int b = c->b, h_kv = c->h_kv, d = c->d, max_seq = c->max_seq;
    const int n_rep = h / h_kv;
    const int past_len = c->len;
    const int new_len = past_len + s;
    const int half = d / 2;
    if (past_len + s > rope_max_seq) return LO_ERR_ROPE_RANGE;
    if (new_len > max_seq) return LO_ERR_KV_OVERFLOW;

    /* rotated q in [B,H,S,D] */
    float *q_rot = (float *)malloc(sizeof(float) * (size_t)b * h * s * d);
#pragma omp parallel for schedule(static) collapse(2)
    for (int bb = 0; bb < b; ++bb)
        for (int ss = 0; ss < s; ++ss) {
            const float *cr = cos_t + (size_t)(past_len + ss) * d;
            const float *sr = sin_t + (size_t)(past_len + ss) * d;
            for (int hh = 0; hh < h; ++hh) {
                const float *xr = q + (((size_t)bb * s + ss) * h + hh) * d;
                float *o = q_rot + (((size_t)bb * h + hh) * s + ss) * d;
                for (int j = 0; j < half; ++j) {
                    float x1 = xr[j], x2 = xr[j + half];
                    o[j] = x1 * cr[j] - x2 * sr[j];
                    o[j + half] = x2 * cr[j] + x1 * sr[j];
                }
            }
            for (int hk = 0; hk < h_kv; ++hk) {
                const float *xr = k + (((size_t)bb * s + ss) * h_kv + hk) * d;
                const float *vr = v + (((size_t)bb * s + ss) * h_kv + hk) * d;
                float *ko = c->k + (((size_t)bb * h_kv + hk) * max_seq + past_len + ss) * d;
                float *vo = c->v + (((size_t)bb * h_kv + hk) * max_seq + past_len + ss) * d;
                for (int j = 0; j < half; ++j) {
                    float x1 = xr[j], x2 = xr[j + half];
                    ko[j] = x1 * cr[j] - x2 * sr[j];
                    ko[j + half] = x2 * cr[j] + x1 * sr[j];
                }
                memcpy(vo, vr, sizeof(float) * (size_t)d);
            }
        }
    c->len = new_len;
    const int L = new_len;

#pragma omp parallel
    {
        float *scores = (float *)malloc(sizeof(float) * (size_t)L);
#pragma omp for schedule(dynamic, 8) collapse(3)
        for (int bb = 0; bb < b; ++bb)
            for (int hq = 0; hq < h; ++hq)
                for (int i = 0; i < s; ++i) {
                    const int hk = hq / n_rep;
                    const float *k_mat = c->k + ((size_t)bb * h_kv + hk) * max_seq * d;
                    const float *v_mat = c->v + ((size_t)bb * h_kv + hk) * max_seq * d;
                    const float *q_vec = q_rot + (((size_t)bb * h + hq) * s + i) * d;
                    const int q_abs = past_len + i;
                    const int j_end = causal ? (q_abs + 1 < L ? q_abs + 1 : L) : L;
                    float maxv = -INFINITY;
                    for (int j = 0; j < j_end; ++j) {
                        float val = dot8(q_vec, k_mat + (size_t)j * d, d) * scale;
                        scores[j] = val;
                        if (val > maxv) maxv = val;
                    }
                    float sum = 0.0f;
                    for (int j = 0; j < j_end; ++j) {
                        float e = expf(scores[j] - maxv);
                        scores[j] = e;
                        sum += e;
                    }
                    float inv = 1.0f / (sum + 1e-9f);
                    float *o = out + (((size_t)bb * s + i) * h + hq) * d;
                    for (int t = 0; t < d; ++t) o[t] = 0.0f;
                    for (int j = 0; j < j_end; ++j) {
                        float p = scores[j] * inv;
                        const float *vr = v_mat + (size_t)j * d;
                        for (int t = 0; t < d; ++t) o[t] += p * vr[t];
                    }
                }
        free(scores);
    }
    free(q_rot);
    return LO_OK;
}

/* ------------------------------------------------------------------------
 * LlamaModel.  src/models/llama.rs:138-206 (+ LlamaMLP :59-65,
 * LlamaDecoderLayer::forward_infer :104-116, SelfAttention::forward
 * self_attention.rs:96-427, init/reset_kv_caches llama.rs:161-176)
 * ---------------------------------------------------------------------- */
struct lo_llama {
    lo_llama_config cfg;
    int head_dim;
    float scale;
    const float *embed, *final_norm, *lm_head;
    lo_llama_layer *layers;
    lo_kv_cache **caches;
    float *cos_t, *sin_t; /* one table; the reference builds an identical one per layer */
};

lo_llama *lo_llama_new(const lo_llama_config *cfg) {
    lo_llama *m = (lo_llama *)calloc(1, sizeof(*m));
    m->cfg = *cfg;
    m->head_dim = cfg->head_dim > 0 ? cfg->head_dim : cfg->hidden_size / cfg->num_attention_heads;
    m->scale = 1.0f / sqrtf((float)m->head_dim); /* self_attention.rs:89 sqrt().recip() */
    m->layers = (lo_llama_layer *)calloc((size_t)cfg->num_hidden_layers, sizeof(lo_llama_layer));
    m->caches = (lo_kv_cache **)calloc((size_t)cfg->num_hidden_layers, sizeof(lo_kv_cache *));
    for (int i = 0; i < cfg->num_hidden_layers; ++i)
        m->caches[i] = lo_kv_cache_new(1, cfg->num_key_value_heads, cfg->max_seq_len, m->head_dim);
    m->cos_t = (float *)malloc(sizeof(float) * (size_t)cfg->max_seq_len * m->head_dim);
    m->sin_t = (float *)malloc(sizeof(float) * (size_t)cfg->max_seq_len * m->head_dim);
    lo_rope_table(m->cos_t, m->sin_t, m->head_dim, cfg->max_seq_len, cfg->rope_theta);
    return m;
}

void lo_llama_free(lo_llama *m) {
    if (!m) return;
    for (int i = 0; i < m->cfg.num_hidden_layers; ++i) lo_kv_cache_free(m->caches[i]);
    free(m->caches);
    free(m->layers);
    free(m->cos_t);
    free(m->sin_t);
    free(m);
}

void lo_llama_set_globals(lo_llama *m, const float *embed, const float *final_norm,
                          const float *lm_head) {
    m->embed = embed;
    m->final_norm = final_norm;
    m->lm_head = m->cfg.tie_embeddings ? embed : lm_head;
}

void lo_llama_set_layer(lo_llama *m, int layer, const lo_llama_layer *w) { m->layers[layer] = *w; }

void lo_llama_reset(lo_llama *m) {
    for (int i = 0; i < m->cfg.num_hidden_layers; ++i) lo_kv_cache_reset(m->caches[i]);
}

int lo_llama_kv_len(const lo_llama *m) { return m->caches[0]->len; }
const float *lo_llama_cache_k(const lo_llama *m, int layer) { return m->caches[layer]->k; }
const float *lo_llama_cache_v(const lo_llama *m, int layer) { return m->caches[layer]->v; }

/* KVCacheInner's k, v and len are public fields (self_attention.rs:24-31): a caller may fill a cache with rows
 * computed elsewhere and go on from there.  k, v: [1, Hkv, max_seq, D]; only rows [0, len) are copied. */
int lo_llama_set_kv(lo_llama *m, int layer, const float *k, const float *v, int len) {
    if (layer < 0 || layer >= m->cfg.num_hidden_layers) return LO_ERR_CACHE_COUNT;
    lo_kv_cache *c = m->caches[layer];
    if (len < 0 || len > c->max_seq) return LO_ERR_KV_OVERFLOW;
    for (int h = 0; h < c->h_kv; ++h) {
        const size_t off = (size_t)h * c->max_seq * c->d;
        memcpy(c->k + off, k + off, sizeof(float) * (size_t)len * c->d);
        memcpy(c->v + off, v + off, sizeof(float) * (size_t)len * c->d);
    }
    c->len = len;
    return LO_OK;
}

int lo_llama_forward(lo_llama *m, const float *ids, int s, float *logits) {
    const lo_llama_config *cfg = &m->cfg;
    const int H = cfg->hidden_size, I = cfg->intermediate_size, V = cfg->vocab_size;
    const int Hq = cfg->num_attention_heads, Hkv = cfg->num_key_value_heads, D = m->head_dim;
    const int qd = Hq * D, kvd = Hkv * D;
    int rc = LO_OK;

    float *x = (float *)malloc(sizeof(float) * (size_t)s * H);
    float *nx = (float *)malloc(sizeof(float) * (size_t)s * H);
    float *hbuf = (float *)malloc(sizeof(float) * (size_t)s * H);
    float *q = (float *)malloc(sizeof(float) * (size_t)s * qd);
    float *k = (float *)malloc(sizeof(float) * (size_t)s * kvd);
    float *v = (float *)malloc(sizeof(float) * (size_t)s * kvd);
    float *ctx = (float *)malloc(sizeof(float) * (size_t)s * qd);
    float *attn_out = (float *)malloc(sizeof(float) * (size_t)s * H);
    float *gate = (float *)malloc(sizeof(float) * (size_t)s * I);
    float *up = (float *)malloc(sizeof(float) * (size_t)s * I);

    rc = lo_embedding_f32(m->embed, ids, s, V, H, x); /* llama.rs:191 */
    for (int li = 0; rc == LO_OK && li < cfg->num_hidden_layers; ++li) {
        const lo_llama_layer *w = &m->layers[li];
        lo_kv_cache *cache = m->caches[li];
        lo_rmsnorm_f32(x, w->input_norm, nx, s, H, cfg->rms_norm_eps);  /* llama.rs:107 */
        lo_matmul_f32(nx, w->wq, q, s, qd, H, H);                      /* self_attention.rs:106 */
        lo_matmul_f32(nx, w->wk, k, s, kvd, H, H);                     /* :107 */
        lo_matmul_f32(nx, w->wv, v, s, kvd, H, H);                     /* :108 */
        if (cfg->qk_norm) { /* extension: per-head RMSNorm before RoPE */
            lo_rmsnorm_f32(q, w->q_norm, q, s * Hq, D, cfg->rms_norm_eps);
            lo_rmsnorm_f32(k, w->k_norm, k, s * Hkv, D, cfg->rms_norm_eps);
        }
        if (s == 1)
            rc = lo_attn_decode_f32(cache, q, k, v, ctx, Hq, m->cos_t, m->sin_t, cfg->max_seq_len,
                                    m->scale, 1);
        else
            rc = lo_attn_prefill_f32(cache, q, k, v, ctx, s, Hq, m->cos_t, m->sin_t,
                                     cfg->max_seq_len, m->scale, 1);
        if (rc != LO_OK) break;
        lo_matmul_f32(ctx, w->wo, attn_out, s, H, qd, qd);             /* :303 / :424 */
        lo_add_f32(x, attn_out, hbuf, (long)s * H);                    /* llama.rs:110 */
        lo_rmsnorm_f32(hbuf, w->post_norm, nx, s, H, cfg->rms_norm_eps); /* :113 */
        lo_matmul_f32(nx, w->w_gate, gate, s, I, H, H);                /* llama.rs:60 */
        lo_silu_f32(gate, gate, (long)s * I);                          /* :61 */
        lo_matmul_f32(nx, w->w_up, up, s, I, H, H);                    /* :62 */
        lo_mul_f32(gate, up, gate, (long)s * I);                       /* :63 */
        lo_matmul_f32(gate, w->w_down, attn_out, s, H, I, I);          /* :64 */
        lo_add_f32(hbuf, attn_out, x, (long)s * H);                    /* llama.rs:115 */
    }
    if (rc == LO_OK) {
        lo_rmsnorm_f32(x, m->final_norm, nx, s, H, cfg->rms_norm_eps); /* llama.rs:202 */
        lo_matmul_f32(nx, m->lm_head, logits, s, V, H, H);             /* llama.rs:205 */
    }
    free(x); free(nx); free(hbuf); free(q); free(k); free(v); free(ctx); free(attn_out);
    free(gate); free(up);
    return rc;
}
