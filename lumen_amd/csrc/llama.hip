// LlamaModel on one GPU: src/models/llama.rs:129-280.
//
// Everything a decode step touches is allocated once at create time: the
// weights (q|k|v rows concatenated, gate/up rows interleaved so that their
// GEMVs run as one launch each), one KV slab for all layers, the activation
// vectors, the token id and the position counter.  A decode step is a fixed
// sequence of 5 kernels per layer that reads the token id and position from
// device memory, so the whole step is captured once as a HIP graph and
// replayed per token; greedy generation never returns to the host between
// tokens.
#include "internal.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <string>

struct LayerW {
    void *wqkv = nullptr, *wo = nullptr, *wgu = nullptr, *wdown = nullptr;  // weight dtype
    float *in_norm = nullptr, *post_norm = nullptr, *q_norm = nullptr, *k_norm = nullptr;
};

struct lumen_llama {
    lumen_ctx *ctx = nullptr;
    lumen_llama_config cfg = {};
    int D = 0, qd = 0, kvd = 0, qkvd = 0;
    bool bf16 = false;
    bool layer_only = false;  // the state of a decode step without a model (lumen_decoder_layer_*)
    unsigned layer_epoch = 0;  // ... and the count of its launches, which their hand-over tags are made of
    size_t esz = 4;
    float scale = 0.f;
    float *embed = nullptr;    // [V,H] f32 (bf16 sources are widened: same values)
    void *lm_head = nullptr;   // [V,H] weight dtype; aliases embed when tied and f32
    bool lm_head_owned = false;
    float *final_norm = nullptr;
    std::vector<LayerW> layers;
    float *cos_dev = nullptr, *sin_dev = nullptr;
    float *k_slab = nullptr, *v_slab = nullptr;  // [layers][1][Hkv][max_seq][D]
    size_t cache_stride = 0;
    int len = 0;  // host mirror of *d_pos
    // decode state
    float *x = nullptr, *h = nullptr, *qkv = nullptr, *attn = nullptr, *act = nullptr, *logits = nullptr;
    int *d_tok = nullptr, *d_pos = nullptr;
    int *tok_hist = nullptr;  // [max_seq + 1]: greedy pick made at position p sits at index p + 1
    float *part = nullptr;                          // slice states for the o_proj product to fold (defer_merge)
    unsigned long long *part_merge = nullptr;       // slice states folded inside the attention launch (tagged words)
    int nsplit = 1;     // slices of a long cache in the decode attention kernel
    bool defer_merge = false;  // the o_proj GEMV, not the attention kernel, may merge the slices of a long cache
    // short caches: attention and o_proj chained in one launch (attn_oproj.hip); its hand-over buffer, the decode
    // step counter its tags are made of, the flag a timed-out wait leaves, and the poll limit of a wait
    int chain_ao = 0;  // 0: off, 1: attention -> o_proj, 2: q|k|v -> attention -> o_proj
    unsigned long long *x_tagged = nullptr, *qkv_tagged = nullptr;
    unsigned *d_step = nullptr;
    int *d_err = nullptr;
    unsigned spin_limit = 1u << 22;
    // timing of the chain's o_proj workgroups, per form: weight requests this long after the workgroup's start and
    // first poll this long after them (units of 0.1 us), pause between polls (units of 256 clocks); measured optima
    // on the 2048-wide model, see attn_oproj.hip
    int chain_pre[3] = {0, 11, 55}, chain_delay[3] = {0, 17, 15}, chain_gap[3] = {0, 1, 1};
    std::string prof_names[16];  // per kernel class: the instance the last lumen_llama_decode_profile launched
    hipGraph_t graph = nullptr;
    hipGraphExec_t graph_exec = nullptr;
    int graph_expect_short = 0;            // the hint the captured attention launches carry
    int graph_slices = 0;                  // ... and the slices of their chained launch
    // narrow models: gate|up and down chained in one launch (mlp_chain.hip); pauses of its down workgroups
    bool chain_mlp = false, chain_ao_on = true;
    unsigned long long *act_tagged = nullptr;  // [I]
    // (no pauses: between its two roles there is no hand-over that the down weights could get in the way of;
    // measured on the Qwen3-0.6B shape: 0.677 ms per token without, 0.698 with 30 / 10)
    int mlp_pre = 0, mlp_delay = 0, mlp_gap = 1;
    int chain_max_slices = 8;                      // caches beyond that many slices take separate launches
    int chain_slice_trips = 0;                     // > 0: trips per slice fixed (measurements), else chosen by length
    unsigned long long *part_tagged = nullptr;     // [Hq][ATTN_CHAIN_MAX_SLICES][D + 2]
    int decode_mode = LUMEN_DECODE_GRAPH;
    unsigned long long *amax_word = nullptr;  // per-workgroup candidates of the lm_head product's arg-max
    unsigned *amax_epoch = nullptr;
    // prefill buffers (grown on demand, kept)
    int pf_cap = 0, pf_logit_cap = 0;
    float *p_x = nullptr, *p_h = nullptr, *p_n = nullptr, *p_qkv = nullptr, *p_qrot = nullptr, *p_attn = nullptr,
          *p_act = nullptr, *p_logits = nullptr;
    int *p_ids = nullptr;
    std::vector<void *> allocs;
};

static int dmalloc(lumen_llama *m, void **p, size_t bytes) {
    HIP_TRY(hipMalloc(p, bytes ? bytes : 16));
    m->allocs.push_back(*p);
    return LUMEN_OK;
}

// a weight matrix: zero until a parameter is set, so that a file that lacks a tensor gives defined results
static int dmalloc_weight(lumen_llama *m, void **p, size_t bytes) {
    LUMEN_TRY(dmalloc(m, p, bytes));
    HIP_TRY(hipMemsetAsync(*p, 0, bytes ? bytes : 16, m->ctx->stream));
    return LUMEN_OK;
}

template <typename T>
static int dmalloc_t(lumen_llama *m, T **p, size_t count) { return dmalloc(m, (void **)p, count * sizeof(T)); }

static int fill_ones(lumen_llama *m, float *dst, size_t n) {
    std::vector<float> ones(n, 1.0f);
    return lumen_upload(m->ctx, dst, ones.data(), n * sizeof(float));
}

extern "C" int lumen_llama_destroy(lumen_llama *m) {
    if (!m) return LUMEN_OK;
    hipStreamSynchronize(m->ctx->stream);
    if (m->graph_exec) hipGraphExecDestroy(m->graph_exec);
    if (m->graph) hipGraphDestroy(m->graph);
    for (void *p : m->allocs) hipFree(p);
    hipFree(m->p_x); hipFree(m->p_h); hipFree(m->p_n); hipFree(m->p_qkv); hipFree(m->p_qrot);
    hipFree(m->p_attn); hipFree(m->p_act); hipFree(m->p_logits); hipFree(m->p_ids);
    delete m;
    return LUMEN_OK;
}

static int ensure_prefill_buffers(lumen_llama *m, int s, bool all_rows);
static int ensure_decode_graph(lumen_llama *m);

// layer_only: the state of a decode step without a model around it -- activations, RoPE tables, hand-over words,
// position counter, launch choices -- for the layer-level operator (lumen_decoder_layer_*): no weights, no caches, no
// logits, no prompt-pass buffers, no recorded step.
static int llama_create_impl(lumen_ctx *ctx, const lumen_llama_config *cfg, bool layer_only, lumen_llama **out) {
    if (!ctx || !cfg || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_create: null argument");
    *out = nullptr;
    const int H = cfg->hidden_size, I = cfg->intermediate_size, V = cfg->vocab_size, L = cfg->num_hidden_layers;
    const int Hq = cfg->num_attention_heads, Hkv = cfg->num_key_value_heads;
    if (H <= 0 || I <= 0 || V <= 0 || L <= 0 || Hq <= 0 || Hkv <= 0 || cfg->max_seq_len <= 0)
        LUMEN_FAIL(LUMEN_ERR_SHAPE, "llama_create: non-positive dimension");
    if (cfg->head_dim == 0 && H % Hq)  // self_attention.rs:69-73
        LUMEN_FAIL(LUMEN_ERR_SHAPE, "Embed dim must be divisible by n_head (%d %% %d)", H, Hq);
    if (Hq % Hkv) LUMEN_FAIL(LUMEN_ERR_SHAPE, "n_head %d not a multiple of n_kv_head %d", Hq, Hkv);
    if (cfg->weight_dtype != LUMEN_DTYPE_F32 && cfg->weight_dtype != LUMEN_DTYPE_BF16)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_create: weight_dtype %d", cfg->weight_dtype);
    const int D = cfg->head_dim > 0 ? cfg->head_dim : H / Hq;
    const int nrep = Hq / Hkv;
    if (!(D == 16 || D == 32 || D == 64 || D == 128))
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "head_dim %d outside the attention kernels (16, 32, 64, 128)", D);
    (void)nrep;
    if (H % 8 || I % 8 || (Hq * D) % 8)
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "hidden %d, intermediate %d and n_head*head_dim %d must be multiples of 8", H, I, Hq * D);
    if (H > 16384 || I > 16384 || Hq * D > 16384)
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "inner dimensions above 16384 do not fit the GEMV's LDS stage");
    HIP_TRY(hipSetDevice(ctx->device));

    lumen_llama *m = new lumen_llama();
    m->ctx = ctx; m->cfg = *cfg; m->D = D; m->qd = Hq * D; m->kvd = Hkv * D; m->qkvd = m->qd + 2 * m->kvd;
    m->bf16 = cfg->weight_dtype == LUMEN_DTYPE_BF16;
    m->esz = m->bf16 ? 2 : 4;
    m->scale = 1.0f / sqrtf((float)D);  // self_attention.rs:89 (sqrt().recip())
    m->layers.resize(L);
    m->layer_only = layer_only;
    int rc = LUMEN_OK;
#define M_TRY(e) do { rc = (e); if (rc != LUMEN_OK) { lumen_llama_destroy(m); return rc; } } while (0)
    if (!layer_only) {
    M_TRY(dmalloc_weight(m, (void **)&m->embed, (size_t)V * H * sizeof(float)));
    if (cfg->tie_embeddings && !m->bf16) {
        m->lm_head = m->embed;
    } else {
        M_TRY(dmalloc_weight(m, &m->lm_head, (size_t)V * H * m->esz));
        m->lm_head_owned = true;
    }
    M_TRY(dmalloc_t(m, &m->final_norm, (size_t)H));
    M_TRY(fill_ones(m, m->final_norm, H));  // RMSNorm::new, rms_norm.rs:14-20
    for (int l = 0; l < L; ++l) {
        LayerW &w = m->layers[l];
        M_TRY(dmalloc_weight(m, &w.wqkv, (size_t)m->qkvd * H * m->esz));
        M_TRY(dmalloc_weight(m, &w.wo, (size_t)H * m->qd * m->esz));
        M_TRY(dmalloc_weight(m, &w.wgu, (size_t)2 * I * H * m->esz));
        M_TRY(dmalloc_weight(m, &w.wdown, (size_t)H * I * m->esz));
        M_TRY(dmalloc_t(m, &w.in_norm, (size_t)H));
        M_TRY(dmalloc_t(m, &w.post_norm, (size_t)H));
        M_TRY(fill_ones(m, w.in_norm, H));
        M_TRY(fill_ones(m, w.post_norm, H));
        if (cfg->qk_norm) {
            M_TRY(dmalloc_t(m, &w.q_norm, (size_t)D));
            M_TRY(dmalloc_t(m, &w.k_norm, (size_t)D));
            M_TRY(fill_ones(m, w.q_norm, D));
            M_TRY(fill_ones(m, w.k_norm, D));
        }
    }
    }
    // one RoPE table for all layers (the reference builds an identical one per layer, self_attention.rs:78)
    {
        std::vector<float> c, s;
        rope_tables_host(c, s, D, cfg->max_seq_len, cfg->rope_theta);
        M_TRY(dmalloc_t(m, &m->cos_dev, c.size()));
        M_TRY(dmalloc_t(m, &m->sin_dev, s.size()));
        M_TRY(lumen_upload(ctx, m->cos_dev, c.data(), c.size() * sizeof(float)));
        M_TRY(lumen_upload(ctx, m->sin_dev, s.data(), s.size() * sizeof(float)));
    }
    // init_kv_caches(1), llama.rs:161-169: zero-filled [1,Hkv,max_seq,D] per layer
    m->cache_stride = (size_t)Hkv * cfg->max_seq_len * D;
    if (!layer_only) {
        M_TRY(dmalloc_t(m, &m->k_slab, m->cache_stride * L));
        M_TRY(dmalloc_t(m, &m->v_slab, m->cache_stride * L));
        if (hipMemsetAsync(m->k_slab, 0, m->cache_stride * L * sizeof(float), ctx->stream) != hipSuccess ||
            hipMemsetAsync(m->v_slab, 0, m->cache_stride * L * sizeof(float), ctx->stream) != hipSuccess) {
            lumen_llama_destroy(m);
            LUMEN_FAIL(LUMEN_ERR_HIP, "llama_create: clearing the KV slab failed");
        }
    }
    M_TRY(dmalloc_t(m, &m->x, (size_t)H));
    M_TRY(dmalloc_t(m, &m->h, (size_t)H));
    M_TRY(dmalloc_t(m, &m->qkv, (size_t)m->qkvd));
    M_TRY(dmalloc_t(m, &m->attn, (size_t)m->qd));
    M_TRY(dmalloc_t(m, &m->act, (size_t)I));
    if (!layer_only) M_TRY(dmalloc_t(m, &m->logits, (size_t)V));
    M_TRY(dmalloc_t(m, &m->d_tok, 4));
    M_TRY(dmalloc_t(m, &m->d_pos, 4));
    if (!layer_only) M_TRY(dmalloc_t(m, &m->tok_hist, (size_t)cfg->max_seq_len + 1));
    m->nsplit = attn_decode_nsplit(cfg->max_seq_len, D);
    // Where a cache is cut into 2 to 16 slices the o_proj GEMV can fold the slices' partial states while it
    // stages its input: an atomic and a second round of loads fewer inside the attention kernel.  With more
    // slices the partials would outweigh what the GEMV workgroups can re-read.  q/k norm models rotate
    // inside the attention kernel: not covered.  Used on the long side of the short-cache boundary only.
    // Leaving the merge of the slices to the o_proj GEMV makes every one of its workgroups read every
    // slice's state of every element out of L2: it pays while that stays a few tens of MB (33 MB for a
    // 2048-wide model: 1.13 -> 1.09 ms per token at 4000 rows; 268 MB for a 4096-wide one with 32 KV
    // heads, where o_proj went from 8 to 24 us)
    const size_t fold_bytes = (size_t)gemv_grid(ctx, H, m->qd, m->bf16, EPI_RESIDUAL, nullptr) * (size_t)m->qd *
                              GEMV_FOLD_MAX_SLICES * sizeof(float);
    m->defer_merge = m->nsplit >= 2 && m->nsplit <= GEMV_FOLD_MAX_SLICES && !cfg->qk_norm &&
                     cfg->max_seq_len <= m->nsplit * attn_decode_trip_rows(D) && fold_bytes <= ((size_t)64 << 20);
    M_TRY(dmalloc_t(m, &m->part, attn_decode_part_floats(1, Hq, D, m->nsplit)));
    M_TRY(dmalloc_t(m, &m->part_merge, attn_decode_part_floats(1, Hq, D, m->nsplit)));
    // (q/k-norm models rotate inside the attention role: only the three-role form serves them)
    m->chain_ao = qkv_attn_oproj_supported(Hq, Hkv, D, H, m->qd, m->bf16, cfg->qk_norm)                 ? 2
                  : (!cfg->qk_norm && attn_oproj_supported(Hq, Hkv, D, H, m->qd, m->bf16)) ? 1
                                                                                           : 0;
    // The chain pays where its products are latency: every role at most one workgroup per compute unit (hidden and
    // q|k|v rows up to ~2048-4096).  Larger products stream better as launches of their own (Llama-2-7B shape: 2.73
    // against 2.95 ms per token); lumen_llama_set_handover can still switch the chain on.
    if (m->chain_ao == 2 && m->qkvd / 16 > ctx->num_cus) m->chain_ao = cfg->qk_norm ? 0 : 1;
    if (m->chain_ao && (H + 7) / 8 > ctx->num_cus) m->chain_ao = 0;
    // the o_proj workgroups hold their weight requests back until q has changed hands, which takes longer the more
    // q|k|v weights stream in front (measured optima: 5.4-5.7 us at 21 MB, 4.5-4.7 us at 17 MB)
    m->chain_pre[2] = 25 + (int)(1.45 * (double)((size_t)m->qkvd * H * m->esz) / 1e6);
    // (every role of the MLP chain at most ... two rounds of workgroups: the products of a narrow model)
    m->chain_mlp = mlp_chain_supported(H, I, m->bf16) && mlp_chain_workgroups(H, I) <= 2 * ctx->num_cus;
    M_TRY(dmalloc_t(m, &m->act_tagged, (size_t)I));
    M_TRY(dmalloc_t(m, &m->x_tagged, (size_t)m->qd));
    M_TRY(dmalloc_t(m, &m->qkv_tagged, (size_t)m->qkvd));
    M_TRY(dmalloc_t(m, &m->part_tagged, (size_t)Hq * ATTN_CHAIN_MAX_SLICES * (D + 2) + 2));
    M_TRY(dmalloc_t(m, &m->d_step, 4));
    M_TRY(dmalloc_t(m, &m->d_err, 4));
    if (hipMemsetAsync(m->x_tagged, 0, sizeof(unsigned long long) * m->qd, ctx->stream) != hipSuccess ||
        hipMemsetAsync(m->qkv_tagged, 0, sizeof(unsigned long long) * m->qkvd, ctx->stream) != hipSuccess ||
        hipMemsetAsync(m->act_tagged, 0, sizeof(unsigned long long) * I, ctx->stream) != hipSuccess ||
        hipMemsetAsync(m->part_tagged, 0, sizeof(unsigned long long) * ((size_t)Hq * ATTN_CHAIN_MAX_SLICES * (D + 2) + 2), ctx->stream) != hipSuccess ||
        hipMemsetAsync(m->d_step, 0, 4 * sizeof(unsigned), ctx->stream) != hipSuccess ||
        hipMemsetAsync(m->d_err, 0, 4 * sizeof(int), ctx->stream) != hipSuccess) {
        lumen_llama_destroy(m);
        LUMEN_FAIL(LUMEN_ERR_HIP, "llama_create: clearing the hand-over state failed");
    }
    if (hipMemsetAsync(m->part_merge, 0, sizeof(unsigned long long) * attn_decode_part_floats(1, Hq, D, m->nsplit), ctx->stream) != hipSuccess ||
        hipMemsetAsync(m->d_tok, 0, 4 * sizeof(int), ctx->stream) != hipSuccess ||
        hipMemsetAsync(m->d_pos, 0, 4 * sizeof(int), ctx->stream) != hipSuccess ||
        hipStreamSynchronize(ctx->stream) != hipSuccess) {
        lumen_llama_destroy(m);
        LUMEN_FAIL(LUMEN_ERR_HIP, "llama_create: clearing decode state failed");
    }
    {
        const size_t nb = (size_t)std::max(gemv_max_blocks(ctx), ctx->num_cus);
        M_TRY(dmalloc_t(m, &m->amax_word, nb));
        M_TRY(dmalloc_t(m, &m->amax_epoch, 4));
        if (hipMemsetAsync(m->amax_word, 0, nb * sizeof(unsigned long long), ctx->stream) != hipSuccess ||
            hipMemsetAsync(m->amax_epoch, 0, 4 * sizeof(unsigned), ctx->stream) != hipSuccess ||
            hipStreamSynchronize(ctx->stream) != hipSuccess) {
            lumen_llama_destroy(m);
            LUMEN_FAIL(LUMEN_ERR_HIP, "llama_create: clearing the arg-max candidates failed");
        }
    }
    m->decode_mode = LUMEN_DECODE_GRAPH;
    if (layer_only) {
        m->decode_mode = LUMEN_DECODE_EAGER;
        // (its launches are not followed by a call of this library that synchronises: a wait that runs out is flagged
        // where lumen_ctx_synchronize / lumen_download find it)
        m->d_err = ctx->err_host;
    } else {
        // buffers of a prompt pass of up to 512 rows now, not under the first prompt (longer prompts grow them)
        M_TRY(ensure_prefill_buffers(m, std::min(cfg->max_seq_len, 512), false));
        // ... and the decode step recorded and instantiated for a short cache (recorded again when the cache outgrows it)
        M_TRY(ensure_decode_graph(m));
        if (m->graph_exec) hipGraphUpload(m->graph_exec, ctx->stream);
    }
    if (hipStreamSynchronize(ctx->stream) != hipSuccess) {
        lumen_llama_destroy(m);
        LUMEN_FAIL(LUMEN_ERR_HIP, "llama_create: preparing the decode graph failed");
    }
#undef M_TRY
    *out = m;
    return LUMEN_OK;
}

extern "C" int lumen_llama_create(lumen_ctx *ctx, const lumen_llama_config *cfg, lumen_llama **out) {
    return llama_create_impl(ctx, cfg, false, out);
}

// ----------------------------------------------------------- parameter upload
static void f32_to_bf16_host(const float *src, uint16_t *dst, size_t n) {
    for (size_t i = 0; i < n; ++i) {
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

static void bf16_to_f32_host(const uint16_t *src, float *dst, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        const uint32_t u = (uint32_t)src[i] << 16;  // half::bf16::to_f32, src/loader.rs:58
        memcpy(dst + i, &u, 4);
    }
}

// Copies a [rows, cols] host matrix (src dtype) into device memory of dst dtype
// whose row r lands at dst + (row0 + r*row_step) * cols.
static int upload_matrix(lumen_llama *m, void *dst, bool dst_bf16, const void *src, int src_dtype, size_t rows,
                         size_t cols, size_t row0, size_t row_step) {
    const size_t dsz = dst_bf16 ? 2 : 4;
    const bool src_bf16 = src_dtype == LUMEN_DTYPE_BF16;
    const size_t chunk_rows = std::max<size_t>(1, (size_t)(64u << 20) / (cols * 4));
    std::vector<char> stage;
    for (size_t r0 = 0; r0 < rows; r0 += chunk_rows) {
        const size_t nr = std::min(chunk_rows, rows - r0);
        const void *p;
        if (src_bf16 == dst_bf16) {
            p = (const char *)src + r0 * cols * dsz;
        } else {
            stage.resize(nr * cols * dsz);
            if (dst_bf16) f32_to_bf16_host((const float *)src + r0 * cols, (uint16_t *)stage.data(), nr * cols);
            else bf16_to_f32_host((const uint16_t *)src + r0 * cols, (float *)stage.data(), nr * cols);
            p = stage.data();
        }
        char *d = (char *)dst + (row0 + r0 * row_step) * cols * dsz;
        HIP_TRY(hipMemcpy2DAsync(d, row_step * cols * dsz, p, cols * dsz, cols * dsz, nr, hipMemcpyHostToDevice,
                                 m->ctx->stream));
        HIP_TRY(hipStreamSynchronize(m->ctx->stream));
    }
    return LUMEN_OK;
}

static int want_shape(const char *name, const int64_t *shape, int ndim, int64_t a, int64_t b) {
    const bool ok = (b < 0) ? (ndim == 1 && shape[0] == a) : (ndim == 2 && shape[0] == a && shape[1] == b);
    if (!ok) {
        if (b < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "Shape mismatch for %s: expected [%lld]", name, (long long)a);
        LUMEN_FAIL(LUMEN_ERR_SHAPE, "Shape mismatch for %s: expected [%lld, %lld]", name, (long long)a, (long long)b);
    }
    return LUMEN_OK;
}

extern "C" int lumen_llama_set_param(lumen_llama *m, const char *name, const void *data, int dtype,
                                     const int64_t *shape, int ndim) {
    if (!m || !name || !data || !shape) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_set_param: null argument");
    if (dtype != LUMEN_DTYPE_F32 && dtype != LUMEN_DTYPE_BF16)  // loader.rs:67
        LUMEN_FAIL(LUMEN_ERR_INVALID, "Unsupported dtype: %d for %s", dtype, name);
    const lumen_llama_config &c = m->cfg;
    const int H = c.hidden_size, I = c.intermediate_size, V = c.vocab_size;
    const std::string n(name);
    if (n == "model.embed_tokens.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, V, H));
        LUMEN_TRY(upload_matrix(m, m->embed, false, data, dtype, V, H, 0, 1));
        if (c.tie_embeddings && m->lm_head_owned) return upload_matrix(m, m->lm_head, m->bf16, data, dtype, V, H, 0, 1);
        return LUMEN_OK;
    }
    if (n == "lm_head.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, V, H));
        if (c.tie_embeddings) LUMEN_FAIL(LUMEN_ERR_INVALID, "lm_head.weight given but embeddings are tied");
        return upload_matrix(m, m->lm_head, m->bf16, data, dtype, V, H, 0, 1);
    }
    if (n == "model.norm.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, H, -1));
        return upload_matrix(m, m->final_norm, false, data, dtype, 1, H, 0, 1);
    }
    int layer = -1, consumed = 0;
    if (sscanf(name, "model.layers.%d.%n", &layer, &consumed) != 1 || consumed == 0 || layer < 0 ||
        layer >= c.num_hidden_layers)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "Parameter %s not found in model", name);
    const std::string rest(name + consumed);
    LayerW &w = m->layers[layer];
    if (rest == "self_attn.q_proj.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, m->qd, H));
        return upload_matrix(m, w.wqkv, m->bf16, data, dtype, m->qd, H, 0, 1);
    }
    if (rest == "self_attn.k_proj.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, m->kvd, H));
        return upload_matrix(m, w.wqkv, m->bf16, data, dtype, m->kvd, H, m->qd, 1);
    }
    if (rest == "self_attn.v_proj.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, m->kvd, H));
        return upload_matrix(m, w.wqkv, m->bf16, data, dtype, m->kvd, H, m->qd + m->kvd, 1);
    }
    if (rest == "self_attn.o_proj.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, H, m->qd));
        return upload_matrix(m, w.wo, m->bf16, data, dtype, H, m->qd, 0, 1);
    }
    if (rest == "mlp.gate_proj.weight") {  // row i -> fused row 2i
        LUMEN_TRY(want_shape(name, shape, ndim, I, H));
        return upload_matrix(m, w.wgu, m->bf16, data, dtype, I, H, 0, 2);
    }
    if (rest == "mlp.up_proj.weight") {  // row i -> fused row 2i+1
        LUMEN_TRY(want_shape(name, shape, ndim, I, H));
        return upload_matrix(m, w.wgu, m->bf16, data, dtype, I, H, 1, 2);
    }
    if (rest == "mlp.down_proj.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, H, I));
        return upload_matrix(m, w.wdown, m->bf16, data, dtype, H, I, 0, 1);
    }
    if (rest == "input_layernorm.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, H, -1));
        return upload_matrix(m, w.in_norm, false, data, dtype, 1, H, 0, 1);
    }
    if (rest == "post_attention_layernorm.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, H, -1));
        return upload_matrix(m, w.post_norm, false, data, dtype, 1, H, 0, 1);
    }
    if (c.qk_norm && rest == "self_attn.q_norm.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, m->D, -1));
        return upload_matrix(m, w.q_norm, false, data, dtype, 1, m->D, 0, 1);
    }
    if (c.qk_norm && rest == "self_attn.k_norm.weight") {
        LUMEN_TRY(want_shape(name, shape, ndim, m->D, -1));
        return upload_matrix(m, w.k_norm, false, data, dtype, 1, m->D, 0, 1);
    }
    LUMEN_FAIL(LUMEN_ERR_INVALID, "Parameter %s not found in model", name);
}

// Names and shapes of the model's parameters, LlamaModel::named_parameters (llama.rs:218-279),
// plus the per-head q/k norm gains of the Qwen3 extension; no lm_head when it is tied.
int lumen_llama_param_list(const lumen_llama *m, std::vector<std::string> &names,
                           std::vector<std::vector<int64_t>> &shapes) {
    if (!m) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_param_list: null model");
    const lumen_llama_config &c = m->cfg;
    const int64_t H = c.hidden_size, I = c.intermediate_size, V = c.vocab_size;
    auto add = [&](const std::string &n, std::vector<int64_t> sh) {
        names.push_back(n);
        shapes.push_back(sh);
    };
    add("model.embed_tokens.weight", {V, H});
    for (int l = 0; l < c.num_hidden_layers; ++l) {
        const std::string p = "model.layers." + std::to_string(l) + ".";
        add(p + "self_attn.q_proj.weight", {m->qd, H});
        add(p + "self_attn.k_proj.weight", {m->kvd, H});
        add(p + "self_attn.v_proj.weight", {m->kvd, H});
        add(p + "self_attn.o_proj.weight", {H, m->qd});
        add(p + "mlp.gate_proj.weight", {I, H});
        add(p + "mlp.up_proj.weight", {I, H});
        add(p + "mlp.down_proj.weight", {H, I});
        add(p + "input_layernorm.weight", {H});
        add(p + "post_attention_layernorm.weight", {H});
        if (c.qk_norm) {
            add(p + "self_attn.q_norm.weight", {m->D});
            add(p + "self_attn.k_norm.weight", {m->D});
        }
    }
    add("model.norm.weight", {H});
    if (!c.tie_embeddings) add("lm_head.weight", {V, H});
    return LUMEN_OK;
}

// ------------------------------------------------------------------- decode
// One token through all layers; every launch reads the token id and the
// position from device memory, so the sequence is the same for every token.
// Kernel classes of a decode step, for per-kernel timing.
enum { KC_EMBED = 0, KC_QKV, KC_ATTN, KC_OPROJ, KC_GATEUP, KC_DOWN, KC_LMHEAD, KC_ARGMAX, KC_ATTN_OPROJ, KC_MLP, KC_COUNT };

struct StepProbe {  // brackets every launch with a HIP event pair when profiling, and keeps the kernel's name
    std::vector<hipEvent_t> ev;
    std::vector<int> cls;
    hipStream_t s = nullptr;
    bool on = false;
    lumen_ctx *ctx = nullptr;
    std::string *names = nullptr;  // [KC_COUNT]
    void before(int c) {
        if (!on) return;
        hipEvent_t e0, e1;
        hipEventCreate(&e0);
        hipEventCreate(&e1);
        ev.push_back(e0);
        ev.push_back(e1);
        cls.push_back(c);
        hipEventRecord(e0, s);
    }
    void after() {
        if (!on) return;
        hipEventRecord(ev.back(), s);
        if (names && ctx) names[cls.back()] = ctx->last_kernel;
    }
};

// Is the cache short enough for the one-workgroup-per-head form of decode attention?  A hint for the
// kernel (it starts that form before it has read the position); a wrong one only costs time.
static int expect_short_cache(const lumen_llama *m) { return m->len + 1 <= attn_decode_short_rows(m->D); }

// Attention workgroups per query head of the chained launch for the step at the current length, and the rows each
// takes.  Up to two trips of rows one workgroup walks them in turn (a second trip costs what handing a slice's
// state on would); up to four trips the slices are one trip each, beyond that two -- more, shorter slices mean more
// workgroups than the chip holds at once.  The count is rounded up to a power of two so that a captured step
// serves a range of lengths.  0: the cache is too long for the chain (or the model has none): separate launches.
static int chain_slices(const lumen_llama *m, int *slice_rows_out = nullptr) {
    if (!m->chain_ao) return 0;
    const int T = attn_decode_trip_rows(m->D);
    const int trips = m->len / T + 1;
    int per = trips <= 2 ? 2 : trips <= 4 ? 1 : 2;
    if (m->chain_slice_trips > 0) per = m->chain_slice_trips;
    const int need = trips <= 2 && m->chain_slice_trips <= 0 ? 1 : (trips + per - 1) / per;
    int s = 1;
    while (s < need) s *= 2;
    if (slice_rows_out) *slice_rows_out = per * T;
    return s <= m->chain_max_slices ? s : 0;
}

// what a captured step depends on: slices and rows per slice
static int chain_plan_key(const lumen_llama *m) {
    int rows = 0;
    const int s = chain_slices(m, &rows);
    return s ? s * 65536 + rows : 0;
}

// One decoder layer of a decode step, LlamaDecoderLayer::forward_infer for S == 1 (src/models/llama.rs:104-116):
// three launches (two for narrow models, five where no chain applies).  x_in [H] is the layer input -- or, with
// row_sel, row *row_sel of the table x_in points at (the embedding gather of llama.rs:191 folded into the first
// layer) --, y_out [H] its output (may be x_in); k_cache / v_cache the layer's cache [Hkv, max_seq, D]; the new
// token's position is *m->d_pos; tag_slot < tag_mul tells the launches of one step apart (their hand-over tags are
// *d_step * tag_mul + tag_slot + 1).
static int enqueue_decoder_layer(lumen_llama *m, const LayerW &w, float *k_cache, float *v_cache, const float *x_in,
                                 const int *row_sel, float *y_out, unsigned tag_mul, unsigned tag_slot, StepProbe *pr) {
    lumen_ctx *ctx = m->ctx;
    const lumen_llama_config &c = m->cfg;
    const int H = c.hidden_size, I = c.intermediate_size;
    // RoPE + KV append ride on the q|k|v product unless q/k need a per-head norm first.
    const bool fuse_rope = !c.qk_norm;
    GemvArgs g = {};
    // input_layernorm + q|k|v projections, llama.rs:107, self_attention.rs:106-108
    g.W = w.wqkv; g.x = x_in; g.y = m->qkv; g.N = m->qkvd; g.K = H; g.w_bf16 = m->bf16;
    g.pro = PRO_RMSNORM; g.norm_w = w.in_norm; g.eps = c.rms_norm_eps; g.epi = EPI_STORE;
    if (row_sel) { g.row_sel = row_sel; g.row_stride = H; g.x_sel = 1; }
    if (fuse_rope) {
        g.epi = EPI_ROPE_QKV; g.cos_t = m->cos_dev; g.sin_t = m->sin_dev; g.pos = m->d_pos;
        g.k_cache = k_cache; g.v_cache = v_cache;
        g.hq = c.num_attention_heads; g.hkv = c.num_key_value_heads; g.D = m->D; g.max_seq = c.max_seq_len;
    }
    int slice_rows = 0;
    const int slices = chain_slices(m, &slice_rows);
    const bool chain_short = slices > 0;
    const bool chain_qkv = chain_short && m->chain_ao > 1;
    if (!chain_qkv) {
        pr->before(KC_QKV);
        LUMEN_TRY(launch_gemv(ctx, g));
        pr->after();
    }
    AttnDecodeArgs a = {};
    a.q = m->qkv; a.k_new = m->qkv + m->qd; a.v_new = m->qkv + m->qd + m->kvd; a.out = m->attn;
    a.k_cache = k_cache; a.v_cache = v_cache;
    a.cos_t = m->cos_dev; a.sin_t = m->sin_dev; a.pos_dev = m->d_pos; a.pos_host = 0;
    a.b = 1; a.hq = c.num_attention_heads; a.hkv = c.num_key_value_heads; a.d = m->D; a.max_seq = c.max_seq_len;
    a.scale = m->scale; a.q_norm_w = w.q_norm; a.k_norm_w = w.k_norm; a.norm_eps = c.rms_norm_eps;
    a.part = m->part; a.nsplit = m->nsplit; a.pre_rotated = fuse_rope;
    // (slices merged inside the attention launch: tagged words, the tag made of the step counter like the chains')
    a.part_tagged = m->part_merge; a.tag_dev = m->d_step; a.tag_mul = tag_mul; a.tag_add = tag_slot + 1u;
    a.spin_limit = m->spin_limit; a.err_dev = m->d_err;
    a.expect_short = expect_short_cache(m);
    // (a graph is captured anew when the cache crosses the short / long boundary, so the choices below are the
    // same for every launch of a step)
    if (chain_short) {
        // short caches: (q|k|v,) attention and o_proj + residual chained in one launch
        AttnOprojArgs f = {};
        f.attn = a;
        f.attn.out_tagged = m->x_tagged;
        f.Wo = w.wo; f.residual = x_in; f.y = m->h; f.N = H; f.K = m->qd; f.w_bf16 = m->bf16;
        if (row_sel) { f.row_sel = row_sel; f.row_stride = H; }
        f.x_tagged = m->x_tagged; f.step_dev = m->d_step;
        f.tag_mul = tag_mul; f.tag_add = tag_slot + 1u;
        f.err_dev = m->d_err; f.spin_limit = m->spin_limit;
        f.pre_sleep = m->chain_pre[m->chain_ao]; f.poll_delay = m->chain_delay[m->chain_ao]; f.poll_gap = m->chain_gap[m->chain_ao];
        // (the fold of the slices is one more hand-over in front of o_proj, and two-trip slices take a trip longer:
        // polling earlier only puts polls in the way of those hand-overs; measured optima, 1.7 / 3.7 us)
        if (slices > 1) f.poll_delay += slice_rows > attn_decode_trip_rows(m->D) ? 37 : 17;
        f.nslices = slices; f.slice_rows = slice_rows; f.part_tagged = m->part_tagged;
        f.t0_tagged = m->part_tagged + (size_t)c.num_attention_heads * ATTN_CHAIN_MAX_SLICES * (m->D + 2);  // (one word behind the states)
        if (chain_qkv) {
            f.Wqkv = w.wqkv; f.in_norm_w = w.in_norm; f.norm_eps = c.rms_norm_eps; f.qkv_tagged = m->qkv_tagged;
        }
        pr->before(KC_ATTN_OPROJ);
        LUMEN_TRY(launch_attn_oproj(ctx, f));
        pr->after();
    } else {
        const bool defer = m->defer_merge && !a.expect_short;
        a.defer_merge = defer;
        pr->before(KC_ATTN);
        LUMEN_TRY(launch_attn_decode(ctx, a));
        pr->after();
        // o_proj + residual, self_attention.rs:303, llama.rs:110
        g = {};
        g.W = w.wo; g.x = m->attn; g.y = m->h; g.N = H; g.K = m->qd; g.w_bf16 = m->bf16;
        g.pro = PRO_NONE; g.epi = EPI_RESIDUAL; g.residual = x_in;
        if (defer) {
            g.pro = PRO_ATTN_FOLD; g.attn_part = m->part; g.attn_pos = m->d_pos; g.attn_nslices = m->nsplit; g.attn_d = m->D;
            g.attn_trip = attn_decode_trip_rows(m->D); g.attn_short_rows = attn_decode_short_rows(m->D);
        }
        if (row_sel) { g.row_sel = row_sel; g.row_stride = H; g.residual_sel = 1; }
        pr->before(KC_OPROJ);
        LUMEN_TRY(launch_gemv(ctx, g));
        pr->after();
    }
    if (m->chain_mlp && m->chain_ao_on) {
        // narrow models: post_attention_layernorm + gate|up + silu*up + down + residual as one launch
        MlpChainArgs mc = {};
        mc.Wgu = w.wgu; mc.h = m->h; mc.norm_w = w.post_norm; mc.eps = c.rms_norm_eps; mc.Wdown = w.wdown; mc.y = y_out;
        mc.N = H; mc.I = I; mc.w_bf16 = m->bf16; mc.act_tagged = m->act_tagged; mc.step_dev = m->d_step;
        mc.tag_mul = tag_mul; mc.tag_add = tag_slot + 1u;
        mc.err_dev = m->d_err; mc.spin_limit = m->spin_limit;
        mc.pre_sleep = m->mlp_pre; mc.poll_delay = m->mlp_delay; mc.poll_gap = m->mlp_gap;
        pr->before(KC_MLP);
        LUMEN_TRY(launch_mlp_chain(ctx, mc));
        pr->after();
        return LUMEN_OK;
    }
    // post_attention_layernorm + gate|up + silu*up, llama.rs:113, :60-63
    g = {};
    g.W = w.wgu; g.x = m->h; g.y = m->act; g.N = 2 * I; g.K = H; g.w_bf16 = m->bf16;
    g.pro = PRO_RMSNORM; g.norm_w = w.post_norm; g.eps = c.rms_norm_eps; g.epi = EPI_SWIGLU;
    pr->before(KC_GATEUP);
    LUMEN_TRY(launch_gemv(ctx, g));
    pr->after();
    // down_proj + residual, llama.rs:64, :115
    g = {};
    g.W = w.wdown; g.x = m->act; g.y = y_out; g.N = H; g.K = I; g.w_bf16 = m->bf16;
    g.pro = PRO_NONE; g.epi = EPI_RESIDUAL; g.residual = m->h;
    pr->before(KC_DOWN);
    LUMEN_TRY(launch_gemv(ctx, g));
    pr->after();
    return LUMEN_OK;
}

static int enqueue_decode_step(lumen_llama *m, StepProbe *pr = nullptr) {
    StepProbe none;
    if (!pr) pr = &none;
    lumen_ctx *ctx = m->ctx;
    const lumen_llama_config &c = m->cfg;
    const int H = c.hidden_size, V = c.vocab_size;
    // Embedding::forward (llama.rs:191) is folded into the first layer: its launches read row *d_tok of the table
    for (int l = 0; l < c.num_hidden_layers; ++l)
        LUMEN_TRY(enqueue_decoder_layer(m, m->layers[l], m->k_slab + m->cache_stride * l, m->v_slab + m->cache_stride * l,
                                        l == 0 ? m->embed : m->x, l == 0 ? m->d_tok : nullptr, m->x,
                                        (unsigned)c.num_hidden_layers, (unsigned)l, pr));
    // final norm + lm_head, llama.rs:202-205
    GemvArgs g = {};
    g.W = m->lm_head; g.x = m->x; g.y = m->logits; g.N = V; g.K = H;
    g.w_bf16 = (m->lm_head == (void *)m->embed) ? 0 : (int)m->bf16;
    g.pro = PRO_RMSNORM; g.norm_w = m->final_norm; g.eps = c.rms_norm_eps;
    // the greedy pick is folded in: it becomes the next token id and the position counter advances
    g.epi = EPI_ARGMAX; g.amax_word = m->amax_word; g.amax_epoch = m->amax_epoch; g.err_dev = m->d_err; g.spin_limit = m->spin_limit;
    g.tok_out = m->d_tok; g.pos_inc = m->d_pos; g.tok_hist = m->tok_hist; g.step_inc = m->d_step;
    pr->before(KC_LMHEAD);
    const int rc = launch_gemv(ctx, g);
    pr->after();
    return rc;
}

static int ensure_decode_graph(lumen_llama *m) {
    if (m->decode_mode != LUMEN_DECODE_GRAPH) return LUMEN_OK;
    if (m->graph_exec && (m->graph_expect_short != expect_short_cache(m) || m->graph_slices != chain_plan_key(m))) {
        // the captured attention launches carry the hint for the other side of the boundary
        HIP_TRY(hipStreamSynchronize(m->ctx->stream));
        hipGraphExecDestroy(m->graph_exec);
        hipGraphDestroy(m->graph);
        m->graph_exec = nullptr;
        m->graph = nullptr;
    }
    if (m->graph_exec) return LUMEN_OK;
    m->graph_expect_short = expect_short_cache(m);
    m->graph_slices = chain_plan_key(m);
    hipStream_t s = m->ctx->stream;
    HIP_TRY(hipStreamSynchronize(s));
    HIP_TRY(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    const int rc = enqueue_decode_step(m);
    hipGraph_t g = nullptr;
    const hipError_t e = hipStreamEndCapture(s, &g);
    if (rc != LUMEN_OK) {
        if (g) hipGraphDestroy(g);
        return rc;
    }
    if (e != hipSuccess) LUMEN_FAIL(LUMEN_ERR_HIP, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
    const hipError_t ei = hipGraphInstantiate(&m->graph_exec, g, nullptr, nullptr, 0);
    if (ei != hipSuccess) {
        hipGraphDestroy(g);
        m->graph_exec = nullptr;
        LUMEN_FAIL(LUMEN_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(ei));
    }
    m->graph = g;
    return LUMEN_OK;
}

// one decode step: a graph replay, or the same launches one by one
static hipError_t launch_step(lumen_llama *m) {
    if (m->decode_mode == LUMEN_DECODE_GRAPH) return hipGraphLaunch(m->graph_exec, m->ctx->stream);
    return enqueue_decode_step(m) == LUMEN_OK ? hipSuccess : hipErrorLaunchFailure;
}

extern "C" int lumen_llama_set_decode_mode(lumen_llama *m, int mode) {
    if (!m) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_set_decode_mode: null model");
    if (mode != LUMEN_DECODE_EAGER && mode != LUMEN_DECODE_GRAPH && mode != LUMEN_DECODE_PERSISTENT)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_set_decode_mode: unknown mode %d", mode);
    if (mode == LUMEN_DECODE_PERSISTENT)
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED,
                   "this library holds no persistent decode kernel (a grid-wide hand-over costs more on this chip "
                   "than the kernel boundary it would replace); use LUMEN_DECODE_GRAPH");
    m->decode_mode = mode;
    return LUMEN_OK;
}

extern "C" int lumen_llama_set_handover(lumen_llama *m, int enable, int64_t spin_limit, int pre_sleep, int poll_delay, int poll_gap) {
    if (!m) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_set_handover: null model");
    if (enable == 1 && (m->cfg.qk_norm || !attn_oproj_supported(m->cfg.num_attention_heads, m->cfg.num_key_value_heads, m->D,
                                                                m->cfg.hidden_size, m->qd, m->bf16)))
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "the attention -> o_proj launch does not cover this model shape");
    if (enable > 1 && !qkv_attn_oproj_supported(m->cfg.num_attention_heads, m->cfg.num_key_value_heads, m->D, m->cfg.hidden_size,
                                                m->qd, m->bf16, m->cfg.qk_norm))
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "the q|k|v -> attention -> o_proj launch does not cover this model shape");
    if (spin_limit > (int64_t)HANDOVER_MAX_SPINS || pre_sleep > HANDOVER_MAX_TENTHS || poll_delay > HANDOVER_MAX_TENTHS ||
        poll_gap > HANDOVER_MAX_GAP)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_set_handover: spin_limit at most %u, pre_sleep and poll_delay at most %d "
                                      "(tenths of a microsecond), poll_gap at most %d", HANDOVER_MAX_SPINS,
                   HANDOVER_MAX_TENTHS, HANDOVER_MAX_GAP);
    if (enable >= 0) {
        m->chain_ao = enable > 2 ? 2 : enable;
        m->chain_ao_on = enable > 0;  // (enable 0 also takes the MLP chain of narrow models apart)
    }
    if (spin_limit >= 0) m->spin_limit = (unsigned)spin_limit;
    if (pre_sleep >= 0) m->chain_pre[m->chain_ao] = pre_sleep;
    if (poll_delay >= 0) m->chain_delay[m->chain_ao] = poll_delay;
    if (poll_gap >= 0) m->chain_gap[m->chain_ao] = poll_gap;
    // the captured step carries the old choice
    if (m->graph_exec) {
        HIP_TRY(hipStreamSynchronize(m->ctx->stream));
        hipGraphExecDestroy(m->graph_exec);
        hipGraphDestroy(m->graph);
        m->graph_exec = nullptr;
        m->graph = nullptr;
    }
    return LUMEN_OK;
}

extern "C" int lumen_llama_get_decode_mode(const lumen_llama *m, int *mode_out) {
    if (!m || !mode_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_get_decode_mode: null argument");
    *mode_out = m->decode_mode;
    return LUMEN_OK;
}

// after a synchronisation: did a wait inside the attention -> o_proj chain run into its limit?
static int check_handover(lumen_llama *m) {
    int err = 0;
    HIP_TRY(hipMemcpy(&err, m->d_err, sizeof(int), hipMemcpyDeviceToHost));
    if (!err) return LUMEN_OK;
    HIP_TRY(hipMemset(m->d_err, 0, sizeof(int)));
    LUMEN_FAIL(LUMEN_ERR_HIP, "decode: a workgroup gave up waiting for a value handed over inside a launch (poll "
                              "limit %u); the results of this call are invalid, reset the model", m->spin_limit);
}

static int sync_pos_to_device(lumen_llama *m) {
    HIP_TRY(hipMemcpyAsync(m->d_pos, &m->len, sizeof(int), hipMemcpyHostToDevice, m->ctx->stream));
    HIP_TRY(hipStreamSynchronize(m->ctx->stream));
    return LUMEN_OK;
}

static int check_room(const lumen_llama *m, int add) {
    if (m->len + add > m->cfg.max_seq_len)  // self_attention.rs:144-149, 341-346
        LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "KV cache overflow: new_len=%d > max_seq=%d", m->len + add, m->cfg.max_seq_len);
    return LUMEN_OK;
}

static int ids_to_int(const lumen_llama *m, const float *ids, int s, std::vector<int> &out) {
    out.resize(s);
    for (int t = 0; t < s; ++t) {
        const float f = ids[t];
        const long long idx = (f > 0.0f) ? (f >= 9.0e18f ? (long long)9e18 : (long long)f) : 0;  // `as usize`
        if (idx >= m->cfg.vocab_size)  // embedding.rs:55
            LUMEN_FAIL(LUMEN_ERR_EMBED_OOB, "Embedding index out of bounds: %lld >= %d", idx, m->cfg.vocab_size);
        out[t] = (int)idx;
    }
    return LUMEN_OK;
}

// ------------------------------------------------------------------ prefill
static int ensure_prefill_buffers(lumen_llama *m, int s, bool all_rows) {
    const lumen_llama_config &c = m->cfg;
    if (s > m->pf_cap) {
        HIP_TRY(hipStreamSynchronize(m->ctx->stream));
        hipFree(m->p_x); hipFree(m->p_h); hipFree(m->p_n); hipFree(m->p_qkv); hipFree(m->p_qrot);
        hipFree(m->p_attn); hipFree(m->p_act); hipFree(m->p_ids);
        m->p_x = m->p_h = m->p_n = m->p_qkv = m->p_qrot = m->p_attn = m->p_act = nullptr;
        m->p_ids = nullptr;
        m->pf_cap = 0;
        const size_t S = (size_t)s;
        HIP_TRY(hipMalloc((void **)&m->p_x, S * c.hidden_size * 4));
        HIP_TRY(hipMalloc((void **)&m->p_h, S * c.hidden_size * 4));
        HIP_TRY(hipMalloc((void **)&m->p_n, S * c.hidden_size * 4));
        HIP_TRY(hipMalloc((void **)&m->p_qkv, S * m->qkvd * 4));
        HIP_TRY(hipMalloc((void **)&m->p_qrot, S * m->qd * 4));
        HIP_TRY(hipMalloc((void **)&m->p_attn, S * m->qd * 4));
        HIP_TRY(hipMalloc((void **)&m->p_act, S * c.intermediate_size * 4));
        HIP_TRY(hipMalloc((void **)&m->p_ids, S * sizeof(int)));
        m->pf_cap = s;
        // the split-K workspace of the four products at this many rows, so that no launch has to grow it
        const int H = c.hidden_size, I = c.intermediate_size;
        size_t ws = gemm_workspace_bytes(m->ctx, s, m->qkvd, H, m->bf16);
        ws = std::max(ws, gemm_workspace_bytes(m->ctx, s, H, m->qd, m->bf16));
        ws = std::max(ws, gemm_workspace_bytes(m->ctx, s, 2 * I, H, m->bf16));
        ws = std::max(ws, gemm_workspace_bytes(m->ctx, s, H, I, m->bf16));
        if (ws) LUMEN_TRY(gemm_reserve_workspace(m->ctx, ws));
    }
    if (all_rows && s > m->pf_logit_cap) {
        HIP_TRY(hipStreamSynchronize(m->ctx->stream));
        hipFree(m->p_logits);
        m->p_logits = nullptr;
        m->pf_logit_cap = 0;
        HIP_TRY(hipMalloc((void **)&m->p_logits, (size_t)s * c.vocab_size * 4));
        m->pf_logit_cap = s;
    }
    return LUMEN_OK;
}

static int run_prefill(lumen_llama *m, const std::vector<int> &ids, float *logits_host, int all_rows) {
    lumen_ctx *ctx = m->ctx;
    const lumen_llama_config &c = m->cfg;
    const int s = (int)ids.size();
    const int H = c.hidden_size, I = c.intermediate_size, V = c.vocab_size;
    LUMEN_TRY(ensure_prefill_buffers(m, s, all_rows != 0));
    HIP_TRY(hipMemcpyAsync(m->p_ids, ids.data(), sizeof(int) * s, hipMemcpyHostToDevice, ctx->stream));
    LUMEN_TRY(launch_embedding(ctx, m->embed, m->p_ids, s, H, V, m->p_x));
    for (int l = 0; l < c.num_hidden_layers; ++l) {
        const LayerW &w = m->layers[l];
        // (from the second layer on the down product of the layer before has left the normalised rows in p_n)
        if (l == 0) LUMEN_TRY(launch_rmsnorm(ctx, m->p_x, w.in_norm, m->p_n, s, H, c.rms_norm_eps));
        GemmArgs g = {};
        g.A = m->p_n; g.W = w.wqkv; g.C = m->p_qkv; g.M = s; g.N = m->qkvd; g.K = H; g.w_bf16 = m->bf16; g.epi = EPI_STORE;
        // the RoPE pass adds the K splits of this product itself (one launch and one pass less)
        int qkv_splits = 1;
        g.keep_splits = m->qkvd % 4 == 0;
        g.splits_used = &qkv_splits;
        LUMEN_TRY(launch_gemm(ctx, g));
        const float *qkv = qkv_splits > 1 ? ctx->gemm_ws : m->p_qkv;
        AttnPrefillArgs a = {};
        a.in_splits = qkv_splits; a.in_split_stride = (size_t)s * m->qkvd;
        a.q = qkv; a.k = qkv + m->qd; a.v = qkv + m->qd + m->kvd; a.out = m->p_attn;
        a.k_cache = m->k_slab + m->cache_stride * l; a.v_cache = m->v_slab + m->cache_stride * l;
        a.cos_t = m->cos_dev; a.sin_t = m->sin_dev;
        a.b = 1; a.s = s; a.hq = c.num_attention_heads; a.hkv = c.num_key_value_heads; a.d = m->D;
        a.max_seq = c.max_seq_len; a.past_len = m->len;
        a.q_stride = a.k_stride = a.v_stride = m->qkvd;
        a.scale = m->scale; a.causal = 1; a.q_norm_w = w.q_norm; a.k_norm_w = w.k_norm; a.norm_eps = c.rms_norm_eps;
        a.q_rot = m->p_qrot;
        LUMEN_TRY(launch_attn_prefill(ctx, a));
        g = {};
        g.A = m->p_attn; g.W = w.wo; g.C = m->p_h; g.M = s; g.N = H; g.K = m->qd; g.w_bf16 = m->bf16;
        g.epi = EPI_RESIDUAL; g.residual = m->p_x;
        g.norm_w = w.post_norm; g.norm_out = m->p_n; g.norm_eps = c.rms_norm_eps;  // post_attention_layernorm rides along
        LUMEN_TRY(launch_gemm(ctx, g));
        g = {};
        g.A = m->p_n; g.W = w.wgu; g.C = m->p_act; g.M = s; g.N = 2 * I; g.K = H; g.w_bf16 = m->bf16; g.epi = EPI_SWIGLU;
        LUMEN_TRY(launch_gemm(ctx, g));
        g = {};
        g.A = m->p_act; g.W = w.wdown; g.C = m->p_x; g.M = s; g.N = H; g.K = I; g.w_bf16 = m->bf16;
        g.epi = EPI_RESIDUAL; g.residual = m->p_h;
        // the next layer's input_layernorm -- or, where every row's logits are wanted, the final norm -- rides along
        if (l + 1 < c.num_hidden_layers) { g.norm_w = m->layers[l + 1].in_norm; g.norm_out = m->p_n; g.norm_eps = c.rms_norm_eps; }
        else if (all_rows) { g.norm_w = m->final_norm; g.norm_out = m->p_n; g.norm_eps = c.rms_norm_eps; }
        LUMEN_TRY(launch_gemm(ctx, g));
    }
    const int head_bf16 = (m->lm_head == (void *)m->embed) ? 0 : (int)m->bf16;
    if (all_rows) {  // what the reference computes, llama.rs:202-205 (the final norm came with the last down product)
        if (c.num_hidden_layers == 0) LUMEN_TRY(launch_rmsnorm(ctx, m->p_x, m->final_norm, m->p_n, s, H, c.rms_norm_eps));
        GemmArgs g = {};
        g.A = m->p_n; g.W = m->lm_head; g.C = m->p_logits; g.M = s; g.N = V; g.K = H; g.w_bf16 = head_bf16; g.epi = EPI_STORE;
        LUMEN_TRY(launch_gemm(ctx, g));
        m->len += s;
        if (logits_host) LUMEN_TRY(lumen_download(ctx, logits_host, m->p_logits, sizeof(float) * (size_t)s * V));
    } else {  // what its caller keeps, main.rs:155-163
        GemvArgs g = {};
        g.W = m->lm_head; g.x = m->p_x + (size_t)(s - 1) * H; g.y = m->logits; g.N = V; g.K = H; g.w_bf16 = head_bf16;
        g.pro = PRO_RMSNORM; g.norm_w = m->final_norm; g.eps = c.rms_norm_eps; g.epi = EPI_STORE;
        LUMEN_TRY(launch_gemv(ctx, g));
        m->len += s;
        if (logits_host) LUMEN_TRY(lumen_download(ctx, logits_host, m->logits, sizeof(float) * (size_t)V));
    }
    return sync_pos_to_device(m);
}

extern "C" int lumen_llama_forward(lumen_llama *m, const float *ids_host, int s, float *logits_host, int all_rows) {
    if (!m || (!ids_host && s > 0)) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_forward: null argument");
    if (s <= 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "llama_forward: empty input");
    HIP_TRY(hipSetDevice(m->ctx->device));
    std::vector<int> ids;
    LUMEN_TRY(ids_to_int(m, ids_host, s, ids));
    LUMEN_TRY(check_room(m, s));
    if (s > 1) return run_prefill(m, ids, logits_host, all_rows);
    // S == 1: the decode path (self_attention.rs:125)
    LUMEN_TRY(ensure_decode_graph(m));
    hipStream_t st = m->ctx->stream;
    HIP_TRY(hipMemcpyAsync(m->d_tok, ids.data(), sizeof(int), hipMemcpyHostToDevice, st));
    HIP_TRY(hipStreamSynchronize(st));
    HIP_TRY(launch_step(m));
    m->len += 1;
    if (logits_host) {
        LUMEN_TRY(lumen_download(m->ctx, logits_host, m->logits, sizeof(float) * (size_t)m->cfg.vocab_size));
        return check_handover(m);
    }
    // (no logits wanted: the step stays in flight, and a wait that gave up inside it is reported by the next call
    // that synchronises -- lumen_llama_forward with logits, lumen_llama_decode_greedy, lumen_llama_decode_profile)
    return LUMEN_OK;
}

extern "C" int lumen_llama_decode_greedy(lumen_llama *m, int first_id, int n, int32_t *ids_out, float *logits_out) {
    if (!m) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_decode_greedy: null model");
    if (n < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "llama_decode_greedy: n=%d", n);
    if (first_id < 0 || first_id >= m->cfg.vocab_size)
        LUMEN_FAIL(LUMEN_ERR_EMBED_OOB, "Embedding index out of bounds: %d >= %d", first_id, m->cfg.vocab_size);
    if (n == 0) return LUMEN_OK;
    HIP_TRY(hipSetDevice(m->ctx->device));
    LUMEN_TRY(check_room(m, n));
    LUMEN_TRY(ensure_decode_graph(m));
    hipStream_t st = m->ctx->stream;
    const size_t V = (size_t)m->cfg.vocab_size;
    HIP_TRY(hipMemcpyAsync(m->d_tok, &first_id, sizeof(int), hipMemcpyHostToDevice, st));
    HIP_TRY(hipStreamSynchronize(st));
    // the arg-max epilogue leaves every pick in tok_hist at the index of the position it is the token of
    const int len0 = m->len;
    int rc = LUMEN_OK;
    for (int t = 0; t < n && rc == LUMEN_OK; ++t) {
        // (the graph is captured anew at the step where the cache crosses the short / long attention boundary)
        rc = ensure_decode_graph(m);
        if (rc != LUMEN_OK) break;
        hipError_t e = launch_step(m);
        if (e == hipSuccess && logits_out)
            e = hipMemcpyAsync(logits_out + (size_t)t * V, m->logits, sizeof(float) * V, hipMemcpyDeviceToHost, st);
        if (e != hipSuccess) {
            lumen_set_error("decode step %d failed: %s", t, hipGetErrorString(e));
            rc = LUMEN_ERR_HIP;
        } else {
            m->len += 1;
        }
    }
    hipError_t e = hipStreamSynchronize(st);
    if (rc == LUMEN_OK && e == hipSuccess && ids_out)
        e = hipMemcpy(ids_out, m->tok_hist + len0 + 1, sizeof(int) * (size_t)n, hipMemcpyDeviceToHost);
    if (rc == LUMEN_OK && e != hipSuccess) LUMEN_FAIL(LUMEN_ERR_HIP, "decode_greedy: %s", hipGetErrorString(e));
    if (rc == LUMEN_OK) rc = check_handover(m);
    return rc;
}

// n greedy decode steps launched kernel by kernel (no graph), each launch
// bracketed by HIP events on the ctx stream: per kernel class the summed
// event-to-event milliseconds and the launch count.
extern "C" int lumen_llama_decode_profile(lumen_llama *m, int first_id, int n, double *ms_sum_out, int *count_out,
                                          int n_classes) {
    if (!m || !ms_sum_out || !count_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_decode_profile: null argument");
    if (n_classes < KC_COUNT) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_decode_profile: need %d classes", (int)KC_COUNT);
    if (first_id < 0 || first_id >= m->cfg.vocab_size)
        LUMEN_FAIL(LUMEN_ERR_EMBED_OOB, "Embedding index out of bounds: %d >= %d", first_id, m->cfg.vocab_size);
    for (int i = 0; i < n_classes; ++i) { ms_sum_out[i] = 0.0; count_out[i] = 0; }
    if (n <= 0) return LUMEN_OK;
    HIP_TRY(hipSetDevice(m->ctx->device));
    LUMEN_TRY(check_room(m, n));
    hipStream_t st = m->ctx->stream;
    HIP_TRY(hipMemcpyAsync(m->d_tok, &first_id, sizeof(int), hipMemcpyHostToDevice, st));
    HIP_TRY(hipStreamSynchronize(st));
    int rc = LUMEN_OK;
    for (int t = 0; t < n && rc == LUMEN_OK; ++t) {
        StepProbe pr;
        pr.on = true;
        pr.s = st;
        pr.ctx = m->ctx;
        pr.names = m->prof_names;
        m->ctx->note_kernels = true;
        rc = enqueue_decode_step(m, &pr);
        m->ctx->note_kernels = false;
        const hipError_t e = hipStreamSynchronize(st);
        if (rc == LUMEN_OK && e == hipSuccess) {
            m->len += 1;
            for (size_t i = 0; i < pr.cls.size(); ++i) {
                float ms = 0.f;
                if (hipEventElapsedTime(&ms, pr.ev[2 * i], pr.ev[2 * i + 1]) == hipSuccess) {
                    ms_sum_out[pr.cls[i]] += ms;
                    count_out[pr.cls[i]] += 1;
                }
            }
        }
        for (hipEvent_t ev : pr.ev) hipEventDestroy(ev);
        if (rc == LUMEN_OK && e != hipSuccess) {
            lumen_set_error("decode_profile step %d: %s", t, hipGetErrorString(e));
            rc = LUMEN_ERR_HIP;
        }
        if (rc == LUMEN_OK) rc = check_handover(m);  // (figures of a step whose wait gave up would mean nothing)
    }
    return rc;
}

extern "C" int lumen_llama_profile_kernel_name(const lumen_llama *m, int kernel_class, char *buf, int buf_len) {
    if (!m || !buf || buf_len <= 0) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_profile_kernel_name: null argument");
    if (kernel_class < 0 || kernel_class >= KC_COUNT)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_profile_kernel_name: class %d of %d", kernel_class, (int)KC_COUNT);
    snprintf(buf, (size_t)buf_len, "%s", m->prof_names[kernel_class].c_str());
    return LUMEN_OK;
}

// ---------------------------------------------------------------- the layer-level operator
struct lumen_decoder_layer {
    lumen_llama *m = nullptr;
};

__global__ void set_pos_kernel(int *p, int v) { *p = v; }

extern "C" int lumen_decoder_layer_create(lumen_ctx *ctx, const lumen_llama_config *cfg, lumen_decoder_layer **out) {
    if (!ctx || !cfg || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "decoder_layer_create: null argument");
    *out = nullptr;
    lumen_llama_config c = *cfg;
    c.vocab_size = 1;         // (no embedding, no lm_head here)
    c.num_hidden_layers = 1;
    c.tie_embeddings = 0;
    lumen_llama *m = nullptr;
    LUMEN_TRY(llama_create_impl(ctx, &c, true, &m));
    lumen_decoder_layer *h = new lumen_decoder_layer();
    h->m = m;
    *out = h;
    return LUMEN_OK;
}

extern "C" int lumen_decoder_layer_destroy(lumen_decoder_layer *h) {
    if (!h) return LUMEN_OK;
    lumen_llama_destroy(h->m);
    delete h;
    return LUMEN_OK;
}

extern "C" int lumen_decoder_layer_decode_f32(lumen_decoder_layer *h, lumen_kv_cache *cache, const void *wqkv, const void *wo,
                                              const void *wgu, const void *wdown, const float *input_norm, const float *post_norm,
                                              const float *q_norm, const float *k_norm, const float *x, float *y) {
    if (!h || !cache || !wqkv || !wo || !wgu || !wdown || !input_norm || !post_norm || !x || !y)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "decoder_layer_decode: null argument");
    lumen_llama *m = h->m;
    const lumen_llama_config &c = m->cfg;
    if (cache->ctx != m->ctx) LUMEN_FAIL(LUMEN_ERR_INVALID, "decoder_layer_decode: the cache belongs to another context");
    if (cache->b != 1 || cache->h_kv != c.num_key_value_heads || cache->d != m->D || cache->max_seq != c.max_seq_len)
        LUMEN_FAIL(LUMEN_ERR_SHAPE, "decoder_layer_decode: cache [%d, %d, %d, %d] against a layer of %d kv heads x %d, %d rows",
                   cache->b, cache->h_kv, cache->max_seq, cache->d, c.num_key_value_heads, m->D, c.max_seq_len);
    if ((c.qk_norm != 0) != (q_norm != nullptr && k_norm != nullptr))
        LUMEN_FAIL(LUMEN_ERR_INVALID, "decoder_layer_decode: q/k norm gains %s", c.qk_norm ? "missing" : "given to a layer without q/k norm");
    if (cache->len + 1 > cache->max_seq)  // self_attention.rs:144-149
        LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "KV cache overflow: new_len=%d > max_seq=%d", cache->len + 1, cache->max_seq);
    HIP_TRY(hipSetDevice(m->ctx->device));
    // the position lives in device memory (the launches read it there); it follows the cache's length, which
    // changes once per token for a stack of layers that share this state
    if (m->len != cache->len || m->layer_epoch == 0) {
        m->len = cache->len;
        hipLaunchKernelGGL(set_pos_kernel, dim3(1), dim3(1), 0, m->ctx->stream, m->d_pos, m->len);
        LUMEN_CHECK_LAUNCH();
    }
    LayerW w;
    w.wqkv = const_cast<void *>(wqkv); w.wo = const_cast<void *>(wo); w.wgu = const_cast<void *>(wgu); w.wdown = const_cast<void *>(wdown);
    w.in_norm = const_cast<float *>(input_norm); w.post_norm = const_cast<float *>(post_norm);
    w.q_norm = const_cast<float *>(q_norm); w.k_norm = const_cast<float *>(k_norm);
    // the hand-over tags of this call's launches: every call its own (the step counter in device memory stays 0 here)
    if (++m->layer_epoch >= 0xfffffff0u) m->layer_epoch = 1;
    StepProbe none;
    LUMEN_TRY(enqueue_decoder_layer(m, w, cache->k, cache->v, x, nullptr, y, 0u, m->layer_epoch, &none));
    cache->len += 1;
    return LUMEN_OK;
}

extern "C" int lumen_llama_reset(lumen_llama *m) {
    if (!m) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_reset: null model");
    m->len = 0;  // KVCacheInner::reset, self_attention.rs:41-43: data stays
    return sync_pos_to_device(m);
}

extern "C" int lumen_llama_set_kv_len(lumen_llama *m, int len) {
    if (!m) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_set_kv_len: null model");
    if (len < 0 || len > m->cfg.max_seq_len)
        LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "llama_set_kv_len: %d outside [0, %d]", len, m->cfg.max_seq_len);
    HIP_TRY(hipSetDevice(m->ctx->device));
    m->len = len;
    return sync_pos_to_device(m);
}

extern "C" int lumen_llama_get_config(const lumen_llama *m, lumen_llama_config *cfg_out) {
    if (!m || !cfg_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_get_config: null argument");
    *cfg_out = m->cfg;
    return LUMEN_OK;
}

extern "C" int lumen_llama_kv_len(const lumen_llama *m, int *len_out) {
    if (!m || !len_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_kv_len: null argument");
    *len_out = m->len;
    return LUMEN_OK;
}

extern "C" int lumen_llama_cache_download(lumen_llama *m, int layer, float *k_host, float *v_host) {
    if (!m || !k_host || !v_host) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_cache_download: null argument");
    if (layer < 0 || layer >= m->cfg.num_hidden_layers)  // llama.rs:182-188 analogue
        LUMEN_FAIL(LUMEN_ERR_CACHE_COUNT, "KV cache index %d outside [0,%d)", layer, m->cfg.num_hidden_layers);
    const size_t bytes = m->cache_stride * sizeof(float);
    LUMEN_TRY(lumen_download(m->ctx, k_host, m->k_slab + m->cache_stride * layer, bytes));
    return lumen_download(m->ctx, v_host, m->v_slab + m->cache_stride * layer, bytes);
}

extern "C" int lumen_llama_cache_upload(lumen_llama *m, int layer, const float *k_host, const float *v_host) {
    if (!m || !k_host || !v_host) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_cache_upload: null argument");
    if (layer < 0 || layer >= m->cfg.num_hidden_layers)
        LUMEN_FAIL(LUMEN_ERR_CACHE_COUNT, "KV cache index %d outside [0,%d)", layer, m->cfg.num_hidden_layers);
    const size_t bytes = m->cache_stride * sizeof(float);
    LUMEN_TRY(lumen_upload(m->ctx, m->k_slab + m->cache_stride * layer, k_host, bytes));
    return lumen_upload(m->ctx, m->v_slab + m->cache_stride * layer, v_host, bytes);
}

extern "C" int lumen_llama_decode_bytes(const lumen_llama *m, int len, double *bytes_out) {
    if (!m || !bytes_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "llama_decode_bytes: null argument");
    const lumen_llama_config &c = m->cfg;
    const double H = c.hidden_size, I = c.intermediate_size, V = c.vocab_size, L = c.num_hidden_layers;
    const double per_layer = ((double)m->qkvd * H + H * m->qd + 3.0 * H * I) * (double)m->esz;
    const double head = V * H * ((m->lm_head == (void *)m->embed) ? 4.0 : (double)m->esz);
    const double norms = (2.0 * L + 1.0) * H * 4.0 + (c.qk_norm ? 2.0 * L * m->D * 4.0 : 0.0);
    const double kv = L * 2.0 * c.num_key_value_heads * m->D * 4.0 * (double)len;
    *bytes_out = L * per_layer + head + norms + kv;
    return LUMEN_OK;
}
