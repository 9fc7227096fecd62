// Runs the library's decode-path device code ON THE CPU (the shim in tests/cpu_emu/shim stands in for the HIP
// runtime; see its header), under AddressSanitizer / UndefinedBehaviorSanitizer, through the same C ABI the GPU tests
// use, and holds the results to the CPU checker (oracle/).  Covered: the chained q|k|v -> attention -> o_proj launch
// in its three forms (with a q|k|v role, attention + o_proj only, separate launches), with one and with several
// attention workgroups per head (slices + fold), rotated and un-rotated (q/k-norm) hand-over, f32 and bf16 weights;
// the gate|up -> down chain; the few-row product of short prompts with ragged shapes and all three epilogues; the
// streaming vector-matrix product and the stand-alone decode attention those forms fall back to, the latter also
// at operator level over a sliced cache (slices merged inside the launch).
//
//   emu_test [case ...]      cases: chain sliced qknorm bf16 skinny attn layerop (default: all)
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <string>
#include <vector>

#include "../../include/lumen_hip.h"
extern "C" {
#include "lumen_oracle.h"
}

static int g_failures = 0;
#define CHECK(cond, ...)                                    \
    do {                                                    \
        if (!(cond)) {                                      \
            ++g_failures;                                   \
            fprintf(stderr, "FAIL %s:%d: ", __FILE__, __LINE__); \
            fprintf(stderr, __VA_ARGS__);                   \
            fprintf(stderr, "\n");                          \
        }                                                   \
    } while (0)
#define OK(call)                                                                               \
    do {                                                                                       \
        const int rc_ = (call);                                                                \
        if (rc_ != LUMEN_OK) {                                                                 \
            fprintf(stderr, "%s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, rc_, lumen_last_error()); \
            exit(2);                                                                           \
        }                                                                                      \
    } while (0)

// deterministic values: a 64-bit LCG and the sum of four uniforms (close enough to a bell for test weights)
static uint64_t g_state = 0x9e3779b97f4a7c15ull;
static float rnd() {
    float s = 0.f;
    for (int i = 0; i < 4; ++i) {
        g_state = g_state * 6364136223846793005ull + 1442695040888963407ull;
        s += (float)((g_state >> 40) & 0xffffff) / 16777216.0f - 0.5f;
    }
    return s * 1.7320508f;  // unit variance
}
static std::vector<float> randn(size_t n, float std_, float mean = 0.f) {
    std::vector<float> v(n);
    for (float &x : v) x = mean + std_ * rnd();
    return v;
}
static void to_bf16_values(std::vector<float> &v) {  // round to nearest even, keep as f32
    for (float &x : v) {
        uint32_t u;
        memcpy(&u, &x, 4);
        u += 0x7fffu + ((u >> 16) & 1u);
        u &= 0xffff0000u;
        memcpy(&x, &u, 4);
    }
}
static double max_rel(const float *got, const float *ref, size_t n) {
    double worst = 0, scale = 1e-30;
    for (size_t i = 0; i < n; ++i) scale = fmax(scale, fabs((double)ref[i]));
    for (size_t i = 0; i < n; ++i) {
        const double d = fabs((double)got[i] - (double)ref[i]);
        worst = fmax(worst, isnan(d) ? INFINITY : d);
    }
    return worst / scale;
}

struct Model {
    lumen_llama_config cfg;
    lumen_llama *gpu = nullptr;
    lo_llama *ora = nullptr;
    std::vector<std::vector<float>> keep;  // the checker borrows the arrays
    int D = 0;
};

static const float *param(Model &m, const std::string &name, size_t rows, size_t cols, float std_, float mean, bool bf16) {
    m.keep.push_back(randn(rows * (cols ? cols : 1), std_, mean));
    std::vector<float> &v = m.keep.back();
    if (bf16 && cols) to_bf16_values(v);
    const int64_t shape[2] = {(int64_t)rows, (int64_t)cols};
    OK(lumen_llama_set_param(m.gpu, name.c_str(), v.data(), LUMEN_DTYPE_F32, shape, cols ? 2 : 1));
    return v.data();
}

static Model build(lumen_ctx *ctx, int V, int H, int I, int L, int hq, int hkv, int head_dim, int max_seq, bool qk_norm,
                   bool tie, bool bf16) {
    Model m;
    memset(&m.cfg, 0, sizeof m.cfg);
    m.cfg.vocab_size = V; m.cfg.hidden_size = H; m.cfg.intermediate_size = I; m.cfg.num_hidden_layers = L;
    m.cfg.num_attention_heads = hq; m.cfg.num_key_value_heads = hkv; m.cfg.rms_norm_eps = 1e-5f;
    m.cfg.max_seq_len = max_seq; m.cfg.rope_theta = 10000.f; m.cfg.head_dim = head_dim; m.cfg.qk_norm = qk_norm;
    m.cfg.tie_embeddings = tie; m.cfg.weight_dtype = bf16 ? LUMEN_DTYPE_BF16 : LUMEN_DTYPE_F32;
    m.D = head_dim ? head_dim : H / hq;
    OK(lumen_llama_create(ctx, &m.cfg, &m.gpu));
    lo_llama_config oc;
    memset(&oc, 0, sizeof oc);
    oc.vocab_size = V; oc.hidden_size = H; oc.intermediate_size = I; oc.num_hidden_layers = L;
    oc.num_attention_heads = hq; oc.num_key_value_heads = hkv; oc.rms_norm_eps = 1e-5f; oc.max_seq_len = max_seq;
    oc.rope_theta = 10000.f; oc.head_dim = head_dim; oc.qk_norm = qk_norm; oc.tie_embeddings = tie;
    m.ora = lo_llama_new(&oc);
    m.keep.reserve((size_t)L * 11 + 3);
    const size_t qd = (size_t)hq * m.D, kvd = (size_t)hkv * m.D;
    // (the embedding table stays f32 on the GPU side whatever the weight dtype; with tied bf16 weights the head is its
    // rounded copy, so the table is made of bf16-exact values then)
    const float *embed = param(m, "model.embed_tokens.weight", V, H, 0.1f, 0.f, bf16 && tie);
    const float *fnorm = param(m, "model.norm.weight", H, 0, 0.1f, 1.f, false);
    const float *head = tie ? embed : param(m, "lm_head.weight", V, H, 0.1f, 0.f, bf16);
    lo_llama_set_globals(m.ora, embed, fnorm, head);
    for (int l = 0; l < L; ++l) {
        const std::string p = "model.layers." + std::to_string(l) + ".";
        lo_llama_layer w;
        memset(&w, 0, sizeof w);
        w.wq = param(m, p + "self_attn.q_proj.weight", qd, H, 0.06f, 0.f, bf16);
        w.wk = param(m, p + "self_attn.k_proj.weight", kvd, H, 0.06f, 0.f, bf16);
        w.wv = param(m, p + "self_attn.v_proj.weight", kvd, H, 0.06f, 0.f, bf16);
        w.wo = param(m, p + "self_attn.o_proj.weight", H, qd, 0.06f, 0.f, bf16);
        w.w_gate = param(m, p + "mlp.gate_proj.weight", I, H, 0.06f, 0.f, bf16);
        w.w_up = param(m, p + "mlp.up_proj.weight", I, H, 0.06f, 0.f, bf16);
        w.w_down = param(m, p + "mlp.down_proj.weight", H, I, 0.06f, 0.f, bf16);
        w.input_norm = param(m, p + "input_layernorm.weight", H, 0, 0.1f, 1.f, false);
        w.post_norm = param(m, p + "post_attention_layernorm.weight", H, 0, 0.1f, 1.f, false);
        if (qk_norm) {
            w.q_norm = param(m, p + "self_attn.q_norm.weight", m.D, 0, 0.1f, 1.f, false);
            w.k_norm = param(m, p + "self_attn.k_norm.weight", m.D, 0, 0.1f, 1.f, false);
        }
        lo_llama_set_layer(m.ora, l, &w);
    }
    return m;
}

static void destroy(Model &m) {
    lumen_llama_destroy(m.gpu);
    lo_llama_free(m.ora);
}

// the same tokens through both; every row of logits compared
static void forward_both(Model &m, const std::vector<int> &ids, double tol, const char *what) {
    const int V = m.cfg.vocab_size, S = (int)ids.size();
    std::vector<float> f(ids.begin(), ids.end()), got((size_t)S * V), ref((size_t)S * V);
    OK(lumen_llama_forward(m.gpu, f.data(), S, got.data(), 1));
    const int rc = lo_llama_forward(m.ora, f.data(), S, ref.data());
    CHECK(rc == LO_OK, "%s: checker status %d", what, rc);
    const double e = max_rel(got.data(), ref.data(), got.size());
    printf("  %-58s %d row(s), max rel err %.2e\n", what, S, e);
    CHECK(e <= tol, "%s: max rel err %.3g > %.1g", what, e, tol);
}

// both caches filled with the same made-up rows (what they hold does not matter to the comparison)
static void fill_caches(Model &m, int len) {
    const size_t n = (size_t)m.cfg.num_key_value_heads * m.cfg.max_seq_len * m.D;
    for (int l = 0; l < m.cfg.num_hidden_layers; ++l) {
        std::vector<float> k = randn(n, 0.7f), v = randn(n, 0.7f);
        OK(lumen_llama_cache_upload(m.gpu, l, k.data(), v.data()));
        CHECK(lo_llama_set_kv(m.ora, l, k.data(), v.data(), len) == LO_OK, "set_kv");
    }
    OK(lumen_llama_set_kv_len(m.gpu, len));
}

static void decode_forms(Model &m, double tol, const char *label, bool qk_norm) {
    char what[160];
    int tok = 5;
    for (int form = 2; form >= 0; --form) {
        if (form == 1 && qk_norm) continue;  // (attention + o_proj alone wants a rotated q from an earlier launch)
        OK(lumen_llama_set_handover(m.gpu, form, -1, -1, -1, -1));
        for (int mode = LUMEN_DECODE_GRAPH; mode >= LUMEN_DECODE_EAGER; --mode) {
            OK(lumen_llama_set_decode_mode(m.gpu, mode));
            snprintf(what, sizeof what, "%s: form %d, %s step", label, form, mode == LUMEN_DECODE_GRAPH ? "graph" : "eager");
            forward_both(m, {tok}, tol, what);
            tok = (tok * 7 + 3) % m.cfg.vocab_size;
        }
    }
    OK(lumen_llama_set_handover(m.gpu, 2, -1, -1, -1, -1));
    OK(lumen_llama_set_decode_mode(m.gpu, LUMEN_DECODE_GRAPH));
}

static void case_chain(lumen_ctx *ctx) {
    printf("chain: hidden 512, 8/2 heads of 64, intermediate 1024 (MLP chain), f32\n");
    Model m = build(ctx, 96, 512, 1024, 2, 8, 2, 0, 1024, false, false, false);
    forward_both(m, {3, 1, 4}, 1e-4, "prompt of 3 rows (few-row product, row-loop attention)");
    forward_both(m, {1, 5}, 1e-4, "prompt of 2 rows into the live cache");
    decode_forms(m, 1e-4, "5-10 cached rows", false);
    fill_caches(m, 300);  // a second trip of rows in one workgroup
    decode_forms(m, 1e-4, "300 cached rows", false);
    int32_t picks[3];
    std::vector<float> logits((size_t)3 * m.cfg.vocab_size), ref((size_t)m.cfg.vocab_size);
    OK(lumen_llama_decode_greedy(m.gpu, 7, 3, picks, logits.data()));  // the arg-max tail and the on-device loop
    int tok = 7;
    for (int t = 0; t < 3; ++t) {
        const float f = (float)tok;
        lo_llama_forward(m.ora, &f, 1, ref.data());
        CHECK(max_rel(logits.data() + (size_t)t * m.cfg.vocab_size, ref.data(), ref.size()) <= 1e-4, "greedy step %d", t);
        CHECK(picks[t] == lo_argmax_f32(ref.data(), m.cfg.vocab_size), "greedy pick %d: %d", t, picks[t]);
        tok = picks[t];
    }
    printf("  greedy call of 3 steps: picks %d %d %d\n", picks[0], picks[1], picks[2]);
    destroy(m);
}

static void case_sliced(lumen_ctx *ctx) {
    printf("sliced: the same shape, caches of 700 and 1400 rows (4 slices of one / of two trips + fold)\n");
    Model m = build(ctx, 96, 512, 1024, 1, 8, 2, 0, 2048, false, false, false);
    fill_caches(m, 700);
    decode_forms(m, 1e-4, "700 cached rows", false);
    fill_caches(m, 1400);
    forward_both(m, {9}, 1e-4, "1400 cached rows: form 2, graph step");
    fill_caches(m, 767);  // the new row is the last of a slice, the next step opens the fourth slice
    forward_both(m, {2}, 1e-4, "767 cached rows (last row of a slice)");
    forward_both(m, {8}, 1e-4, "768 cached rows (first row of the next slice)");
    destroy(m);
}

static void case_qknorm(lumen_ctx *ctx) {
    printf("qknorm: hidden 512, 4/2 heads of 128 with per-head q/k norm, tied head: un-rotated hand-over\n");
    Model m = build(ctx, 80, 512, 1024, 1, 4, 2, 128, 1024, true, true, false);
    forward_both(m, {3, 1, 4, 1}, 1e-4, "prompt of 4 rows");
    decode_forms(m, 1e-4, "4-7 cached rows", true);
    fill_caches(m, 300);  // head_dim 128: trips of 128 rows, so 4 slices of one trip
    decode_forms(m, 1e-4, "300 cached rows", true);
    destroy(m);
}

static void case_bf16(lumen_ctx *ctx) {
    printf("bf16: hidden 1024, 16/4 heads of 64, intermediate 2048, bf16 weights\n");
    Model m = build(ctx, 64, 1024, 2048, 1, 16, 4, 0, 512, false, false, true);
    forward_both(m, {3, 1}, 2e-2, "prompt of 2 rows");
    forward_both(m, {4}, 2e-2, "form 2, graph step");
    OK(lumen_llama_set_handover(m.gpu, 0, -1, -1, -1, -1));
    forward_both(m, {5}, 2e-2, "separate launches");
    destroy(m);
}

// the few-row product on its own: ragged N and K, all three epilogues through the operator-level entry points
static void case_skinny(lumen_ctx *ctx) {
    printf("skinny: lumen_matmul_f32 / lumen_gemm_bf16w with 2 rows (vector ALU) and 3-32 rows (f32 matrix instruction), ragged shapes\n");
    // (three to 32 rows: the weight-streaming kernel with the f32 matrix instruction, K split inside and across workgroups)
    const int shapes[][3] = {{2, 37, 100}, {2, 64, 1032}, {3, 64, 1032}, {4, 129, 264}, {4, 6, 4}, {5, 37, 100}, {16, 40, 1032}, {32, 18, 40}, {9, 16, 4}};
    for (const auto &sh : shapes) {
        const int M = sh[0], N = sh[1], K = sh[2];
        std::vector<float> A = randn((size_t)M * K, 1.f), W = randn((size_t)N * K, 0.05f), C((size_t)M * N), R((size_t)M * N);
        void *dA, *dW, *dC;
        OK(lumen_malloc(ctx, A.size() * 4, &dA));
        OK(lumen_malloc(ctx, W.size() * 4, &dW));
        OK(lumen_malloc(ctx, C.size() * 4, &dC));
        OK(lumen_upload(ctx, dA, A.data(), A.size() * 4));
        OK(lumen_upload(ctx, dW, W.data(), W.size() * 4));
        OK(lumen_matmul_f32(ctx, (const float *)dA, (const float *)dW, (float *)dC, M, N, K, K));
        OK(lumen_download(ctx, C.data(), dC, C.size() * 4));
        lo_gemm_f32(A.data(), W.data(), R.data(), M, N, K);
        const double e = max_rel(C.data(), R.data(), C.size());
        printf("  %d x %d x %d f32: max rel err %.2e\n", M, N, K, e);
        CHECK(e <= 1e-5, "skinny %dx%dx%d: %.3g", M, N, K, e);
        if (K % 8 == 0 && M <= 16) {  // (more rows with bf16 weights: the bf16 matrix instructions, not emulated)
            std::vector<float> Wb = W;
            to_bf16_values(Wb);
            std::vector<uint16_t> bits(Wb.size());
            for (size_t i = 0; i < Wb.size(); ++i) {
                uint32_t u;
                memcpy(&u, &Wb[i], 4);
                bits[i] = (uint16_t)(u >> 16);
            }
            void *dB;
            OK(lumen_malloc(ctx, bits.size() * 2, &dB));
            OK(lumen_upload(ctx, dB, bits.data(), bits.size() * 2));
            OK(lumen_gemm_bf16w(ctx, (const float *)dA, (const uint16_t *)dB, (float *)dC, M, N, K));
            OK(lumen_download(ctx, C.data(), dC, C.size() * 4));
            lo_gemm_f32(A.data(), Wb.data(), R.data(), M, N, K);
            const double eb = max_rel(C.data(), R.data(), C.size());
            printf("  %d x %d x %d bf16 weights: max rel err %.2e\n", M, N, K, eb);
            CHECK(eb <= 1e-5, "skinny bf16 %dx%dx%d: %.3g", M, N, K, eb);
            OK(lumen_free(ctx, dB));
        }
        OK(lumen_free(ctx, dA));
        OK(lumen_free(ctx, dW));
        OK(lumen_free(ctx, dC));
    }
}

// the operator-level decode attention over a sliced cache: slices merged inside the launch (tagged words polled by
// the workgroup of the last slice), through the allocating entry point and through the one with the fixed scratch
static void case_attn(lumen_ctx *ctx) {
    printf("attn: lumen_attn_decode_f32 / lumen_attn_decode_static_f32, 4/2 heads of 64, 700 and 40 cached rows\n");
    const int h = 4, hkv = 2, d = 64, max_seq = 1024;
    const float scale = 0.125f;
    lumen_rope *rope = nullptr;
    OK(lumen_rope_create(ctx, d, max_seq, 10000.f, &rope));
    std::vector<float> cs((size_t)max_seq * d), sn((size_t)max_seq * d);
    lo_rope_table(cs.data(), sn.data(), d, max_seq, 10000.f);
    for (int filled : {700, 40}) {
        lumen_kv_cache *ca = nullptr, *cb = nullptr;
        OK(lumen_kv_cache_create(ctx, 1, hkv, max_seq, d, &ca));
        OK(lumen_kv_cache_create(ctx, 1, hkv, max_seq, d, &cb));
        lo_kv_cache *co = lo_kv_cache_new(1, hkv, max_seq, d);
        std::vector<float> k0 = randn((size_t)hkv * filled * d, 1.f), v0 = randn((size_t)hkv * filled * d, 1.f);
        void *dk, *dv;
        OK(lumen_malloc(ctx, k0.size() * 4, &dk));
        OK(lumen_malloc(ctx, v0.size() * 4, &dv));
        OK(lumen_upload(ctx, dk, k0.data(), k0.size() * 4));
        OK(lumen_upload(ctx, dv, v0.data(), v0.size() * 4));
        for (lumen_kv_cache *c : {ca, cb}) {
            OK(lumen_kv_cache_update(c, (const float *)dk, (const float *)dv, filled, 0));
            OK(lumen_kv_cache_set_len(c, filled));
        }
        for (int hk = 0; hk < hkv; ++hk) {
            memcpy(co->k + (size_t)hk * max_seq * d, k0.data() + (size_t)hk * filled * d, sizeof(float) * filled * d);
            memcpy(co->v + (size_t)hk * max_seq * d, v0.data() + (size_t)hk * filled * d, sizeof(float) * filled * d);
        }
        co->len = filled;
        void *dq, *dkn, *dvn, *dout;
        OK(lumen_malloc(ctx, (size_t)h * d * 4, &dq));
        OK(lumen_malloc(ctx, (size_t)hkv * d * 4, &dkn));
        OK(lumen_malloc(ctx, (size_t)hkv * d * 4, &dvn));
        OK(lumen_malloc(ctx, (size_t)h * d * 4, &dout));
        for (int step = 0; step < 2; ++step) {
            std::vector<float> q = randn((size_t)h * d, 1.f), kn = randn((size_t)hkv * d, 1.f), vn = randn((size_t)hkv * d, 1.f);
            std::vector<float> ref((size_t)h * d), got((size_t)h * d), got_static((size_t)h * d);
            OK(lumen_upload(ctx, dq, q.data(), q.size() * 4));
            OK(lumen_upload(ctx, dkn, kn.data(), kn.size() * 4));
            OK(lumen_upload(ctx, dvn, vn.data(), vn.size() * 4));
            OK(lumen_attn_decode_f32(ca, rope, (const float *)dq, (const float *)dkn, (const float *)dvn, (float *)dout, h, scale, 1));
            OK(lumen_download(ctx, got.data(), dout, got.size() * 4));
            OK(lumen_attn_decode_static_f32(cb, rope, (const float *)dq, (const float *)dkn, (const float *)dvn, (float *)dout, h, scale, 1));
            OK(lumen_download(ctx, got_static.data(), dout, got_static.size() * 4));
            CHECK(lo_attn_decode_f32(co, q.data(), kn.data(), vn.data(), ref.data(), h, cs.data(), sn.data(), max_seq, scale, 1) == LO_OK, "checker");
            const double e = max_rel(got.data(), ref.data(), ref.size());
            printf("  %d cached rows: max rel err %.2e, fixed-scratch entry %s\n", filled + step, e,
                   memcmp(got.data(), got_static.data(), got.size() * 4) ? "DIFFERS" : "bit-equal");
            CHECK(e <= 2e-5, "attn %d rows: %.3g", filled + step, e);
            CHECK(!memcmp(got.data(), got_static.data(), got.size() * 4), "fixed-scratch entry differs at %d rows", filled + step);
        }
        for (void *p : {dk, dv, dq, dkn, dvn, dout}) OK(lumen_free(ctx, p));
        OK(lumen_kv_cache_destroy(ca));
        OK(lumen_kv_cache_destroy(cb));
        lo_kv_cache_free(co);
    }
    OK(lumen_rope_destroy(rope));
}

// LlamaDecoderLayer::forward_infer for one token as ONE operator call per layer (lumen_decoder_layer_decode_f32): two
// layers of the chain shape driven layer by layer, embedding row in, final norm + lm_head by the checker's own
// operators, against the checker's whole-model step
static void case_layerop(lumen_ctx *ctx) {
    printf("layerop: lumen_decoder_layer_decode_f32, two layers of hidden 512, 8/2 heads of 64, intermediate 1024\n");
    const int V = 96, H = 512, I = 1024, L = 2, hq = 8, hkv = 2, D = 64, max_seq = 256;
    Model m = build(ctx, V, H, I, L, hq, hkv, 0, max_seq, false, false, false);
    lumen_decoder_layer *op = nullptr;
    OK(lumen_decoder_layer_create(ctx, &m.cfg, &op));
    // the layers' weights laid out as the fused step wants them: q|k|v rows one after the other, gate / up interleaved
    // (m.keep: embed, final norm, lm_head, then per layer wq wk wv wo gate up down input_norm post_norm)
    struct Dev { void *wqkv, *wo, *wgu, *wdown, *n1, *n2; lumen_kv_cache *cache; } dev[2];
    const size_t qd = (size_t)hq * D, kvd = (size_t)hkv * D;
    for (int l = 0; l < L; ++l) {
        const std::vector<float> *w = &m.keep[3 + (size_t)l * 9];
        std::vector<float> qkv;
        for (int i = 0; i < 3; ++i) qkv.insert(qkv.end(), w[i].begin(), w[i].end());
        std::vector<float> gu((size_t)2 * I * H);
        for (int i = 0; i < I; ++i) {
            memcpy(&gu[(size_t)(2 * i) * H], &w[4][(size_t)i * H], sizeof(float) * H);
            memcpy(&gu[(size_t)(2 * i + 1) * H], &w[5][(size_t)i * H], sizeof(float) * H);
        }
        auto up = [&](const std::vector<float> &v) {
            void *d;
            OK(lumen_malloc(ctx, v.size() * 4, &d));
            OK(lumen_upload(ctx, d, v.data(), v.size() * 4));
            return d;
        };
        CHECK(qkv.size() == (qd + 2 * kvd) * H, "q|k|v rows");
        dev[l].wqkv = up(qkv); dev[l].wo = up(w[3]); dev[l].wgu = up(gu); dev[l].wdown = up(w[6]);
        dev[l].n1 = up(w[7]); dev[l].n2 = up(w[8]);
        OK(lumen_kv_cache_create(ctx, 1, hkv, max_seq, D, &dev[l].cache));
    }
    void *dx;
    OK(lumen_malloc(ctx, (size_t)H * 4, &dx));
    std::vector<float> x(H), nx(H), got(V), ref(V);
    int tok = 11;
    for (int t = 0; t < 3; ++t) {
        OK(lumen_upload(ctx, dx, m.keep[0].data() + (size_t)tok * H, (size_t)H * 4));  // Embedding::forward
        for (int l = 0; l < L; ++l)
            OK(lumen_decoder_layer_decode_f32(op, dev[l].cache, dev[l].wqkv, dev[l].wo, dev[l].wgu, dev[l].wdown,
                                              (const float *)dev[l].n1, (const float *)dev[l].n2, nullptr, nullptr,
                                              (const float *)dx, (float *)dx));
        OK(lumen_download(ctx, x.data(), dx, (size_t)H * 4));
        lo_rmsnorm_f32(x.data(), m.keep[1].data(), nx.data(), 1, H, m.cfg.rms_norm_eps);
        lo_gemv_f32(m.keep[2].data(), nx.data(), got.data(), V, H);
        const float f = (float)tok;
        lo_llama_forward(m.ora, &f, 1, ref.data());
        const double e = max_rel(got.data(), ref.data(), ref.size());
        printf("  token %d through %d layer calls: max rel err %.2e\n", t, L, e);
        CHECK(e <= 1e-4, "layer operator, token %d: %.3g", t, e);
        tok = (tok * 5 + 1) % V;
    }
    int len = 0;
    OK(lumen_kv_cache_len(dev[1].cache, &len));
    CHECK(len == 3, "cache length %d", len);
    for (int l = 0; l < L; ++l) {
        for (void *p : {dev[l].wqkv, dev[l].wo, dev[l].wgu, dev[l].wdown, dev[l].n1, dev[l].n2}) OK(lumen_free(ctx, p));
        OK(lumen_kv_cache_destroy(dev[l].cache));
    }
    OK(lumen_free(ctx, dx));
    OK(lumen_decoder_layer_destroy(op));
    destroy(m);
}

// The harness checks itself: a product whose output array is one element short must be stopped by the sanitizer.
static void selfcheck_oob(lumen_ctx *ctx) {
    const int N = 64, K = 256;
    std::vector<float> W = randn((size_t)N * K, 0.1f), x = randn(K, 1.f);
    void *dW, *dx, *dy;
    OK(lumen_malloc(ctx, W.size() * 4, &dW));
    OK(lumen_malloc(ctx, x.size() * 4, &dx));
    OK(lumen_malloc(ctx, (size_t)(N - 1) * 4, &dy));
    OK(lumen_upload(ctx, dW, W.data(), W.size() * 4));
    OK(lumen_upload(ctx, dx, x.data(), x.size() * 4));
    fprintf(stderr, "selfcheck: a product of %d rows into an array of %d\n", N, N - 1);
    lumen_gemv_f32(ctx, (const float *)dW, (const float *)dx, (float *)dy, N, K);
    fprintf(stderr, "selfcheck: the write past the array went unnoticed\n");
}


// the row-count dispatch of the products (2 rows: vector ALU; 3-32: f32 matrix instruction, bf16-stored weights up to
// 16 rows) over pseudo-random ragged shapes: every access bounds-checked by the sanitizer, values against the checker
static void case_shapes(lumen_ctx *ctx) {
    printf("shapes: 48 pseudo-random products of 2-32 rows, f32 and bf16-stored weights\n");
    unsigned long long st = 12345;
    auto rnd = [&]() { st = st * 6364136223846793005ull + 1442695040888963407ull; return (double)(st >> 11) / 9007199254740992.0; };
    double worst = 0.0;
    for (int it = 0; it < 48; ++it) {
        const int M = 2 + (int)(rnd() * 31), N = 1 + (int)(rnd() * 70), K = 4 * (1 + (int)(rnd() * (it % 3 == 0 ? 700 : 40)));
        const bool bf16 = (it & 1) && K % 8 == 0 && M <= 16;
        std::vector<float> A = randn((size_t)M * K, 1.f), W = randn((size_t)N * K, 0.05f), C((size_t)M * N), R((size_t)M * N);
        std::vector<uint16_t> bits(W.size());
        if (bf16) {
            to_bf16_values(W);
            for (size_t i = 0; i < W.size(); ++i) {
                uint32_t u;
                memcpy(&u, &W[i], 4);
                bits[i] = (uint16_t)(u >> 16);
            }
        }
        void *dA, *dW, *dC;
        OK(lumen_malloc(ctx, A.size() * 4, &dA));
        OK(lumen_malloc(ctx, bf16 ? bits.size() * 2 : W.size() * 4, &dW));
        OK(lumen_malloc(ctx, C.size() * 4, &dC));
        OK(lumen_upload(ctx, dA, A.data(), A.size() * 4));
        if (bf16) OK(lumen_upload(ctx, dW, bits.data(), bits.size() * 2));
        else OK(lumen_upload(ctx, dW, W.data(), W.size() * 4));
        if (bf16) OK(lumen_gemm_bf16w(ctx, (const float *)dA, (const uint16_t *)dW, (float *)dC, M, N, K));
        else OK(lumen_matmul_f32(ctx, (const float *)dA, (const float *)dW, (float *)dC, M, N, K, K));
        OK(lumen_download(ctx, C.data(), dC, C.size() * 4));
        lo_gemm_f32(A.data(), W.data(), R.data(), M, N, K);
        const double e = max_rel(C.data(), R.data(), C.size());
        worst = e > worst ? e : worst;
        CHECK(e <= 1e-5, "product %d x %d x %d%s: %.3g", M, N, K, bf16 ? " bf16 weights" : "", e);
        OK(lumen_free(ctx, dA));
        OK(lumen_free(ctx, dW));
        OK(lumen_free(ctx, dC));
    }
    printf("  worst max rel err %.2e\n", worst);
}

int main(int argc, char **argv) {
    lo_set_threads(4);
    lumen_ctx *ctx = nullptr;
    OK(lumen_ctx_create(0, &ctx));
    if (argc == 2 && !strcmp(argv[1], "selfcheck-oob")) {
        selfcheck_oob(ctx);
        return 0;  // (reached only if nothing stopped the program: the test expects a sanitizer report instead)
    }
    struct { const char *name; void (*fn)(lumen_ctx *); } cases[] = {
        {"chain", case_chain}, {"sliced", case_sliced}, {"qknorm", case_qknorm}, {"bf16", case_bf16}, {"skinny", case_skinny}, {"attn", case_attn}, {"layerop", case_layerop}, {"shapes", case_shapes}};
    for (const auto &c : cases) {
        bool run = argc <= 1;
        for (int i = 1; i < argc; ++i) run = run || !strcmp(argv[i], c.name);
        if (run) c.fn(ctx);
    }
    lumen_ctx_destroy(ctx);
    if (g_failures) {
        fprintf(stderr, "%d check(s) failed\n", g_failures);
        return 1;
    }
    printf("cpu emulation: all checks passed\n");
    return 0;
}
