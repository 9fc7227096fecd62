// Parity tests of the C++ host layer (include/lumen.hpp) against the CPU checker
// (oracle/lumen_oracle.h).  The host layer only routes to the C ABI, so every check
// below goes through liblumen_hip.so.
//
//   test_host              all checks; needs an MI355X
//   test_host --host-only  the checks that touch no device
//
// Tolerances: GEMV / elementwise max|d| / max|ref| <= 1e-5; logits <= 1e-4 (fp32).
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/lumen.hpp"
#include "../../oracle/lumen_oracle.h"

using namespace lumen;

static int g_failed = 0, g_checks = 0;
#define EXPECT(cond, ...)                                   \
    do {                                                    \
        ++g_checks;                                         \
        if (!(cond)) {                                      \
            ++g_failed;                                     \
            std::printf("FAIL %s:%d: ", __FILE__, __LINE__); \
            std::printf(__VA_ARGS__);                       \
            std::printf("\n");                              \
        }                                                   \
    } while (0)

template <class F> static int status_of(F &&f) {
    try {
        f();
    } catch (const Error &e) {
        return e.status();
    }
    return LUMEN_OK;
}

// deterministic values, roughly N(0, std): sum of four uniforms from a 64-bit LCG
struct Gen {
    uint64_t s;
    explicit Gen(uint64_t seed) : s(seed * 2862933555777941757ull + 3037000493ull) {}
    float uni() {
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        return (float)(s >> 40) * (1.0f / 16777216.0f);
    }
    float normal(float std) { return (uni() + uni() + uni() + uni() - 2.0f) * 1.7320508f * std; }
    std::vector<float> vec(size_t n, float std) {
        std::vector<float> v(n);
        for (auto &x : v) x = normal(std);
        return v;
    }
};

static double rel_err(const std::vector<float> &got, const float *ref, size_t n) {
    double worst = 0, scale = 0;
    for (size_t i = 0; i < n; ++i) {
        worst = std::max(worst, (double)std::fabs(got[i] - ref[i]));
        scale = std::max(scale, (double)std::fabs(ref[i]));
    }
    return scale > 0 ? worst / scale : worst;
}
static double rel_err(const std::vector<float> &got, const std::vector<float> &ref) {
    return got.size() == ref.size() ? rel_err(got, ref.data(), ref.size()) : 1e30;
}

// ------------------------------------------------------------------ no device needed
static void test_mode_flags() {
    set_inference_mode(false);
    EXPECT(!is_no_grad(), "grad mode is the default");
    {
        NoGradGuard g;
        EXPECT(is_no_grad(), "guard");
        no_grad([] { EXPECT(is_no_grad(), "nested"); });
        EXPECT(is_no_grad(), "still inside the outer guard");
    }
    EXPECT(!is_no_grad(), "guard released");
    set_inference_mode(true);
    EXPECT(is_no_grad() && is_inference_mode(), "inference mode");
    set_inference_mode(false);
}

static void test_sampler_matches_checker() {
    Gen g(7);
    std::vector<float> logits = g.vec(500, 2.0f);
    std::vector<int32_t> recent = {3, 17, 17, 499, 250};
    std::vector<int> recent_i(recent.begin(), recent.end());
    for (int i = 0; i < 64; ++i) {
        const float r = g.uni(), temp = 0.2f + 1.5f * g.uni(), top_p = g.uni(), pen = 1.0f + 0.3f * g.uni();
        const int want = lo_sample_top_p(logits.data(), 500, temp, top_p, pen, recent_i.data(), 5, r);
        const int got = sample_top_p(logits, temp, top_p, pen, recent, r);
        EXPECT(got == want, "sample_top_p draw %d: %d vs %d", i, got, want);
    }
    std::vector<float> bad = logits;
    bad[9] = NAN;
    EXPECT(status_of([&] { sample_top_p(bad, 1.f, 0.9f, 1.f, {}, 0.5f); }) == LUMEN_ERR_INVALID, "NaN logit");
}

// ---------------------------------------------------------------------------- device
static void test_ops() {
    Gen g(1);
    const size_t K = 300, N = 77, M = 9;
    std::vector<float> w = g.vec(N * K, 0.05f), x = g.vec(K, 1.f), a = g.vec(M * K, 1.f);
    Tensor W = Tensor::from_vec(w, {N, K});
    // one row: GEMV, output shape keeps the leading dimensions
    Tensor y = ops::matmul(Tensor::from_vec(x, {1, 1, K}), W);
    EXPECT((y.shape() == std::vector<size_t>{1, 1, N}), "matmul output shape");
    std::vector<float> ref(N);
    lo_gemv_f32(w.data(), x.data(), ref.data(), (int)N, (int)K);
    EXPECT(rel_err(y.data(), ref) <= 1e-5, "GEMV rel err %.2e", rel_err(y.data(), ref));
    // several rows: GEMM
    Tensor c = ops::matmul(Tensor::from_vec(a, {1, M, K}), W);
    std::vector<float> refc(M * N);
    lo_gemm_f32(a.data(), w.data(), refc.data(), (int)M, (int)N, (int)K);
    EXPECT(rel_err(c.data(), refc) <= 1e-5, "GEMM rel err %.2e", rel_err(c.data(), refc));
    // the reference's panics
    EXPECT(status_of([&] { ops::matmul(Tensor::from_vec(x, {1, K}), Tensor::from_vec(w, {N, K / 2, 2})); }) == LUMEN_ERR_SHAPE,
           "RHS must be 2-D");
    EXPECT(status_of([&] { ops::matmul(Tensor::from_vec(g.vec(K - 1, 1.f), {1, K - 1}), W); }) == LUMEN_ERR_SHAPE,
           "K mismatch");

    std::vector<float> p = g.vec(1000, 1.f), q = g.vec(1000, 1.f), r(1000);
    Tensor P = Tensor::from_vec(p, {10, 100}), Q = Tensor::from_vec(q, {10, 100});
    lo_add_f32(p.data(), q.data(), r.data(), 1000);
    EXPECT((P + Q).data() == r, "add is exact");
    lo_mul_f32(p.data(), q.data(), r.data(), 1000);
    EXPECT((P * Q).data() == r, "mul is exact");
    EXPECT(status_of([&] { P + Tensor::from_vec(q, {100, 10}); }) == LUMEN_ERR_SHAPE, "add shape");
    lo_silu_f32(p.data(), r.data(), 1000);
    EXPECT(rel_err(SiLU().forward(P).data(), r) <= 1e-6, "SiLU");

    RMSNorm norm(100, 1e-5f);
    std::vector<float> gain = g.vec(100, 1.f);
    norm.weight.set_raw_data({100}, gain);
    lo_rmsnorm_f32(p.data(), gain.data(), r.data(), 10, 100, 1e-5f);
    EXPECT(rel_err(norm.forward(P).data(), r) <= 1e-6, "RMSNorm rel err %.2e", rel_err(norm.forward(P).data(), r));
    EXPECT(status_of([&] { norm.forward(Tensor::from_vec(p, {100, 10})); }) == LUMEN_ERR_SHAPE, "RMSNorm dim");

    Embedding emb(50, 20);
    std::vector<float> table = g.vec(1000, 1.f);
    emb.weight.set_raw_data({50, 20}, table);
    std::vector<float> ids = {49, 0, 7, 7};
    Tensor e = emb.forward(Tensor::from_vec(ids, {1, 4}));
    EXPECT((e.shape() == std::vector<size_t>{1, 4, 20}), "embedding shape");
    std::vector<float> eref(80);
    lo_embedding_f32(table.data(), ids.data(), 4, 50, 20, eref.data());
    EXPECT(e.data() == eref, "embedding rows");
    EXPECT(status_of([&] { emb.forward(Tensor::from_vec({50.f}, {1, 1})); }) == LUMEN_ERR_EMBED_OOB, "embedding OOB");

    // handles share data; reshape is a view; detach is a copy
    Tensor view = P.reshape({-1, 50});
    EXPECT((view.shape() == std::vector<size_t>{20, 50}) && view.same_storage(P), "reshape view");
    EXPECT(status_of([&] { P.reshape({7, -1, -1}); }) == LUMEN_ERR_SHAPE, "two -1");
    EXPECT(status_of([&] { P.reshape({7, 11}); }) == LUMEN_ERR_SHAPE, "count mismatch");
    Tensor copy = P.detach(), alias = P;
    P.set_raw_data({1000}, q);
    EXPECT(alias.data() == q && alias.shape() == std::vector<size_t>{1000}, "clones see set_raw_data");
    EXPECT(copy.data() == p && !copy.same_storage(P), "detach copied");
}

static void test_rope() {
    const size_t D = 32, MAXS = 40;
    RotaryEmbedding rope(D, MAXS, 10000.f);
    std::vector<float> cos_t(MAXS * D), sin_t(MAXS * D);
    lo_rope_table(cos_t.data(), sin_t.data(), (int)D, (int)MAXS, 10000.f);
    auto [c, s] = rope.cos_sin_row_vec(17);
    EXPECT(std::equal(c.begin(), c.end(), cos_t.begin() + 17 * D) && std::equal(s.begin(), s.end(), sin_t.begin() + 17 * D),
           "table row 17 equals the checker's bit for bit");
    EXPECT(status_of([&] { rope.cos_sin_row_vec(MAXS); }) == LUMEN_ERR_ROPE_RANGE, "row out of range");

    Gen g(2);
    const int B = 1, H = 3, S = 5;
    std::vector<float> x = g.vec(B * H * S * D, 1.f), ref(x.size());
    lo_rope_forward(x.data(), ref.data(), cos_t.data(), sin_t.data(), B, H, S, (int)D, 30, (int)MAXS);
    Tensor out = rope.forward(Tensor::from_vec(x, {(size_t)B, (size_t)H, (size_t)S, D}), 30);
    EXPECT(rel_err(out.data(), ref) <= 1e-6, "RoPE forward rel err %.2e", rel_err(out.data(), ref));
    EXPECT(status_of([&] { rope.forward(Tensor::from_vec(x, {(size_t)B, (size_t)H, (size_t)S, D}), MAXS - S + 1); }) ==
               LUMEN_ERR_ROPE_RANGE,
           "offset + S beyond the table");
    std::vector<float> v = g.vec(D, 1.f), dst, dref(D);
    rope.rope_1token_copy(v, dst, 39);
    lo_rope_1token_copy(v.data(), dref.data(), cos_t.data(), sin_t.data(), (int)D, 39, (int)MAXS);
    EXPECT(rel_err(dst, dref) <= 1e-6, "rope_1token_copy");
    EXPECT(status_of([&] { rope.rope_1token_copy(v, dst, MAXS); }) == LUMEN_ERR_ROPE_RANGE, "pos out of range");
}

static LlamaConfig tiny_config() {
    LlamaConfig c;
    c.vocab_size = 300;
    c.hidden_size = 128;
    c.intermediate_size = 352;
    c.num_hidden_layers = 3;
    c.num_attention_heads = 4;
    c.num_key_value_heads = 2;
    c.max_seq_len = 24;
    return c;
}

// the checker's model over the same host arrays
struct CheckerModel {
    lo_llama *m;
    explicit CheckerModel(const LlamaConfig &c, const std::unordered_map<std::string, std::vector<float>> &w) {
        lo_llama_config oc{};
        oc.vocab_size = (int)c.vocab_size;
        oc.hidden_size = (int)c.hidden_size;
        oc.intermediate_size = (int)c.intermediate_size;
        oc.num_hidden_layers = (int)c.num_hidden_layers;
        oc.num_attention_heads = (int)c.num_attention_heads;
        oc.num_key_value_heads = (int)c.num_key_value_heads;
        oc.rms_norm_eps = c.rms_norm_eps;
        oc.max_seq_len = (int)c.max_seq_len;
        oc.rope_theta = c.rope_theta;
        m = lo_llama_new(&oc);
        lo_llama_set_globals(m, w.at("model.embed_tokens.weight").data(), w.at("model.norm.weight").data(),
                             w.at("lm_head.weight").data());
        for (size_t i = 0; i < c.num_hidden_layers; ++i) {
            const std::string p = "model.layers." + std::to_string(i);
            lo_llama_layer l{};
            l.wq = w.at(p + ".self_attn.q_proj.weight").data();
            l.wk = w.at(p + ".self_attn.k_proj.weight").data();
            l.wv = w.at(p + ".self_attn.v_proj.weight").data();
            l.wo = w.at(p + ".self_attn.o_proj.weight").data();
            l.w_gate = w.at(p + ".mlp.gate_proj.weight").data();
            l.w_up = w.at(p + ".mlp.up_proj.weight").data();
            l.w_down = w.at(p + ".mlp.down_proj.weight").data();
            l.input_norm = w.at(p + ".input_layernorm.weight").data();
            l.post_norm = w.at(p + ".post_attention_layernorm.weight").data();
            lo_llama_set_layer(m, (int)i, &l);
        }
    }
    ~CheckerModel() { lo_llama_free(m); }
};

static std::unordered_map<std::string, std::vector<float>> fill_model(LlamaModel &model, uint64_t seed) {
    std::unordered_map<std::string, std::vector<float>> host;
    Gen g(seed);
    // sorted names so that the values do not depend on the hash map's order
    std::vector<std::string> names;
    auto params = model.named_parameters();
    for (auto &kv : params) names.push_back(kv.first);
    std::sort(names.begin(), names.end());
    for (const auto &name : names) {
        Tensor t = params.at(name);
        const bool gain = name.find("norm") != std::string::npos;
        std::vector<float> v = g.vec(t.len(), gain ? 0.1f : 0.08f);
        if (gain)
            for (auto &x : v) x += 1.0f;
        t.set_raw_data(t.shape(), v);
        host[name] = std::move(v);
    }
    return host;
}

static void test_llama_model_and_engine() {
    const LlamaConfig cfg = tiny_config();
    LlamaModel model(cfg);
    EXPECT(model.named_parameters().size() == 3 + 9 * cfg.num_hidden_layers, "named_parameters count");
    EXPECT(model.parameters().size() == model.named_parameters().size(), "parameters count");
    auto host = fill_model(model, 5);
    CheckerModel checker(cfg, host);
    const size_t V = cfg.vocab_size;

    Gen g(11);
    std::vector<float> ids(12);
    for (auto &t : ids) t = (float)(int)(g.uni() * (float)V);

    NoGradGuard guard;
    std::vector<KVCache> caches = model.init_kv_caches(1);
    EXPECT(caches.size() == cfg.num_hidden_layers && caches[0]->len() == 0, "fresh caches");
    {
        std::vector<KVCache> few(caches.begin(), caches.begin() + 2);
        EXPECT(status_of([&] { model.forward(Tensor::from_vec({1.f}, {1, 1}), few, 0); }) == LUMEN_ERR_CACHE_COUNT,
               "cache count mismatch");
    }
    // prefill 8 tokens: all rows, as the reference computes them
    const size_t S0 = 8;
    std::vector<float> ref(S0 * V);
    EXPECT(lo_llama_forward(checker.m, ids.data(), (int)S0, ref.data()) == LO_OK, "checker prefill");
    Tensor logits = model.forward(Tensor::from_vec(std::vector<float>(ids.begin(), ids.begin() + S0), {1, S0}), caches, 0);
    EXPECT((logits.shape() == std::vector<size_t>{1, S0, V}), "logits shape");
    double worst = rel_err(logits.data(), ref);
    EXPECT(worst <= 1e-4, "prefill logits rel err %.2e", worst);
    EXPECT(caches[2]->len() == S0, "cache length after prefill");
    // then one token at a time
    std::vector<std::vector<float>> step_logits;
    for (size_t t = S0; t < ids.size(); ++t) {
        std::vector<float> r1(V);
        EXPECT(lo_llama_forward(checker.m, &ids[t], 1, r1.data()) == LO_OK, "checker decode");
        Tensor l1 = model.forward(Tensor::from_vec({ids[t]}, {1, 1}), caches, 0);
        const double e = rel_err(l1.data(), r1);
        EXPECT(e <= 1e-4, "decode step %zu logits rel err %.2e", t, e);
        worst = std::max(worst, e);
        step_logits.push_back(r1);
    }
    // the cache holds RoPE(k) and v at every position filled so far
    const size_t D = cfg.hidden_size / cfg.num_attention_heads;
    const size_t cache_elems = cfg.num_key_value_heads * cfg.max_seq_len * D;
    for (size_t layer : {(size_t)0, cfg.num_hidden_layers - 1}) {
        std::vector<float> k = caches[layer]->k(), v = caches[layer]->v();
        double ek = 0, ev = 0;
        for (size_t hk = 0; hk < cfg.num_key_value_heads; ++hk)
            for (size_t i = 0; i < ids.size() * D; ++i) {
                const size_t at = hk * cfg.max_seq_len * D + i;
                ek = std::max(ek, (double)std::fabs(k[at] - lo_llama_cache_k(checker.m, (int)layer)[at]));
                ev = std::max(ev, (double)std::fabs(v[at] - lo_llama_cache_v(checker.m, (int)layer)[at]));
            }
        EXPECT(k.size() == cache_elems && ek <= 1e-4 && ev <= 1e-4, "layer %zu cache |dk| %.2e |dv| %.2e", layer, ek, ev);
    }
    // the cache holds 24 positions.  A prompt that would pass the end fails in RoPE, whose table is as
    // long as the cache and is consulted first (encoding.rs:63-68 before self_attention.rs:341-346);
    // a single token at a full cache fails the cache's own check (:144-149)
    {
        std::vector<float> many(cfg.max_seq_len - ids.size() + 1, 1.f);
        EXPECT(status_of([&] { model.forward(Tensor::from_vec(many, {1, many.size()}), caches, 0); }) == LUMEN_ERR_ROPE_RANGE,
               "prompt beyond the end of the cache");
        many.pop_back();
        model.forward(Tensor::from_vec(many, {1, many.size()}), caches, 0);
        EXPECT(caches[0]->len() == cfg.max_seq_len, "cache filled to the end");
        EXPECT(status_of([&] { model.forward(Tensor::from_vec({1.f}, {1, 1}), caches, 0); }) == LUMEN_ERR_KV_OVERFLOW,
               "KV overflow");
    }
    model.reset_kv_caches(caches);
    EXPECT(caches[0]->len() == 0 && caches[1]->len() == 0, "reset");
    std::printf("  LlamaModel (operator level): worst logits rel err %.2e\n", worst);

    // the fused engine built from the same parameters
    LlamaEngine engine(model);
    std::vector<float> el = engine.forward(std::vector<float>(ids.begin(), ids.begin() + S0), true);
    double ew = rel_err(el, ref);
    EXPECT(ew <= 1e-4, "engine prefill logits rel err %.2e", ew);
    for (size_t t = S0; t < ids.size(); ++t) {
        std::vector<float> l1 = engine.forward({ids[t]});
        const double e = rel_err(l1, step_logits[t - S0]);
        EXPECT(e <= 1e-4, "engine decode step %zu rel err %.2e", t, e);
        ew = std::max(ew, e);
    }
    EXPECT(engine.kv_len() == ids.size(), "engine cache length");
    std::printf("  LlamaEngine (model level): worst logits rel err %.2e\n", ew);
    // greedy generation on the device equals argmax of step-by-step logits
    engine.reset_kv_caches();
    std::vector<int32_t> picks = engine.decode_greedy((int32_t)ids[0], 6);
    engine.reset_kv_caches();
    int32_t tok = (int32_t)ids[0];
    for (int i = 0; i < 6; ++i) {
        std::vector<float> l1 = engine.forward({(float)tok});
        tok = (int32_t)(std::max_element(l1.begin(), l1.end()) - l1.begin());
        EXPECT(picks[i] == tok, "greedy pick %d: %d vs %d", i, picks[i], tok);
    }
    // a sampled turn: reproducible from its seed, stops at a stop id
    lumen_sampling sp{0.8f, 0.9f, 1.05f, 96, 5, 1234};
    engine.reset_kv_caches();
    std::vector<int32_t> prompt = {5, 9, 250};
    std::vector<int32_t> turn1 = engine.generate_turn(prompt, {}, sp, {});
    engine.reset_kv_caches();
    std::vector<int32_t> turn2 = engine.generate_turn(prompt, {}, sp, {});
    EXPECT(turn1.size() == 5 && turn1 == turn2, "seeded turn repeats");
    engine.reset_kv_caches();
    std::vector<int32_t> stopped = engine.generate_turn(prompt, {}, sp, {turn1[2]});
    EXPECT(stopped.size() <= 2 && std::equal(stopped.begin(), stopped.end(), turn1.begin()), "stop id ends the turn");
}

static void test_self_attention_modes() {
    SelfAttention att(64, 4, 2, 16, 10000.f, true);
    Tensor x = Tensor::from_vec(Gen(3).vec(64, 1.f), {1, 1, 64});
    set_inference_mode(false);
    EXPECT(status_of([&] { att.forward(x, std::nullopt); }) == LUMEN_ERR_UNSUPPORTED, "training path refused");
    EXPECT(status_of([] { SelfAttention(65, 4, 2, 16, 10000.f, true); }) == LUMEN_ERR_SHAPE, "embed dim vs heads");
    NoGradGuard guard;
    auto [out, cache] = att.forward(x, std::nullopt);  // a cache is made when none is given
    EXPECT(cache && (*cache)->len() == 1 && (out.shape() == std::vector<size_t>{1, 1, 64}), "cache created on demand");
    auto [out2, cache2] = att.forward(x, cache);
    EXPECT(cache2 && *cache2 == *cache && (*cache)->len() == 2, "same cache handed back");
    (void)out2;
}

// ---- safetensors: a file written here, read through ModelLoader
static void put_tensor(std::string &json, std::vector<unsigned char> &blob, const std::string &name, const char *dtype,
                       const std::vector<size_t> &shape, const void *bytes, size_t nbytes) {
    if (json.size() > 1) json += ",";
    json += "\"" + name + "\":{\"dtype\":\"" + dtype + "\",\"shape\":[";
    for (size_t i = 0; i < shape.size(); ++i) json += (i ? "," : "") + std::to_string(shape[i]);
    json += "],\"data_offsets\":[" + std::to_string(blob.size()) + "," + std::to_string(blob.size() + nbytes) + "]}";
    blob.insert(blob.end(), (const unsigned char *)bytes, (const unsigned char *)bytes + nbytes);
}
static void write_file(const std::string &path, std::string json, const std::vector<unsigned char> &blob) {
    json += "}";
    std::FILE *f = std::fopen(path.c_str(), "wb");
    uint64_t n = json.size();
    std::fwrite(&n, 8, 1, f);
    std::fwrite(json.data(), 1, json.size(), f);
    std::fwrite(blob.data(), 1, blob.size(), f);
    std::fclose(f);
}

static void test_loader(const std::string &dir) {
    LlamaConfig cfg = tiny_config();
    cfg.num_hidden_layers = 1;
    LlamaModel model(cfg);
    auto params = model.named_parameters();
    Gen g(21);
    std::string json = "{";
    std::vector<unsigned char> blob;
    std::unordered_map<std::string, std::vector<float>> want;
    const std::string skipped = "model.layers.0.mlp.up_proj.weight", as_bf16 = "model.layers.0.self_attn.q_proj.weight";
    for (auto &[name, t] : params) {
        if (name == skipped) continue;
        std::vector<float> v = g.vec(t.len(), 0.05f);
        if (name == as_bf16) {
            std::vector<uint16_t> bits(v.size());
            lo_f32_to_bf16_rne(v.data(), bits.data(), (long)v.size());
            lo_bf16_to_f32(bits.data(), v.data(), (long)v.size());
            put_tensor(json, blob, name, "BF16", t.shape(), bits.data(), bits.size() * 2);
        } else {
            put_tensor(json, blob, name, "F32", t.shape(), v.data(), v.size() * 4);
        }
        want[name] = v;
    }
    const std::string path = dir + "/host_cpp_model.safetensors";
    write_file(path, json, blob);
    auto [loaded, missing] = ModelLoader::load_llama_weights(path, params);
    EXPECT(loaded == (int)params.size() - 1 && missing == 1, "loaded %d missing %d", loaded, missing);
    bool same = true;
    for (auto &[name, v] : want) same = same && params.at(name).data() == v;
    EXPECT(same, "every loaded tensor holds the file's values (bf16 widened exactly)");
    EXPECT(model.layers[0].mlp.up_proj.weight.data() == std::vector<float>(cfg.intermediate_size * cfg.hidden_size, 0.f),
           "the tensor the file lacks is left as it was");
    // the engine reads the same file
    LlamaEngine engine(LlamaEngine::to_c_config(cfg));
    auto [l2, m2] = engine.load_safetensors(path);
    EXPECT(l2 == loaded && m2 == missing, "engine loader counts");

    // element count mismatch and an unsupported dtype
    std::string j2 = "{";
    std::vector<unsigned char> b2;
    std::vector<float> shorter(10, 1.f);
    put_tensor(j2, b2, "model.norm.weight", "F32", {10}, shorter.data(), 40);
    write_file(dir + "/host_cpp_bad_shape.safetensors", j2, b2);
    EXPECT(status_of([&] { ModelLoader::load_llama_weights(dir + "/host_cpp_bad_shape.safetensors", params); }) == LUMEN_ERR_SHAPE,
           "shape mismatch");
    std::string j3 = "{";
    std::vector<unsigned char> b3;
    std::vector<uint16_t> halfs(cfg.hidden_size, 0x3c00);
    put_tensor(j3, b3, "model.norm.weight", "F16", {cfg.hidden_size}, halfs.data(), halfs.size() * 2);
    write_file(dir + "/host_cpp_bad_dtype.safetensors", j3, b3);
    EXPECT(status_of([&] { ModelLoader::load_llama_weights(dir + "/host_cpp_bad_dtype.safetensors", params); }) == LUMEN_ERR_INVALID,
           "unsupported dtype");
    EXPECT(status_of([&] { ModelLoader::load_llama_weights(dir + "/no_such_file", params); }) == LUMEN_ERR_INVALID, "missing file");
    for (const char *f : {"/host_cpp_model.safetensors", "/host_cpp_bad_shape.safetensors", "/host_cpp_bad_dtype.safetensors"})
        std::remove((dir + f).c_str());
}

static void test_legacy_cache() {
    LlamaKVCache cache(16, 2, 8);
    Gen g(4);
    std::vector<float> k = g.vec(2 * 3 * 8, 1.f), v = g.vec(2 * 3 * 8, 1.f);
    cache.update(Tensor::from_vec(k, {1, 2, 3, 8}), Tensor::from_vec(v, {1, 2, 3, 8}), 4);
    auto [kv, vv] = cache.get_view(7);
    std::vector<float> kd = kv.data(), vd = vv.data();
    bool ok = kv.shape() == std::vector<size_t>{1, 2, 7, 8};
    for (size_t h = 0; h < 2 && ok; ++h)
        for (size_t s = 0; s < 7; ++s)
            for (size_t i = 0; i < 8; ++i) {
                const float wk = s < 4 ? 0.f : k[(h * 3 + (s - 4)) * 8 + i], wv = s < 4 ? 0.f : v[(h * 3 + (s - 4)) * 8 + i];
                ok = ok && kd[(h * 7 + s) * 8 + i] == wk && vd[(h * 7 + s) * 8 + i] == wv;
            }
    EXPECT(ok, "update at start_pos 4, view of 7 positions");
    EXPECT(status_of([&] { cache.update(Tensor::from_vec(k, {1, 2, 3, 8}), Tensor::from_vec(v, {1, 2, 3, 8}), 14); }) ==
               LUMEN_ERR_KV_OVERFLOW,
           "legacy cache overflow");
}

int main(int argc, char **argv) {
    const bool host_only = argc > 1 && std::strcmp(argv[1], "--host-only") == 0;
    const char *tmp = std::getenv("TMPDIR");
    const std::string dir = tmp && *tmp ? tmp : "/tmp";
    struct Case {
        const char *name;
        void (*fn)();
        bool device;
    };
    static std::string g_dir;
    g_dir = dir;
    const Case cases[] = {
        {"mode flags", test_mode_flags, false},
        {"sampler", test_sampler_matches_checker, false},
        {"ops", test_ops, true},
        {"rope", test_rope, true},
        {"self attention modes", test_self_attention_modes, true},
        {"legacy cache", test_legacy_cache, true},
        {"loader", [] { test_loader(g_dir); }, true},
        {"llama model and engine", test_llama_model_and_engine, true},
    };
    for (const Case &c : cases) {
        if (host_only && c.device) continue;
        std::printf("[ RUN ] %s\n", c.name);
        std::fflush(stdout);
        const int before = g_failed;
        try {
            c.fn();
        } catch (const std::exception &e) {
            ++g_failed;
            std::printf("FAIL %s: unexpected exception: %s\n", c.name, e.what());
        }
        std::printf("[ %s ] %s\n", g_failed == before ? " OK " : "FAIL", c.name);
        std::fflush(stdout);
    }
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed ? 1 : 0;
}
