// Token sampling and the generation loop of one chat turn, src/main.rs:74-137
// and :325-378.  Host code, like the reference's: it works on the logits of
// the last position, which lumen_llama_forward has brought to the host.
//
// The reference draws its uniform number from an unseeded generator
// (rand01, main.rs:69-72); here the draw is an argument of the sampler and
// the generation loop takes it from a seeded splitmix64 stream, so a run can
// be repeated.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <vector>

#include "../../include/lumen_hip.h"

void lumen_set_error(const char *fmt, ...);

// splitmix64: state += golden gamma, output mixed; the top 24 bits make a float in [0, 1)
extern "C" float lumen_rand01(uint64_t *state) {
    uint64_t z = (*state += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    z ^= z >> 31;
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

extern "C" int lumen_sample_top_p_f32(const float *logits, int n, float temperature, float top_p,
                                      float repetition_penalty, const int32_t *recent, int n_recent, float r,
                                      int32_t *index_out) {
    if (!logits || !index_out || (n_recent > 0 && !recent)) {
        lumen_set_error("sample_top_p: null argument");
        return LUMEN_ERR_INVALID;
    }
    if (n <= 0) {
        lumen_set_error("sample_top_p: empty logits");
        return LUMEN_ERR_SHAPE;
    }
    std::vector<float> p(logits, logits + n);
    if (repetition_penalty > 1.0f)  // main.rs:84-89: divided whatever the sign
        for (int i = 0; i < n_recent; ++i)
            if (recent[i] >= 0 && recent[i] < n) p[recent[i]] /= repetition_penalty;
    const float temp = std::max(temperature, 1e-5f);  // :93
    float maxv = -INFINITY;
    for (int i = 0; i < n; ++i) {
        p[i] /= temp;
        if (p[i] != p[i]) {  // the reference's partial_cmp().unwrap() panics on NaN (:114)
            lumen_set_error("sample_top_p: logit %d is NaN", i);
            return LUMEN_ERR_INVALID;
        }
        if (p[i] > maxv) maxv = p[i];
    }
    float sum = 0.f;
    for (int i = 0; i < n; ++i) {  // :105-110
        p[i] = expf(p[i] - maxv);
        sum += p[i];
    }
    const float inv = 1.0f / (sum + 1e-9f);
    for (int i = 0; i < n; ++i) p[i] *= inv;

    // :113-126 sorts all indices by probability, descending and stable, and keeps the shortest prefix
    // whose running sum reaches the target.  Only that prefix is needed: sort the k largest (ties in
    // index order, which is what a stable sort leaves) and widen k until the prefix is inside.
    std::vector<int> idx(n);
    for (int i = 0; i < n; ++i) idx[i] = i;
    auto before = [&](int a, int b) { return p[a] > p[b] || (p[a] == p[b] && a < b); };
    const float target = std::max(std::min(std::max(top_p, 0.0f), 1.0f), 1e-6f);
    float cumulative = 0.f;
    int cut = 0;
    for (int k = std::min(n, 64);; k = std::min(n, k * 8)) {
        std::partial_sort(idx.begin(), idx.begin() + k, idx.end(), before);
        cumulative = 0.f;
        cut = 0;
        bool reached = false;
        for (int j = 0; j < k; ++j) {
            cumulative += p[idx[j]];
            cut = j + 1;
            if (cumulative >= target) {
                reached = true;
                break;
            }
        }
        if (reached || k == n) break;
    }
    if (cut < 1) cut = 1;
    float acc = 0.f;  // :129-137
    int pick = idx[cut - 1];
    for (int j = 0; j < cut; ++j) {
        acc += p[idx[j]] / cumulative;
        if (r <= acc) {
            pick = idx[j];
            break;
        }
    }
    *index_out = pick;
    return LUMEN_OK;
}

// One turn of the chat loop, main.rs:325-378, without the tokenizer: the caller passes the new
// tokens of the turn and the tokens already in the cache; text-based stops (:364-366) are the
// caller's business.
extern "C" int lumen_llama_generate_turn(lumen_llama *m, const int32_t *new_tokens, int n_new, const int32_t *history,
                                         int n_history, const lumen_sampling *sp, const int32_t *stop_ids, int n_stop,
                                         int32_t *out_ids, int out_cap, int *n_out) {
    if (n_out) *n_out = 0;
    if (!m || !new_tokens || !sp || !out_ids || !n_out || (n_history > 0 && !history) || (n_stop > 0 && !stop_ids)) {
        lumen_set_error("llama_generate_turn: null argument");
        return LUMEN_ERR_INVALID;
    }
    if (n_new <= 0) {
        lumen_set_error("llama_generate_turn: empty turn");
        return LUMEN_ERR_SHAPE;
    }
    lumen_llama_config cfg;
    int rc = lumen_llama_get_config(m, &cfg);
    if (rc != LUMEN_OK) return rc;
    int cur = 0;
    rc = lumen_llama_kv_len(m, &cur);
    if (rc != LUMEN_OK) return rc;
    if (cur + n_new + 8 >= cfg.max_seq_len) {  // :266: the reference resets and rebuilds the prompt here
        lumen_set_error("KV cache overflow: len=%d + %d new tokens + 8 >= max_seq=%d (reset and start a first turn)", cur,
                        n_new, cfg.max_seq_len);
        return LUMEN_ERR_KV_OVERFLOW;
    }
    std::vector<int32_t> all(history, history + (n_history > 0 ? n_history : 0));
    all.insert(all.end(), new_tokens, new_tokens + n_new);
    std::vector<float> ids(n_new), logits((size_t)cfg.vocab_size);
    for (int i = 0; i < n_new; ++i) ids[i] = (float)new_tokens[i];  // tensor_from_token_ids, :143-152
    rc = lumen_llama_forward(m, ids.data(), n_new, logits.data(), 0);
    if (rc != LUMEN_OK) return rc;
    uint64_t state = sp->seed;
    const int window = sp->recent_window > 0 ? sp->recent_window : 0;
    for (int g = 0; g < sp->max_gen && *n_out < out_cap; ++g) {
        const size_t start = all.size() > (size_t)window ? all.size() - (size_t)window : 0;  // :337-338
        int32_t next = 0;
        rc = lumen_sample_top_p_f32(logits.data(), cfg.vocab_size, sp->temperature, sp->top_p, sp->repetition_penalty,
                                    all.data() + start, (int)(all.size() - start), lumen_rand01(&state), &next);
        if (rc != LUMEN_OK) return rc;
        bool stop = false;
        for (int i = 0; i < n_stop; ++i) stop |= (stop_ids[i] == next);
        if (stop) break;  // :348-350
        all.push_back(next);
        out_ids[(*n_out)++] = next;
        const float one = (float)next;
        rc = lumen_llama_forward(m, &one, 1, logits.data(), 0);  // :361-367
        if (rc != LUMEN_OK) return rc;
        rc = lumen_llama_kv_len(m, &cur);
        if (rc != LUMEN_OK) return rc;
        if (cur + 2 >= cfg.max_seq_len) break;  // :370-372
    }
    return LUMEN_OK;
}
