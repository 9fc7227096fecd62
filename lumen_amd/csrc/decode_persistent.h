// Arguments of the persistent decode kernel (decode_persistent.hip).
#pragma once

struct lumen_ctx;

struct PkLayer {
    const void *wqkv, *wo, *wgu, *wdown;  // [qd+2kvd,H] [H,qd] [2I,H] (gate/up rows interleaved) [H,I]
    const float *in_norm, *post_norm, *q_norm, *k_norm;
    float *k_cache, *v_cache;             // [Hkv, max_seq, D]
};

struct PkArgs {
    const PkLayer *layers;  // device array [n_layers]
    int n_layers;
    int H, I, V, qd, kvd, hq, hkv, D, max_seq, nsplit;
    float eps, scale;
    int w_bf16;
    const float *embed;      // [V,H] f32
    const void *lm_head;     // [V,H] weight dtype
    const float *final_norm;
    const float *cos_t, *sin_t;
    float *x, *h, *qkv, *attn, *act, *logits;
    float *part;             // [hq, nsplit, D+2]
    int *head_counters;      // [hkv], zero between launches
    int *tok, *pos;          // device state: next token id, its position
    unsigned *bar;           // grid barrier counter
    int *err;                // set when a barrier wait ran into its time limit
    float *amax_val;         // [workgroups]
    int *amax_idx;           // [workgroups]
    int n_steps;
    int *ids_out;            // [n_steps] or null
    float *logits_out;       // [n_steps, V] or null
    unsigned long long timeout_ticks;
};

bool pk_supported(const PkArgs &a);
int launch_decode_persistent(lumen_ctx *ctx, PkArgs &a);
