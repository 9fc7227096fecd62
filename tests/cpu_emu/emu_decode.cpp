// CPU run of the persistent decode kernel (lumen_amd/csrc/decode_persistent_device.h) on a small
// model: every GPU thread is an OS thread, workgroups run concurrently so the grid barrier, the
// cross-barrier weight prefetch and the split-attention merge execute exactly as written.  The
// logits and greedy picks are checked against the CPU oracle on the same weights.  Built with
// AddressSanitizer, so an out-of-bounds access in the kernel's addressing aborts the run.
//
//   emu_decode <H> <I> <V> <Hq> <Hkv> <D> <layers> <max_seq> <qk_norm> <bf16> <steps> <nblocks> <start_pos>
#include "hip_cpu_shim.h"

thread_local dim3 threadIdx, blockIdx;
dim3 gridDim, blockDim;
thread_local EmuBlock *emu_block;

#include "../../lumen_amd/csrc/decode_persistent_device.h"
#include "../../oracle/lumen_oracle.h"

#include <cstdio>
#include <cstdlib>
#include <memory>

template <typename T>
static T *alloc(size_t n) { return (T *)calloc(n ? n : 1, sizeof(T)); }

static uint32_t g_rng = 12345u;
static float frand() {  // uniform in [-1, 1)
    g_rng = g_rng * 1664525u + 1013904223u;
    return (float)((g_rng >> 8) & 0xffffff) / 8388608.0f - 1.0f;
}
static float *rand_mat(size_t n, float scale) {
    float *p = alloc<float>(n);
    for (size_t i = 0; i < n; ++i) p[i] = frand() * scale;
    return p;
}

struct ThreadArg {
    PkArgs args;
    EmuBlock *blk;
    unsigned bx, tx;
    int D, nrep, bf16;
};

template <int D, int NREP>
static void run_kernel(const PkArgs &a, int bf16) {
    if (bf16) decode_persistent_kernel<D, NREP, true>(a);
    else decode_persistent_kernel<D, NREP, false>(a);
}

static void *thread_main(void *p) {
    ThreadArg *t = (ThreadArg *)p;
    threadIdx.x = t->tx;
    blockIdx.x = t->bx;
    emu_block = t->blk;
    const int key = t->D * 100 + t->nrep;
    switch (key) {
        case 6401: run_kernel<64, 1>(t->args, t->bf16); break;
        case 6402: run_kernel<64, 2>(t->args, t->bf16); break;
        case 6404: run_kernel<64, 4>(t->args, t->bf16); break;
        case 6408: run_kernel<64, 8>(t->args, t->bf16); break;
        case 12801: run_kernel<128, 1>(t->args, t->bf16); break;
        case 12802: run_kernel<128, 2>(t->args, t->bf16); break;
        default: fprintf(stderr, "unsupported D/nrep %d\n", key); exit(2);
    }
    return nullptr;
}

static uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

int main(int argc, char **argv) {
    if (argc != 14) {
        fprintf(stderr, "usage: emu_decode H I V Hq Hkv D layers max_seq qk_norm bf16 steps nblocks start_pos\n");
        return 2;
    }
    const int H = atoi(argv[1]), I = atoi(argv[2]), V = atoi(argv[3]), Hq = atoi(argv[4]), Hkv = atoi(argv[5]);
    const int D = atoi(argv[6]), L = atoi(argv[7]), max_seq = atoi(argv[8]), qk_norm = atoi(argv[9]);
    const int bf16 = atoi(argv[10]), steps = atoi(argv[11]), nblocks = atoi(argv[12]), start_pos = atoi(argv[13]);
    const int qd = Hq * D, kvd = Hkv * D, qkvd = qd + 2 * kvd, nrep = Hq / Hkv;
    const size_t esz = bf16 ? 2 : 4;

    // ---- weights (f32 masters; bf16 copies are rounded and the masters replaced by the rounded values)
    auto quant = [&](float *w, size_t n) -> void * {
        if (!bf16) return w;
        uint16_t *b = alloc<uint16_t>(n);
        for (size_t i = 0; i < n; ++i) {
            b[i] = to_bf16(w[i]);
            w[i] = from_bf16(b[i]);
        }
        return b;
    };
    float *embed = rand_mat((size_t)V * H, 0.3f);
    float *lm_head_f = rand_mat((size_t)V * H, 0.2f);
    void *lm_head = quant(lm_head_f, (size_t)V * H);
    float *final_norm = rand_mat(H, 0.1f);
    for (int i = 0; i < H; ++i) final_norm[i] += 1.f;
    std::vector<PkLayer> layers(L);
    std::vector<lo_llama_layer> olayers(L);
    const size_t cache_stride = (size_t)Hkv * max_seq * D;
    float *k_slab = alloc<float>(cache_stride * L), *v_slab = alloc<float>(cache_stride * L);
    for (int l = 0; l < L; ++l) {
        float *wq = rand_mat((size_t)qd * H, 0.15f), *wk = rand_mat((size_t)kvd * H, 0.15f), *wv = rand_mat((size_t)kvd * H, 0.15f);
        float *wo = rand_mat((size_t)H * qd, 0.15f), *wg = rand_mat((size_t)I * H, 0.15f), *wu = rand_mat((size_t)I * H, 0.15f);
        float *wd = rand_mat((size_t)H * I, 0.15f);
        float *n1 = rand_mat(H, 0.1f), *n2 = rand_mat(H, 0.1f), *qn = rand_mat(D, 0.1f), *kn = rand_mat(D, 0.1f);
        for (int i = 0; i < H; ++i) { n1[i] += 1.f; n2[i] += 1.f; }
        for (int i = 0; i < D; ++i) { qn[i] += 1.f; kn[i] += 1.f; }
        // fused layouts: q|k|v rows concatenated, gate/up rows interleaved
        float *wqkv = alloc<float>((size_t)qkvd * H), *wgu = alloc<float>((size_t)2 * I * H);
        memcpy(wqkv, wq, sizeof(float) * (size_t)qd * H);
        memcpy(wqkv + (size_t)qd * H, wk, sizeof(float) * (size_t)kvd * H);
        memcpy(wqkv + (size_t)(qd + kvd) * H, wv, sizeof(float) * (size_t)kvd * H);
        for (int i = 0; i < I; ++i) {
            memcpy(wgu + (size_t)(2 * i) * H, wg + (size_t)i * H, sizeof(float) * H);
            memcpy(wgu + (size_t)(2 * i + 1) * H, wu + (size_t)i * H, sizeof(float) * H);
        }
        PkLayer &p = layers[l];
        p.wqkv = quant(wqkv, (size_t)qkvd * H); p.wo = quant(wo, (size_t)H * qd);
        p.wgu = quant(wgu, (size_t)2 * I * H); p.wdown = quant(wd, (size_t)H * I);
        p.in_norm = n1; p.post_norm = n2; p.q_norm = qk_norm ? qn : nullptr; p.k_norm = qk_norm ? kn : nullptr;
        p.k_cache = k_slab + cache_stride * l; p.v_cache = v_slab + cache_stride * l;
        if (bf16) {  // the oracle sees the rounded values, un-fused again
            memcpy(wq, wqkv, sizeof(float) * (size_t)qd * H);
            memcpy(wk, wqkv + (size_t)qd * H, sizeof(float) * (size_t)kvd * H);
            memcpy(wv, wqkv + (size_t)(qd + kvd) * H, sizeof(float) * (size_t)kvd * H);
            for (int i = 0; i < I; ++i) {
                memcpy(wg + (size_t)i * H, wgu + (size_t)(2 * i) * H, sizeof(float) * H);
                memcpy(wu + (size_t)i * H, wgu + (size_t)(2 * i + 1) * H, sizeof(float) * H);
            }
        }
        lo_llama_layer &o = olayers[l];
        o.wq = wq; o.wk = wk; o.wv = wv; o.wo = wo; o.w_gate = wg; o.w_up = wu; o.w_down = wd;
        o.input_norm = n1; o.post_norm = n2; o.q_norm = qk_norm ? qn : nullptr; o.k_norm = qk_norm ? kn : nullptr;
    }
    float *cos_t = alloc<float>((size_t)max_seq * D), *sin_t = alloc<float>((size_t)max_seq * D);
    lo_rope_table(cos_t, sin_t, D, max_seq, 10000.0f);

    // ---- oracle: feed start_pos random tokens (fills its cache), then greedy steps
    lo_llama_config oc = {V, H, I, L, Hq, Hkv, 1e-5f, max_seq, 10000.0f, D, qk_norm, 0};
    lo_llama *om = lo_llama_new(&oc);
    lo_llama_set_globals(om, embed, final_norm, lm_head_f);
    for (int l = 0; l < L; ++l) lo_llama_set_layer(om, l, &olayers[l]);
    std::vector<float> ologits((size_t)V * (start_pos > 1 ? start_pos : 1));
    int first_tok = 1 % V;
    if (start_pos > 0) {
        std::vector<float> ids(start_pos);
        for (int i = 0; i < start_pos; ++i) ids[i] = (float)((i * 7 + 3) % V);
        if (lo_llama_forward(om, ids.data(), start_pos, ologits.data()) != LO_OK) return 3;
        // hand the oracle's cache to the kernel: the prefix is an input of the decode step
        for (int l = 0; l < L; ++l) {
            memcpy(k_slab + cache_stride * l, lo_llama_cache_k(om, l), sizeof(float) * cache_stride);
            memcpy(v_slab + cache_stride * l, lo_llama_cache_v(om, l), sizeof(float) * cache_stride);
        }
    }

    // ---- kernel arguments
    PkArgs a = {};
    PkLayer *dl = alloc<PkLayer>(L);
    memcpy(dl, layers.data(), sizeof(PkLayer) * L);
    int nsplit = max_seq / 64; nsplit = nsplit < 1 ? 1 : (nsplit > 64 ? 64 : nsplit);
    a.layers = dl; a.n_layers = L; a.H = H; a.I = I; a.V = V; a.qd = qd; a.kvd = kvd; a.hq = Hq; a.hkv = Hkv; a.D = D;
    a.max_seq = max_seq; a.nsplit = nsplit; a.eps = 1e-5f; a.scale = 1.0f / sqrtf((float)D); a.w_bf16 = bf16;
    a.embed = embed; a.lm_head = lm_head; a.final_norm = final_norm; a.cos_t = cos_t; a.sin_t = sin_t;
    a.x = alloc<float>(H); a.h = alloc<float>(H); a.qkv = alloc<float>(qkvd); a.attn = alloc<float>(qd);
    a.act = alloc<float>(I); a.logits = alloc<float>(V);
    a.part = alloc<float>((size_t)Hq * nsplit * (D + 2)); a.head_counters = alloc<int>(Hkv);
    a.tok = alloc<int>(4); a.pos = alloc<int>(4); a.bar = alloc<unsigned>(4); a.err = alloc<int>(4);
    a.amax_val = alloc<float>(nblocks); a.amax_idx = alloc<int>(nblocks);
    a.n_steps = steps; a.ids_out = alloc<int>(steps); a.logits_out = alloc<float>((size_t)steps * V);
    a.timeout_ticks = 60ull * 100000000ull;
    a.tok[0] = first_tok; a.pos[0] = start_pos;
    (void)esz;

    // ---- launch: nblocks workgroups of PK_THREADS threads, all concurrent
    const int kvec = bf16 ? 8 : 4, sweep = 64 * kvec;
    int kmax = H > I ? H : I; kmax = qd > kmax ? qd : kmax;
    const size_t xs = (size_t)((kmax + sweep - 1) / sweep * sweep);
    const size_t att = (size_t)2 * nrep * D + 3 * D + (size_t)PK_WAVES * nrep * D + 2 * PK_WAVES * nrep + 4;
    const size_t lds_floats = (xs > att ? xs : att) + PK_LDS_HEADER;  // exact size: ASan sees any overrun
    gridDim.x = nblocks; blockDim.x = PK_THREADS;
    std::vector<std::unique_ptr<EmuBlock>> blocks;
    std::vector<ThreadArg> targs((size_t)nblocks * PK_THREADS);
    std::vector<pthread_t> th(targs.size());
    pthread_attr_t attr;
    pthread_attr_init(&attr);
    pthread_attr_setstacksize(&attr, 512 * 1024);
    for (int b = 0; b < nblocks; ++b) {
        blocks.emplace_back(new EmuBlock());
        EmuBlock *eb = blocks.back().get();
        pthread_barrier_init(&eb->bar, nullptr, PK_THREADS);
        eb->wave_bar.resize(PK_WAVES);
        for (auto &wb : eb->wave_bar) pthread_barrier_init(&wb, nullptr, 64);
        eb->slots.assign(PK_WAVES * 64, 0);
        eb->lds.assign(lds_floats, 0.f);
    }
    for (int b = 0; b < nblocks; ++b)
        for (int t = 0; t < PK_THREADS; ++t) {
            ThreadArg &ta = targs[(size_t)b * PK_THREADS + t];
            ta.args = a; ta.blk = blocks[b].get(); ta.bx = b; ta.tx = t; ta.D = D; ta.nrep = nrep; ta.bf16 = bf16;
            if (pthread_create(&th[(size_t)b * PK_THREADS + t], &attr, thread_main, &ta)) { perror("pthread_create"); return 4; }
        }
    for (auto &t : th) pthread_join(t, nullptr);
    if (a.err[0]) { fprintf(stderr, "barrier time limit hit\n"); return 5; }

    // ---- compare with the oracle step by step (teacher-forced on the oracle's picks)
    int tok = first_tok;
    double worst = 0.0;
    int mismatches = 0;
    std::vector<float> ol(V);
    for (int s = 0; s < steps; ++s) {
        float idf = (float)tok;
        if (lo_llama_forward(om, &idf, 1, ol.data()) != LO_OK) return 6;
        const float *kl = a.logits_out + (size_t)s * V;
        double mx = 0, err = 0;
        for (int i = 0; i < V; ++i) { mx = fmax(mx, fabs(ol[i])); err = fmax(err, fabs((double)kl[i] - ol[i])); }
        worst = fmax(worst, err / mx);
        const int opick = lo_argmax_f32(ol.data(), V);
        if (a.ids_out[s] != opick) { ++mismatches; break; }  // sequences diverge after a different pick
        tok = opick;
    }
    printf("steps=%d nblocks=%d worst_rel_err=%.3e pick_mismatches=%d final_pos=%d\n", steps, nblocks, worst, mismatches, a.pos[0]);
    const double tol = bf16 ? 2e-2 : 1e-4;
    return (worst <= tol && mismatches == 0 && a.pos[0] == start_pos + steps) ? 0 : 1;
}
