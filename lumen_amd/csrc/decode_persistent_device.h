// Persistent decode kernel: all layers of one or more decode steps in a single
// cooperative launch, one 512-thread workgroup per compute unit.
//
// A decode step is a chain of matrix-vector products in which every product
// needs the complete output of the one before it, so the chain is a sequence
// of stages separated by grid-wide barriers.  What makes that worth doing in
// one kernel is that the WEIGHTS of the next stage do not depend on anything:
// before a wavefront goes into a barrier it has already issued the loads for
// its first rows of the next stage (16 x 16 bytes per lane, held in
// registers), so HBM keeps streaming while the barrier, the activation
// staging and the reduction tails are in flight.  Launch gaps between kernels
// disappear altogether.
//
// Stages per layer (src/models/llama.rs:104-116, self_attention.rs:125-306):
//   1  RMSNorm(x) -> q|k|v GEMV
//   2  RoPE(q,k), KV append, GQA online-softmax attention over the cache
//   3  o_proj GEMV + residual
//   4  RMSNorm(h) -> gate|up GEMV -> silu(gate)*up
//   5  down GEMV + residual
// then RMSNorm -> lm_head GEMV with a fused arg-max that becomes the next
// token id, so greedy generation of n tokens is one launch.
//
// Memory model: activations are written with ordinary stores.  At a barrier
// every wavefront first waits for its own stores, then one thread per
// workgroup runs release fence -> atomic arrive -> spin -> acquire fence,
// which writes back / invalidates the per-XCD L2 and the CU's L1, so ordinary
// loads after the barrier see every other workgroup's stores.  The spin is
// bounded by a wall-clock limit that raises an error flag all workgroups
// observe: every wavefront always reaches the end of the kernel.
#pragma once
#include "attn_device.h"
#include "decode_persistent.h"

#ifndef PK_DYNAMIC_LDS
#define PK_DYNAMIC_LDS(name) extern __shared__ __align__(16) float name[]
#endif

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

#define PK_WAVES 8
#define PK_THREADS (PK_WAVES * 64)
#define PK_CH 8       // 16-byte loads per lane per chunk
#define PK_PRE 2      // chunks prefetched across a barrier
#define PK_LDS_HEADER 32  // floats of workgroup-shared scalars in front of the dynamic LDS area

struct Pre {
    v4u r[PK_PRE][PK_CH];
};

struct GridBar {
    unsigned *ctr;
    int *err;
    unsigned target, nblocks;
    unsigned long long timeout;
};

// Completes this wavefront's stores (s_waitcnt vmcnt(0)) and keeps the compiler from sinking
// them below this point; loads issued afterwards stay in flight across the barrier.
__device__ __forceinline__ void wait_own_stores() { __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup"); }

// Precondition: every wavefront has waited for its own stores (wait_own_stores)
// BEFORE issuing any prefetch loads it wants to keep in flight.
__device__ __forceinline__ void grid_sync(GridBar &b) {
    b.target += b.nblocks;
    __builtin_amdgcn_s_barrier();
    if (threadIdx.x == 0) {
        __threadfence();
        __hip_atomic_fetch_add(b.ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long t0 = wall_clock64();
        unsigned it = 0;
        while (__hip_atomic_load(b.ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < b.target) {
            __builtin_amdgcn_s_sleep(1);
            if ((++it & 63u) == 0) {
                if (__hip_atomic_load(b.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
                if (wall_clock64() - t0 > b.timeout) {
                    __hip_atomic_store(b.err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
            }
        }
        __threadfence();
    }
    __builtin_amdgcn_s_barrier();
}

__device__ __forceinline__ float wave_sum_pk(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <bool BF16>
__device__ __forceinline__ float dot16_pk(const v4u raw, const float *xs) {
    if (BF16) {
        const v4f xa = *(const v4f *)xs;
        const v4f xb = *(const v4f *)(xs + 4);
        float s = __uint_as_float(raw.x << 16) * xa.x;
        s = fmaf(__uint_as_float(raw.x & 0xffff0000u), xa.y, s);
        s = fmaf(__uint_as_float(raw.y << 16), xa.z, s);
        s = fmaf(__uint_as_float(raw.y & 0xffff0000u), xa.w, s);
        s = fmaf(__uint_as_float(raw.z << 16), xb.x, s);
        s = fmaf(__uint_as_float(raw.z & 0xffff0000u), xb.y, s);
        s = fmaf(__uint_as_float(raw.w << 16), xb.z, s);
        s = fmaf(__uint_as_float(raw.w & 0xffff0000u), xb.w, s);
        return s;
    } else {
        const v4f xa = *(const v4f *)xs;
        float s = __uint_as_float(raw.x) * xa.x;
        s = fmaf(__uint_as_float(raw.y), xa.y, s);
        s = fmaf(__uint_as_float(raw.z), xa.z, s);
        s = fmaf(__uint_as_float(raw.w), xa.w, s);
        return s;
    }
}

// One GEMV stage: W [N, K]; a unit is `rpu` consecutive rows (2 for the gate|up
// pair, else 1) handled by one wavefront; units are dealt so that every
// compute unit gets an equal share: global wavefront id gw = wave*nblocks + block.
// A chunk is PK_CH sweeps (16-byte loads per lane) of one row.
enum { PEPI_STORE = 0, PEPI_RESIDUAL = 1, PEPI_SWIGLU = 2, PEPI_ARGMAX = 3 };

struct GemvDesc {
    const char *W;
    int N, K;
    int rpu, epi;
    const float *x_src;     // [K]
    const float *norm_w;    // RMSNorm gain [K] or null
    const float *residual;  // [N] or null
    float *y;               // [N] ([N/2] for the SwiGLU stage)
};

template <bool BF16>
struct GemvGeom {
    static constexpr int VEC = BF16 ? 8 : 4;
    static constexpr int SWEEP = 64 * VEC;  // elements one wavefront covers per load
    static constexpr int ESZ = BF16 ? 2 : 4;
};

// loads chunk `c` of this wavefront (wave-local numbering over its units, rows and row pieces)
template <bool BF16>
__device__ __forceinline__ void load_chunk(const GemvDesc &d, int c, int cprow, int gw, int nw, v4u (&r)[PK_CH]) {
    typedef GemvGeom<BF16> G;
    const int lane = threadIdx.x & 63;
    const int cpu = cprow * d.rpu;
    const int within = c % cpu;
    const int row = (gw + (c / cpu) * nw) * d.rpu + within / cprow;
    const int s0 = (within % cprow) * PK_CH;
    const char *base = d.W + ((size_t)row * d.K + (size_t)lane * G::VEC) * G::ESZ;
#pragma unroll
    for (int i = 0; i < PK_CH; ++i) {
        const int k = (s0 + i) * G::SWEEP + lane * G::VEC;
        r[i] = (v4u){0u, 0u, 0u, 0u};
        if (row < d.N && k < d.K)
            r[i] = __builtin_nontemporal_load((const v4u *)(base + (size_t)(s0 + i) * G::SWEEP * G::ESZ));
    }
}

template <bool BF16>
__device__ __forceinline__ void prefetch(const GemvDesc &d, Pre &pre, int gw, int nw) {
    typedef GemvGeom<BF16> G;
    const int sw = (d.K + G::SWEEP - 1) / G::SWEEP;
    const int cprow = (sw + PK_CH - 1) / PK_CH;
#pragma unroll
    for (int p = 0; p < PK_PRE; ++p) load_chunk<BF16>(d, p, cprow, gw, nw, pre.r[p]);
}

// Stages x into LDS (optionally RMS-normalised, src/layers/norm/rms_norm.rs:45-58).
__device__ __forceinline__ void stage_x_pk(float *xs, float *red, const float *x, const float *g, float eps, int K,
                                           int kpad) {
    const int tid = threadIdx.x;
    float inv = 1.0f;
    if (g) {
        float ss = 0.f;
        for (int k = tid * 4; k < K; k += PK_THREADS * 4) {
            const v4f v = *(const v4f *)(x + k);
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
        ss = wave_sum_pk(ss);
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < PK_WAVES; ++w) tot += red[w];
        inv = 1.0f / sqrtf(tot / (float)K + eps);
    }
    for (int k = tid * 4; k < kpad; k += PK_THREADS * 4) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        if (k < K) {
            v = *(const v4f *)(x + k);
            if (g) {
                const v4f gg = *(const v4f *)(g + k);
                v.x = v.x * inv * gg.x;
                v.y = v.y * inv * gg.y;
                v.z = v.z * inv * gg.z;
                v.w = v.w * inv * gg.w;
            }
        }
        *(v4f *)(xs + k) = v;
    }
    __syncthreads();
}

// Runs the stage; `pre` holds this wavefront's first PK_PRE chunks (loaded
// before the previous barrier).  best/best_idx: running arg-max (PEPI_ARGMAX).
template <bool BF16>
__device__ __forceinline__ void gemv_stage(const GemvDesc &d, Pre &pre, float *xs, float *red, float eps, int gw,
                                           int nw, float &best, int &best_idx) {
    typedef GemvGeom<BF16> G;
    const int lane = threadIdx.x & 63;
    const int kpad = (d.K + G::SWEEP - 1) / G::SWEEP * G::SWEEP;
    stage_x_pk(xs, red, d.x_src, d.norm_w, eps, d.K, kpad);

    const int sw = kpad / G::SWEEP;
    const int cprow = (sw + PK_CH - 1) / PK_CH;
    const int cpu = cprow * d.rpu;
    const int nunits = d.N / d.rpu;
    const int my_units = (nunits > gw) ? (nunits - gw + nw - 1) / nw : 0;
    const int my_chunks = my_units * cpu;
    float acc = 0.f, first = 0.f;

    for (int c0 = 0; c0 < my_chunks; c0 += PK_PRE) {
        if (c0 > 0) {
#pragma unroll
            for (int p = 0; p < PK_PRE; ++p) load_chunk<BF16>(d, c0 + p, cprow, gw, nw, pre.r[p]);
        }
#pragma unroll
        for (int p = 0; p < PK_PRE; ++p) {
            const int c = c0 + p;
            if (c < my_chunks) {
                const int within = c % cpu;
                const int s0 = (within % cprow) * PK_CH;
#pragma unroll
                for (int i = 0; i < PK_CH; ++i) {
                    const int k = (s0 + i) * G::SWEEP + lane * G::VEC;
                    if (k < kpad) acc += dot16_pk<BF16>(pre.r[p][i], xs + k);
                }
                if ((within % cprow) == cprow - 1) {  // row complete
                    const int u = gw + (c / cpu) * nw;
                    const int j = within / cprow;
                    const int row = u * d.rpu + j;
                    float v = wave_sum_pk(acc);
                    acc = 0.f;
                    if (d.epi == PEPI_SWIGLU) {
                        // rows (2u, 2u+1) = (gate_u, up_u): silu(gate) * up, src/models/llama.rs:60-63
                        if (j == 0) {
                            first = v;
                        } else if (lane == 0) {
                            const float sig = 1.0f / (1.0f + expf(-first));
                            d.y[u] = (first * sig) * v;
                        }
                    } else {
                        if (d.epi == PEPI_RESIDUAL) v = d.residual[row] + v;  // src/models/llama.rs:110,115
                        if (lane == 0) d.y[row] = v;
                        if (d.epi == PEPI_ARGMAX && (v > best || (v == best && row < best_idx))) {
                            best = v;
                            best_idx = row;
                        }
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------- attention
template <int D, int NREP>
__device__ __forceinline__ void attn_stage(const PkArgs &a, const PkLayer &L, int pos, float *lds) {
    typedef AttnGeom<D, PK_WAVES> G;
    float *q_raw = lds;                         // [NREP*D]
    float *q_rot = q_raw + NREP * D;            // [NREP*D]
    float *k_raw = q_rot + NREP * D;            // [D]
    float *k_new = k_raw + D;                   // [D]
    float *v_new = k_new + D;                   // [D]
    float *sacc = v_new + D;                    // [PK_WAVES*NREP*D]
    float *sm = sacc + PK_WAVES * NREP * D;     // [PK_WAVES*NREP]
    float *sl = sm + PK_WAVES * NREP;           // [PK_WAVES*NREP]
    int *s_last = (int *)(sl + PK_WAVES * NREP);

    int nact, chunk;
    decode_slices<D, PK_WAVES>(pos, a.nsplit, nact, chunk);
    const int nunits = a.hkv * nact;
    const float *cs = a.cos_t + (size_t)pos * D, *sn = a.sin_t + (size_t)pos * D;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slot = lane / G::LPR, c = lane % G::LPR;
    const int t = threadIdx.x;

    for (int unit = blockIdx.x; unit < nunits; unit += gridDim.x) {
        const int hk = unit / nact, split = unit % nact;
        const bool has_new = (split == nact - 1);
        const size_t head_base = (size_t)hk * a.max_seq * D;
        __syncthreads();  // LDS reuse across units
        const float *q_src = a.qkv + (size_t)hk * NREP * D;
        for (int i = t; i < NREP * D; i += PK_THREADS) q_raw[i] = q_src[i];
        if (has_new) {
            const float *k_src = a.qkv + a.qd + (size_t)hk * D;
            const float *v_src = a.qkv + a.qd + a.kvd + (size_t)hk * D;
            for (int i = t; i < D; i += PK_THREADS) {
                k_raw[i] = k_src[i];
                v_new[i] = v_src[i];
            }
        }
        __syncthreads();
        norm_rope_heads<D>(q_raw, q_rot, NREP, cs, sn, L.q_norm, a.eps, PK_THREADS);
        if (has_new) norm_rope_heads<D>(k_raw, k_new, 1, cs, sn, L.k_norm, a.eps, PK_THREADS);
        __syncthreads();
        if (has_new) {
            for (int i = t; i < D; i += PK_THREADS) {
                L.k_cache[head_base + (size_t)pos * D + i] = k_new[i];
                L.v_cache[head_base + (size_t)pos * D + i] = v_new[i];
            }
        }
        v4f q[NREP];
        load_q_scaled<D, NREP>(q, q_rot, c, a.scale);
        const int p0 = min(pos, split * chunk), p1 = min(pos, p0 + chunk);
        AttnState<NREP> st;
        state_init<NREP>(st);
        attn_rows<D, NREP, PK_WAVES>(st, q, L.k_cache + head_base, L.v_cache + head_base, p0, p1);
        if (has_new && wave == 0) {
            const v4f kv = *(const v4f *)(k_new + c * 4);
            const v4f vv = *(const v4f *)(v_new + c * 4);
            attn_step<D, NREP>(st, q, kv, vv, slot == 0);
        }
        wave_merge_publish<D, NREP>(st, sm, sl, sacc);
        __syncthreads();
        for (int e = t; e < NREP * D; e += PK_THREADS) {
            const int r = e / D, dd = e % D;
            float mm, ls, cx;
            wave_fold<D, NREP, PK_WAVES>(sm, sl, sacc, r, dd, mm, ls, cx);
            const int hq = hk * NREP + r;
            if (nact == 1) {
                a.attn[(size_t)hq * D + dd] = cx * (1.0f / (ls + 1e-9f));  // self_attention.rs:287-290
            } else {
                float *pp = a.part + ((size_t)hq * a.nsplit + split) * (D + 2);
                part_store(pp + dd, cx);
                if (dd == 0) {
                    part_store(pp + D, mm);
                    part_store(pp + D + 1, ls);
                }
            }
        }
        if (nact > 1) {
            // last workgroup of this KV head to arrive folds the slices in index order
            __syncthreads();
            if (t == 0) {
                const int old = __hip_atomic_fetch_add(&a.head_counters[hk], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                *s_last = (old == nact - 1);
                if (old == nact - 1) __hip_atomic_store(&a.head_counters[hk], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();
            if (*s_last) {
                for (int e = t; e < NREP * D; e += PK_THREADS) {
                    const int r = e / D, dd = e % D;
                    const int hq = hk * NREP + r;
                    a.attn[(size_t)hq * D + dd] = fold_slices<D>(a.part + ((size_t)hq * a.nsplit) * (D + 2), nact, dd);
                }
            }
        }
    }
}

// -------------------------------------------------------------------- kernel
// Stage numbering inside a step: 5*l + {0 q|k|v, 1 attention, 2 o_proj, 3 gate|up, 4 down}; 5*n_layers = lm_head.
__device__ __forceinline__ GemvDesc make_desc(const PkArgs &a, int sidx, const float *x_embed, float *logits) {
    GemvDesc d;
    const int l = sidx / 5, k = sidx % 5;
    d.rpu = 1;
    d.norm_w = nullptr;
    d.residual = nullptr;
    if (l >= a.n_layers) {  // final norm + lm_head, llama.rs:202-205
        d.W = (const char *)a.lm_head; d.N = a.V; d.K = a.H; d.epi = PEPI_ARGMAX;
        d.x_src = a.x; d.norm_w = a.final_norm; d.y = logits;
        return d;
    }
    const PkLayer &L = a.layers[l];
    const float *x_in = (l == 0) ? x_embed : a.x;
    if (k == 0) {  // input_layernorm + q|k|v, llama.rs:107, self_attention.rs:106-108
        d.W = (const char *)L.wqkv; d.N = a.qd + 2 * a.kvd; d.K = a.H; d.epi = PEPI_STORE;
        d.x_src = x_in; d.norm_w = L.in_norm; d.y = a.qkv;
    } else if (k == 2) {  // o_proj + residual, self_attention.rs:303, llama.rs:110
        d.W = (const char *)L.wo; d.N = a.H; d.K = a.qd; d.epi = PEPI_RESIDUAL;
        d.x_src = a.attn; d.residual = x_in; d.y = a.h;
    } else if (k == 3) {  // post_attention_layernorm + gate|up + SwiGLU, llama.rs:113, :60-63
        d.W = (const char *)L.wgu; d.N = 2 * a.I; d.K = a.H; d.epi = PEPI_SWIGLU; d.rpu = 2;
        d.x_src = a.h; d.norm_w = L.post_norm; d.y = a.act;
    } else {  // down_proj + residual, llama.rs:64, :115
        d.W = (const char *)L.wdown; d.N = a.H; d.K = a.I; d.epi = PEPI_RESIDUAL;
        d.x_src = a.act; d.residual = a.h; d.y = a.x;
    }
    return d;
}

template <int D, int NREP, bool BF16>
__global__ __launch_bounds__(PK_THREADS, 1) void decode_persistent_kernel(PkArgs a) {
    PK_DYNAMIC_LDS(lds_all);
    float *red = lds_all;                  // [PK_WAVES]
    float *am_v = lds_all + PK_WAVES;      // [PK_WAVES]
    int *am_i = (int *)(lds_all + 2 * PK_WAVES);
    int *s_tok = (int *)(lds_all + 3 * PK_WAVES);
    float *lds = lds_all + PK_LDS_HEADER;  // activation vector / attention scratch

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nblocks = gridDim.x;
    const int gw = wave * nblocks + blockIdx.x;
    const int nw = PK_WAVES * nblocks;
    GridBar bar = {a.bar, a.err, 0u, (unsigned)nblocks, a.timeout_ticks};

    int tok = *a.tok;
    int pos = *a.pos;
    Pre pre;
    const int n_stages = 5 * a.n_layers + 1;

    // first stage's weights (no barrier precedes it)
    prefetch<BF16>(make_desc(a, 0, a.embed, a.logits), pre, gw, nw);

    for (int step = 0; step < a.n_steps; ++step) {
        const float *x_embed = a.embed + (size_t)tok * a.H;  // Embedding::forward, embedding.rs:47-57
        float *logits = a.logits_out ? a.logits_out + (size_t)step * a.V : a.logits;
        float best = -INFINITY;
        int best_idx = 0x7fffffff;
        for (int sidx = 0; sidx < n_stages; ++sidx) {
            const bool is_attn = (sidx % 5 == 1) && sidx < 5 * a.n_layers;
            if (is_attn) {
                attn_stage<D, NREP>(a, a.layers[sidx / 5], pos, lds);
            } else {
                const GemvDesc d = make_desc(a, sidx, x_embed, logits);
                // the thread that runs the barrier keeps no loads in flight across it: it fetches here
                if (wave == 0 && !(step == 0 && sidx == 0)) prefetch<BF16>(d, pre, gw, nw);
                gemv_stage<BF16>(d, pre, lds, red, a.eps, gw, nw, best, best_idx);
            }
            if (sidx == n_stages - 1) {  // publish this workgroup's arg-max candidate
                if (lane == 0) {
                    am_v[wave] = best;
                    am_i[wave] = best_idx;
                }
                __syncthreads();
                if (threadIdx.x == 0) {
                    float bv = am_v[0];
                    int bi = am_i[0];
                    for (int w = 1; w < PK_WAVES; ++w)
                        if (am_v[w] > bv || (am_v[w] == bv && am_i[w] < bi)) {
                            bv = am_v[w];
                            bi = am_i[w];
                        }
                    a.amax_val[blockIdx.x] = bv;
                    a.amax_idx[blockIdx.x] = bi;
                }
            }
            wait_own_stores();
            // weights of the next GEMV stage start streaming before the barrier (not across the
            // attention stage, which needs the registers itself)
            int nxt = sidx + 1;
            const bool last_of_all = (nxt == n_stages) && (step + 1 == a.n_steps);
            if (nxt == n_stages) nxt = 0;
            const bool nxt_attn = (nxt % 5 == 1) && nxt < 5 * a.n_layers;
            if (wave != 0 && !last_of_all && !nxt_attn) prefetch<BF16>(make_desc(a, nxt, a.embed, a.logits), pre, gw, nw);
            grid_sync(bar);
        }
        // every workgroup folds the per-workgroup maxima itself: lowest index wins ties
        {
            float bv = -INFINITY;
            int bi = 0x7fffffff;
            for (int i = threadIdx.x; i < nblocks; i += PK_THREADS) {
                const float v = a.amax_val[i];
                const int ix = a.amax_idx[i];
                if (v > bv || (v == bv && ix < bi)) {
                    bv = v;
                    bi = ix;
                }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const float ov = __shfl_xor(bv, off, 64);
                const int oi = __shfl_xor(bi, off, 64);
                if (ov > bv || (ov == bv && oi < bi)) {
                    bv = ov;
                    bi = oi;
                }
            }
            __syncthreads();  // am_v / am_i are reused
            if (lane == 0) {
                am_v[wave] = bv;
                am_i[wave] = bi;
            }
            __syncthreads();
            if (threadIdx.x == 0) {
                for (int w = 1; w < PK_WAVES; ++w)
                    if (am_v[w] > bv || (am_v[w] == bv && am_i[w] < bi)) {
                        bv = am_v[w];
                        bi = am_i[w];
                    }
                if (bi == 0x7fffffff) bi = 0;
                *s_tok = bi;
            }
            __syncthreads();
            tok = *s_tok;
        }
        pos += 1;
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            if (a.ids_out) a.ids_out[step] = tok;
            *a.tok = tok;
            *a.pos = pos;
        }
    }
}

