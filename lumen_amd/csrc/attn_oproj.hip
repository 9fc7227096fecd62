// Decode attention and the o_proj product chained inside ONE launch, for short caches.
//
// Reference path: SelfAttention::forward, S == 1 (src/layers/attention/self_attention.rs:183-303): per query head an
// online softmax over the cached rows (:199-293), then out = w_o(ctx) (:303) and the residual add of
// LlamaDecoderLayer::forward_infer (src/models/llama.rs:110).
//
// As two launches the pair is latency, not bytes: a few hundred cached rows keep 32 of 256 compute units busy for
// ~4.5 us while the memory system idles, then a 17 MB product waits ~2.5 us for its first weights.  Here they are one
// grid whose workgroups play two roles:
//
//   [0, hq)       attention, one query head each (attn_short_device.h): exactly the arithmetic of the stand-alone
//                 kernel; the D output values of a head leave as tagged words;
//   next N / 8    o_proj, one row per wavefront: a workgroup requests ALL its weights into registers at once, then
//                 takes the hq * D tagged words of the attention output (each thread its own few), stages them in
//                 LDS, multiplies, adds the residual and stores.
//
// So the weights stream while the attention runs, and the product is ready a few hundred nanoseconds after the
// last attention value has become visible.  A value in flight between the roles is one 8-byte word {bits, tag}
// written and read atomically: a reader that sees the tag has the value, whatever the order of other accesses.
// The tag changes with every decode step and layer (*step_dev * tag_mul + tag_add): a word left by an earlier
// launch never matches.  Workgroups are dispatched in index order, so the attention workgroups are resident (or
// finished) before an o_proj workgroup starts to wait, and every wait ends.  Waits are bounded all the same
// (spin_limit polls, then *err_dev = 1 and the workgroup goes on with whatever it has), so that every wavefront exits.
//
// Timing of the o_proj workgroups (set by the caller): the weight requests go out pre_sleep x 0.1 us after the
// workgroup's start, so that what the roles before ask for enters the memory system first; the first poll follows
// poll_delay x 0.1 us later, and poll_gap x 256 clocks lie between polls, because every poll of the 131072 threads is a
// trip to memory that the weights compete with.  The two delays are taken from the 100 MHz wall clock, not from the
// shader clock: what they are timed against -- the memory system -- does not follow the shader clock either, and
// with cycle-counted pauses the optimum moved from box to box.
//
// q arrives rotated and cache row `pos` is already written (both by the q|k|v product's epilogue) -- or, QKV form,
// that product is a third role in FRONT of the two:
//
//   [0, nq)       RMSNorm of the layer input + q|k|v product + RoPE, one rotation pair of rows (j, j + D/2) per
//                 wavefront with all weights in registers (src/models/llama.rs:107, self_attention.rs:106-108,
//                 :220-227); the rotated q, the new key and the new value leave as tagged words, key and value also
//                 go to cache row `pos` (self_attention.rs:161-176) for the steps to come;
//
// and, q/k-norm models, leaves q / k / v un-rotated: norm, rotation and the cache write then happen in the attention
// workgroups.  Long caches are cut into slices (a power of two of rows each, `slice_rows`): `nslices` attention
// workgroups per query head take one slice each in parallel and leave their online-softmax states as tagged words;
// hq further workgroups behind them fold the slices of a head (in slice order: the same bits every time) and hand
// the result on.  With one slice in use the attention workgroup writes the final output itself.
//
// the attention workgroups request their first trip of cached rows, THEN wait for their head's q and the group's
// new row, and take that row from LDS instead of the cache.  The layer input is read by the first and (as the
// residual) the last role; it was written by an earlier launch.  In this form the o_proj workgroups hold their
// weight requests back (pre_sleep) until q and the new row have changed hands: every trip to memory of a hand-over
// queues behind whatever was requested before it, and 17 MB of weights in the queue cost each trip ~2 us.
#include "internal.h"
#include "attn_device.h"
#include "attn_short_device.h"
#include "wave_reduce.h"
#include "stage_times.h"

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

#define AO_WAVES 8
#define AO_THREADS (AO_WAVES * 64)

// 16 bytes of weights times the matching input values (f32: 4 values, bf16: 8, widened by a shift like loader.rs:58)
template <bool BF16>
__device__ __forceinline__ float ao_dot16(const v4u raw, const float *xs) {
    const v4f xa = *(const v4f *)xs;
    if (BF16) {
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
    }
    float s = __uint_as_float(raw.x) * xa.x;
    s = fmaf(__uint_as_float(raw.y), xa.y, s);
    s = fmaf(__uint_as_float(raw.z), xa.z, s);
    s = fmaf(__uint_as_float(raw.w), xa.w, s);
    return s;
}

// D: head_dim; NLQ / NLO: 16-byte weight loads per lane and row of the q|k|v / the o_proj product (row length = loads
// * 64 * elements per load: hidden / hq * D); QKV: 0 no q|k|v role (q rotated, cache row written by an earlier
// launch), 1 with it, 2 with it for q/k-norm models: the projections leave un-rotated and every attention workgroup
// normalises and rotates its own query head and the group's new key, the group's first head stores the new row.
template <int D, int NLQ, int NLO, bool BF16, int QKV>
__global__ __launch_bounds__(AO_THREADS) void attn_oproj_kernel(const void *Wo_hot, float *k_cache_hot, float *v_cache_hot,
                                                                const float *q_hot, const int *pos_dev_hot,
                                                                const unsigned *step_dev_hot, int max_seq_hot, int hq_hot,
                                                                int hkv_slices_hot, int N_hot, const void *Wqkv_hot,
                                                                const float *x_hot, const float *in_norm_hot,
                                                                AttnOprojArgs a_mem) {
    constexpr int VEC = BF16 ? 8 : 4;
    constexpr int ESZ = BF16 ? 2 : 4;
    constexpr int PW = 1;  // rotation pairs per wavefront of the q|k|v role, rows per wavefront of the o_proj role (two of
                           // each -- half the workgroups in those roles -- measured slower: 0.895 against 0.845 ms per token)
    constexpr int K = NLO * 64 * VEC;  // o_proj row length = hq * D
    constexpr int KQ = NLQ * 64 * VEC;  // q|k|v row length = hidden
    constexpr int EPT = K / AO_THREADS;
    static_assert(K % AO_THREADS == 0 && EPT >= 1, "K must be a multiple of the workgroup size");
    __shared__ __align__(16) float q_rot[D];
    __shared__ __align__(16) float k_new[D];
    __shared__ __align__(16) float v_new[D];
    __shared__ __align__(16) float sacc[AO_WAVES * (D > 64 ? D : 64)];
    __shared__ float sm[AO_WAVES], sl[AO_WAVES];
    __shared__ __align__(16) float xs[K > KQ ? K : KQ];
    STAGE_T(0);
    const unsigned t_start = (unsigned)wall_clock64();
    // the launch's own start, for workgroups that start late (a grid larger than the chip holds at once): the first
    // workgroup leaves its clock reading as a tagged word
    if (blockIdx.x == 0 && threadIdx.x == 0)
        tagged_store(a_mem.t0_tagged, __uint_as_float(t_start), *step_dev_hot * a_mem.tag_mul + a_mem.tag_add);
    const int hq = hq_hot, hkv = hkv_slices_hot & 0xffff, S = hkv_slices_hot >> 16, N = N_hot;  // S: attention slices
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_o = (N + AO_WAVES * PW - 1) / (AO_WAVES * PW);  // o_proj workgroups
    constexpr int HALF = D / 2;
    const int nunits = QKV ? (hq + 2 * hkv) * HALF : 0;  // rotation pairs; a multiple of 16: D / 2 is
    const int nq = nunits / (AO_WAVES * PW);             // q|k|v workgroups
    int blk = blockIdx.x;
    if (QKV && blk < nq) {
        // ---- RMSNorm + q|k|v + RoPE: one pair of rows (j, j + D/2) of one head per wavefront
        constexpr int XP = (KQ / 4 + AO_THREADS - 1) / AO_THREADS;  // 16-byte pieces of x a thread stages
        const int unit = (blk * AO_WAVES + wave) * PW;
        const int hh = unit / HALF, j = unit % HALF;  // PW pairs j, j + 1 of one head: adjacent rows
        const int head = hh;
        const float *x = x_hot;
        if (a_mem.row_sel) x += (long)(*a_mem.row_sel) * a_mem.row_stride;  // (first layer: a trip of its own)
        // x and the gains first: what is requested first arrives first, and the norm is what the multiplies wait for
        v4f xe[XP], ge[XP];
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int k = (tid + i * AO_THREADS) * 4;
            xe[i] = v4f{0.f, 0.f, 0.f, 0.f};
            ge[i] = xe[i];
            if (k < KQ) {
                xe[i] = *(const v4f *)(x + k);
                ge[i] = *(const v4f *)(in_norm_hot + k);
            }
        }
        v4u raw[PW][2][NLQ];
#pragma unroll
        for (int p = 0; p < PW; ++p)
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                const char *rp = (const char *)Wqkv_hot + ((size_t)(head * D + j + p + r * HALF) * KQ + (size_t)lane * VEC) * ESZ;
#pragma unroll
                for (int i = 0; i < NLQ; ++i) raw[p][r][i] = __builtin_nontemporal_load((const v4u *)(rp + (size_t)i * 64 * VEC * ESZ));
            }
        const int pos = *pos_dev_hot;
        const unsigned tag = *step_dev_hot * a_mem.tag_mul + a_mem.tag_add;
        float cs[PW], sn[PW];
#pragma unroll
        for (int p = 0; p < PW; ++p) {
            cs[p] = 1.f;
            sn[p] = 0.f;
            if (QKV == 1) {
                cs[p] = a_mem.attn.cos_t[(size_t)pos * D + j + p];
                sn[p] = a_mem.attn.sin_t[(size_t)pos * D + j + p];
            }
        }
        STAGE_T(1);
        // (x * inv_rms) * g, src/layers/norm/rms_norm.rs:45-58
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < XP; ++i) ss += xe[i].x * xe[i].x + xe[i].y * xe[i].y + xe[i].z * xe[i].z + xe[i].w * xe[i].w;
        ss = wave_sum(ss);
        if (lane == 0) sm[wave] = ss;
        __syncthreads();
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < AO_WAVES; ++w) tot += sm[w];
        const float inv = 1.0f / sqrtf(tot / (float)KQ + a_mem.norm_eps);
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int k = (tid + i * AO_THREADS) * 4;
            if (k < KQ) {
                v4f v = xe[i];
                v.x = v.x * inv * ge[i].x;
                v.y = v.y * inv * ge[i].y;
                v.z = v.z * inv * ge[i].z;
                v.w = v.w * inv * ge[i].w;
                *(v4f *)(xs + k) = v;
            }
        }
        __syncthreads();
        STAGE_T(2);
#pragma unroll
        for (int p = 0; p < PW; ++p) {
            float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
            for (int i = 0; i < NLQ; ++i) {
                acc0 += ao_dot16<BF16>(raw[p][0][i], xs + (i * 64 + lane) * VEC);
                acc1 += ao_dot16<BF16>(raw[p][1][i], xs + (i * 64 + lane) * VEC);
            }
            acc0 = wave_sum(acc0);
            acc1 = wave_sum(acc1);
            if (lane == 0) {
                // half-split rotation at the token's position (src/layers/attention/encoding.rs:196-203)
                float o1 = acc0, o2 = acc1;
                if (QKV == 1 && head < hq + hkv) {
#pragma clang fp contract(off)
                    o1 = acc0 * cs[p] - acc1 * sn[p];
                    o2 = acc0 * sn[p] + acc1 * cs[p];
                }
                unsigned long long *t = a_mem.qkv_tagged + (size_t)head * D + j + p;
                tagged_store(t, o1, tag);
                tagged_store(t + HALF, o2, tag);
                if (QKV == 1 && head >= hq) {  // key / value of the new token: cache row pos
                    float *cache = head < hq + hkv ? k_cache_hot : v_cache_hot;
                    const int hk = head < hq + hkv ? head - hq : head - hq - hkv;
                    float *dst = cache + ((size_t)hk * max_seq_hot + pos) * D;
                    dst[j + p] = o1;
                    dst[j + p + HALF] = o2;
                }
            }
        }
        STAGE_T_STORES_DONE(3);
        return;
    }
    blk -= nq;
    if (blk < hq * S) {
        // ---- attention of one query head (S > 1: of one trip of its cached rows).  Workgroup i of the grid runs on
        // XCD i % 8: consecutive (KV group, slice) units -- the n_rep heads that read the same rows -- share an XCD,
        // so that the rows are fetched into as few L2s as possible.
        AttnDecodeArgs a = a_mem.attn;
        a.k_cache = k_cache_hot;
        a.v_cache = v_cache_hot;
        a.pos_dev = pos_dev_hot;
        a.q = q_hot;
        a.max_seq = max_seq_hot;
        a.hq = hq;
        a.hkv = hkv;
        a.tag = *step_dev_hot * a_mem.tag_mul + a_mem.tag_add;
        a.qkv_tagged = a_mem.qkv_tagged;
        a.spin_limit = a_mem.spin_limit;
        a.poll_gap = a_mem.poll_gap;
        a.err_dev = a_mem.err_dev;
        a.tslices = S;
        a.slice_shift = S > 1 ? 31 - __builtin_clz(a_mem.slice_rows) : 30;
        a.part_tagged = a_mem.part_tagged;
        const int n_att = hq * S;
        const int xcd = (blk + nq) & 7;
        const int w = (n_att % 8 == 0) ? xcd * (n_att / 8) + (blk >> 3) : blk;
        const int nrep = hq / hkv;
        const int unit = w / nrep, r = w % nrep;  // unit = (KV head, slice)
        const int hk = unit / S, slice = unit % S;
        constexpr int SRC = QKV == 0 ? ATTN_SRC_CACHE : QKV == 1 ? ATTN_SRC_TAGGED : ATTN_SRC_TAGGED_RAW;
        // (one slice: rows without end, walked trip by trip)
        attn_decode_short<D, AO_WAVES, SRC, true>(a, r, nrep, hk, 0, -1, 0x7fffffff, q_rot, k_new, v_new, sm, sl, sacc, slice);
        return;
    }
    blk -= hq * S;
    if (S > 1) {
        if (blk < hq) {
            // ---- fold of the slices of one query head: out[d] = sum_s w_s ctx_s[d] / (sum_s w_s l_s + 1e-9),
            // w_s = exp2(m_s - max m) (scores are kept in log2 units), slices in index order.  Wavefronts 0 .. D/64-1
            // take the context elements, the next one the slices' (m, l); all words of a thread are requested
            // together, polled until every one carries the tag.
            const int nact = (*pos_dev_hot >> (31 - __builtin_clz(a_mem.slice_rows))) + 1;
            if (nact == 1) return;  // the only slice in use wrote the final output itself
            const unsigned tag = *step_dev_hot * a_mem.tag_mul + a_mem.tag_add;
            const unsigned long long *ph = a_mem.part_tagged + (size_t)blk * S * (D + 2);
            unsigned long long wv[ATTN_CHAIN_MAX_SLICES];
            unsigned long long wl[ATTN_CHAIN_MAX_SLICES];
            const bool ctx_thread = tid < D, ml_thread = tid >= D && tid < D + 64 && lane < nact;
            unsigned spins = 0;
            bool ok = true;
            do {
                ok = true;
                if (ctx_thread) {
#pragma unroll
                    for (int sI = 0; sI < ATTN_CHAIN_MAX_SLICES; ++sI)
                        if (sI < nact) {
                            wv[sI] = tagged_load(ph + (size_t)sI * (D + 2) + tid);
                            ok = ok && (unsigned)(wv[sI] >> 32) == tag;
                        }
                } else if (ml_thread) {
                    wv[0] = tagged_load(ph + (size_t)lane * (D + 2) + D);
                    wl[0] = tagged_load(ph + (size_t)lane * (D + 2) + D + 1);
                    ok = (unsigned)(wv[0] >> 32) == tag && (unsigned)(wl[0] >> 32) == tag;
                }
                if (!ok) {
                    if (++spins > a_mem.spin_limit) break;
                    handover_pause(a_mem.poll_gap);
                }
            } while (!ok);
            if (!ok) __hip_atomic_store(a_mem.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (tid >= D && tid < D + 64) {  // one wavefront: the weights of the slices and the normaliser
                const float mS = ml_thread ? __uint_as_float((unsigned)wv[0]) : -INFINITY;
                const float lS = ml_thread ? __uint_as_float((unsigned)wl[0]) : 0.f;
                const float M = wave_max(mS);
                const float wS = (ml_thread && mS > -INFINITY) ? fast_exp2(mS - M) : 0.f;
                if (lane < ATTN_CHAIN_MAX_SLICES) sacc[lane] = wS;
                // the normaliser, slices in index order (a fixed order: the same bits every time)
                sacc[ATTN_CHAIN_MAX_SLICES + lane] = lS * wS;
            }
            __syncthreads();
            if (ctx_thread) {
                float L = 0.f, o = 0.f;
#pragma unroll
                for (int sI = 0; sI < ATTN_CHAIN_MAX_SLICES; ++sI)
                    if (sI < nact) {
                        L += sacc[ATTN_CHAIN_MAX_SLICES + sI];
                        o = fmaf(__uint_as_float((unsigned)wv[sI]), sacc[sI], o);
                    }
                tagged_store(a_mem.x_tagged + (size_t)blk * D + tid, o * (1.0f / (L + 1e-9f)), tag);
            }
            return;
        }
        blk -= hq;
    }
    if (blk < n_o) {
        // ---- o_proj: one row per wavefront, all of its weights requested at once (rows past N: clamped, not stored)
        const int row = (blk * AO_WAVES + wave) * PW;
        // (see the head of the file; counted from the launch's start where that is known: with long caches these
        // workgroups wait for a free slot first, and a pause counted from their own start would begin too late)
        unsigned t_ref = t_start;
        {
            const unsigned long long w0 = tagged_load(a_mem.t0_tagged);
            if ((unsigned)(w0 >> 32) == *step_dev_hot * a_mem.tag_mul + a_mem.tag_add) t_ref = (unsigned)w0;
        }
        handover_pause_until32(t_ref, a_mem.pre_sleep);
        v4u raw[PW][NLO];
#pragma unroll
        for (int p = 0; p < PW; ++p) {
            const char *rp = (const char *)Wo_hot + ((size_t)min(row + p, N - 1) * K + (size_t)lane * VEC) * ESZ;
#pragma unroll
            for (int i = 0; i < NLO; ++i) raw[p][i] = __builtin_nontemporal_load((const v4u *)(rp + (size_t)i * 64 * VEC * ESZ));
        }
        const unsigned tag = *step_dev_hot * a_mem.tag_mul + a_mem.tag_add;
        const float *residual = a_mem.residual;
        if (a_mem.row_sel) residual += (long)(*a_mem.row_sel) * a_mem.row_stride;
        float res[PW];
#pragma unroll
        for (int p = 0; p < PW; ++p) res[p] = residual[min(row + p, N - 1)];
        STAGE_T(5);
        // the attention output: this thread's EPT words, polled until every one carries this launch's tag
        handover_pause_until(wall_clock64(), a_mem.poll_delay);
        {
            float v[EPT];
            if (!take_tagged<EPT>(a_mem.x_tagged + (size_t)tid * EPT, tag, a_mem.spin_limit, a_mem.poll_gap, v))
                __hip_atomic_store(a_mem.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int e = 0; e < EPT; ++e) xs[tid * EPT + e] = v[e];
        }
        __syncthreads();
        STAGE_T(6);
#pragma unroll
        for (int p = 0; p < PW; ++p) {
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < NLO; ++i) acc += ao_dot16<BF16>(raw[p][i], xs + (i * 64 + lane) * VEC);
            acc = wave_sum(acc);
            if (lane == 0 && row + p < N) {
                const float hv = res[p] + acc;  // src/ops/arithmetic.rs:48-51 via llama.rs:110
                a_mem.y[row + p] = hv;
            }
        }
        STAGE_T_STORES_DONE(7);
    }
}

static int ao_nl(int K, int w_bf16) {
    const int vec = w_bf16 ? 8 : 4;
    if (K <= 0 || K % (64 * vec) || K % AO_THREADS) return 0;
    return K / (64 * vec);
}

bool attn_oproj_supported(int hq, int hkv, int d, int N, int K, int w_bf16) {
    if (hkv <= 0 || hq % hkv || K != hq * d || N <= 0) return false;
    if (d != 64 && d != 128) return false;
    const int nl = ao_nl(K, w_bf16);
    return nl == 2 || nl == 4 || nl == 8 || nl == 16;
}

// the q|k|v role in front: two of its rows (hidden long) fit a wavefront's registers, and o_proj's rows are as long
// or (head_dim 128) twice as long; q/k-norm models with head_dim 128 only
bool qkv_attn_oproj_supported(int hq, int hkv, int d, int N, int K, int w_bf16, int qk_norm) {
    if (!attn_oproj_supported(hq, hkv, d, N, K, w_bf16)) return false;
    const int nlq = ao_nl(N, w_bf16), nlo = ao_nl(K, w_bf16);
    if (nlq != 2 && nlq != 4 && nlq != 8) return false;
    if (qk_norm && d != 128) return false;
    return nlo == nlq || (d == 128 && nlo == 2 * nlq);
}

int attn_oproj_workgroups(int N) { return (N + AO_WAVES - 1) / AO_WAVES; }

template <int D, bool BF16>
static int launch_ao(lumen_ctx *ctx, const AttnOprojArgs &a) {
    const int nlo = ao_nl(a.K, BF16), nlq = a.Wqkv ? ao_nl(a.N, BF16) : 0;
    const int form = !a.Wqkv ? 0 : a.attn.q_norm_w ? 2 : 1;
    const int S = a.nslices > 1 ? a.nslices : 1;
    const int nq = a.Wqkv ? (a.attn.hq + 2 * a.attn.hkv) * (D / 2) / AO_WAVES : 0;
    const int n_att = a.attn.hq * S + (S > 1 ? a.attn.hq : 0);  // attention workgroups, and those that fold the slices
    const int n_wg = nq + n_att + attn_oproj_workgroups(a.N);
    dim3 grid(n_wg), block(AO_THREADS);
    bool launched = false;
#define AO_LAUNCH(NLQ, NLO, QKV)                                                                                                 \
    do {                                                                                                                         \
        hipLaunchKernelGGL((attn_oproj_kernel<D, NLQ, NLO, BF16, QKV>), grid, block, 0, ctx->stream, a.Wo, a.attn.k_cache,   \
                           a.attn.v_cache, a.attn.q, a.attn.pos_dev, a.step_dev, a.attn.max_seq, a.attn.hq, a.attn.hkv | (S << 16), a.N, \
                           a.Wqkv, a.residual, a.in_norm_w, a);                                                                  \
        launched = true;                                                                                                         \
    } while (0)
// the instances with a q|k|v role: rows of equal length, for head_dim 128 also o_proj rows twice as long; q/k norm: head_dim 128
#define AO_QKV_FORMS(NLQ)                                                            \
    do {                                                                             \
        if (nlo == NLQ && form == 1) AO_LAUNCH(NLQ, NLQ, 1);                          \
        if constexpr (D == 128) {                                                    \
            if (nlo == 2 * NLQ && form == 1) AO_LAUNCH(NLQ, 2 * NLQ, 1);              \
            if (nlo == NLQ && form == 2) AO_LAUNCH(NLQ, NLQ, 2);                      \
            if (nlo == 2 * NLQ && form == 2) AO_LAUNCH(NLQ, 2 * NLQ, 2);              \
        }                                                                            \
    } while (0)
    if (form) {
        if (nlq == 2) AO_QKV_FORMS(2);
        else if (nlq == 4) AO_QKV_FORMS(4);
        else if (nlq == 8) AO_QKV_FORMS(8);
    } else {
        switch (nlo) {
            case 2: AO_LAUNCH(2, 2, 0); break;
            case 4: AO_LAUNCH(4, 4, 0); break;
            case 8: AO_LAUNCH(8, 8, 0); break;
            case 16: AO_LAUNCH(16, 16, 0); break;
        }
    }
#undef AO_QKV_FORMS
#undef AO_LAUNCH
    if (!launched) LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "chained launch: no instance for rows of %d and %d", a.N, a.K);
    LUMEN_CHECK_LAUNCH();
    note_kernel(ctx, "attn_oproj_kernel<%d, %d, %d, %s, %d>", D, form ? nlq : nlo, nlo, BF16 ? "true" : "false", form);
    const int seg[3] = {nq, nq + n_att, n_wg};
    stage_times_report(ctx, "(q|k|v |) attention | o_proj chain", n_wg,
                       "start, then q|k|v: [1] requests out, [2] x staged, [3] acknowledged; attention: [1] rows done, "
                       "[2] merged, [3] stored, [4] acknowledged; o_proj: [5] polls begin, [6] input staged, [7] acknowledged",
                       seg + (nq ? 0 : 1), nq ? 3 : 2);
    return LUMEN_OK;
}

int launch_attn_oproj(lumen_ctx *ctx, const AttnOprojArgs &a) {
    if (!attn_oproj_supported(a.attn.hq, a.attn.hkv, a.attn.d, a.N, a.K, a.w_bf16))
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "attention -> o_proj chain: %d/%d heads of %d, W_o [%d, %d] not covered", a.attn.hq,
                   a.attn.hkv, a.attn.d, a.N, a.K);
    if (!a.attn.pos_dev || a.attn.b != 1 || !a.x_tagged || !a.step_dev || !a.err_dev || !a.attn.out_tagged || !a.t0_tagged)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "attention -> o_proj chain: needs a device position, batch 1 and a hand-over buffer");
    if (a.Wqkv) {
        if (!qkv_attn_oproj_supported(a.attn.hq, a.attn.hkv, a.attn.d, a.N, a.K, a.w_bf16, a.attn.q_norm_w != nullptr))
            LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "q|k|v -> attention -> o_proj chain: hidden %d, %d heads of %d not covered", a.N,
                       a.attn.hq, a.attn.d);
        if (!a.in_norm_w || !a.qkv_tagged || !a.attn.cos_t || !a.attn.sin_t || !a.residual)
            LUMEN_FAIL(LUMEN_ERR_INVALID, "q|k|v -> attention -> o_proj chain: needs norm gains, RoPE tables and a hand-over buffer");
        if ((((uintptr_t)a.Wqkv | (uintptr_t)a.residual | (uintptr_t)a.in_norm_w) & 15) != 0 || (a.row_sel && a.row_stride % 4))
            LUMEN_FAIL(LUMEN_ERR_INVALID, "q|k|v -> attention -> o_proj chain: operands must be 16-byte aligned");
        if (a.attn.q_norm_w && !a.attn.k_norm_w)
            LUMEN_FAIL(LUMEN_ERR_INVALID, "q|k|v -> attention -> o_proj chain: q and k norm gains come together");
    } else if (!a.attn.pre_rotated) {
        LUMEN_FAIL(LUMEN_ERR_INVALID, "attention -> o_proj chain: needs a rotated q and the new cache row in place");
    }
    if ((((uintptr_t)a.Wo | (uintptr_t)a.attn.q | (uintptr_t)a.attn.k_cache | (uintptr_t)a.attn.v_cache) & 15) != 0)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "attention -> o_proj chain: operands must be 16-byte aligned");
    if (a.nslices > 1 && (a.nslices > ATTN_CHAIN_MAX_SLICES || !a.part_tagged || a.attn.hkv > 0xffff || a.slice_rows <= 0 ||
                          (a.slice_rows & (a.slice_rows - 1)) || a.slice_rows % attn_decode_trip_rows(a.attn.d)))
        LUMEN_FAIL(LUMEN_ERR_INVALID, "attention -> o_proj chain: %d slices (at most %d, with a buffer for their states)", a.nslices,
                   ATTN_CHAIN_MAX_SLICES);
    if (!handover_timing_ok(a.spin_limit, a.pre_sleep, a.poll_delay, a.poll_gap))
        LUMEN_FAIL(LUMEN_ERR_INVALID, "attention -> o_proj chain: wait limits out of range (%u polls, pauses %d / %d / %d)",
                   a.spin_limit, a.pre_sleep, a.poll_delay, a.poll_gap);
    if ((size_t)a.attn.max_seq * a.attn.d * sizeof(float) >= ((size_t)1 << 32))
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "attention -> o_proj chain: a KV head of %d rows x %d exceeds 4 GiB", a.attn.max_seq, a.attn.d);
    if (a.attn.d == 64) return a.w_bf16 ? launch_ao<64, true>(ctx, a) : launch_ao<64, false>(ctx, a);
    return a.w_bf16 ? launch_ao<128, true>(ctx, a) : launch_ao<128, false>(ctx, a);
}

LUMEN_DEFINE_WARM(attn_oproj)
