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
// Timing of the o_proj workgroups (units of 256 clocks, set by the caller): pre_sleep before the weight requests, so
// that the attention's own few requests enter the memory system first; poll_delay before the first poll and poll_gap
// between polls, because every poll of the 131072 threads is a trip to memory that the weights compete with.
//
// q arrives rotated and cache row `pos` is already written (both by the q|k|v product's epilogue).
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

__device__ __forceinline__ void ao_sleep(int n) {
    for (int i = 0; i < n; ++i) __builtin_amdgcn_s_sleep(4);  // 256 clocks each
}

// This thread's EPT words of a tagged vector, polled until every one carries `tag`; false after `limit` polls.
template <int EPT>
__device__ __forceinline__ bool take_tagged(const unsigned long long *xp, unsigned tag, unsigned limit, int gap, float (&v)[EPT]) {
    unsigned long long w[EPT];
    unsigned spins = 0;
    bool ok;
    do {
        ok = true;
#pragma unroll
        for (int e = 0; e < EPT; ++e) {
            w[e] = tagged_load(xp + e);
            ok = ok && (unsigned)(w[e] >> 32) == tag;
        }
        if (!ok) {
            if (++spins > limit) break;  // never in a healthy launch: give up so that the wavefront exits
            ao_sleep(gap);
        }
    } while (!ok);
#pragma unroll
    for (int e = 0; e < EPT; ++e) v[e] = __uint_as_float((unsigned)w[e]);
    return ok;
}

// D: head_dim; NLO: 16-byte weight loads per lane and row of the o_proj product (its row length is NLO * 64 *
// elements per load).
template <int D, int NLO, bool BF16>
__global__ __launch_bounds__(AO_THREADS) void attn_oproj_kernel(const void *Wo_hot, float *k_cache_hot, float *v_cache_hot,
                                                                const float *q_hot, const int *pos_dev_hot,
                                                                const unsigned *step_dev_hot, int max_seq_hot, int hq_hot,
                                                                int hkv_hot, int N_hot, AttnOprojArgs a_mem) {
    constexpr int VEC = BF16 ? 8 : 4;
    constexpr int ESZ = BF16 ? 2 : 4;
    constexpr int K = NLO * 64 * VEC;  // o_proj row length = hq * D
    constexpr int EPT = K / AO_THREADS;
    static_assert(K % AO_THREADS == 0 && EPT >= 1, "K must be a multiple of the workgroup size");
    __shared__ __align__(16) float q_rot[D];
    __shared__ __align__(16) float k_new[D];
    __shared__ __align__(16) float v_new[D];
    __shared__ __align__(16) float sacc[AO_WAVES * (D > 64 ? D : 64)];
    __shared__ float sm[AO_WAVES], sl[AO_WAVES];
    __shared__ __align__(16) float xs[K];
    STAGE_T(0);
    const int hq = hq_hot, hkv = hkv_hot, N = N_hot;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_o = (N + AO_WAVES - 1) / AO_WAVES;  // o_proj workgroups
    if ((int)blockIdx.x < hq) {
        // ---- attention of one query head.  Workgroups are dealt round-robin over the 8 XCDs: XCD x takes the hq / 8
        // consecutive heads x * hq / 8 ..., so that a KV group's rows are fetched into as few L2s as possible.
        AttnDecodeArgs a = a_mem.attn;
        a.k_cache = k_cache_hot;
        a.v_cache = v_cache_hot;
        a.pos_dev = pos_dev_hot;
        a.q = q_hot;
        a.max_seq = max_seq_hot;
        a.hq = hq;
        a.hkv = hkv;
        a.tag = *step_dev_hot * a_mem.tag_mul + a_mem.tag_add;
        const int b = blockIdx.x;
        const int h = (hq % 8 == 0) ? (b % 8) * (hq / 8) + b / 8 : b;
        const int nrep = hq / hkv;
        // (a cache of any length: the short form walks it trip by trip)
        attn_decode_short<D, AO_WAVES, true>(a, h % nrep, nrep, h / nrep, 0, -1, 0x7fffffff, q_rot, k_new, v_new, sm, sl, sacc);
        return;
    }
    if ((int)blockIdx.x < hq + n_o) {
        // ---- o_proj: one row per wavefront, all of its weights requested at once (rows past N: clamped, not stored)
        const int wg = (int)blockIdx.x - hq;
        const int row = wg * AO_WAVES + wave;
        ao_sleep(a_mem.pre_sleep);  // (the attention's requests go first)
        v4u raw[NLO];
        {
            const char *rp = (const char *)Wo_hot + ((size_t)min(row, N - 1) * K + (size_t)lane * VEC) * ESZ;
#pragma unroll
            for (int i = 0; i < NLO; ++i) raw[i] = __builtin_nontemporal_load((const v4u *)(rp + (size_t)i * 64 * VEC * ESZ));
        }
        const unsigned tag = *step_dev_hot * a_mem.tag_mul + a_mem.tag_add;
        const float *residual = a_mem.residual;
        if (a_mem.row_sel) residual += (long)(*a_mem.row_sel) * a_mem.row_stride;
        const float res = residual[min(row, N - 1)];
        STAGE_T(5);
        // the attention output: this thread's EPT words, polled until every one carries this launch's tag
        ao_sleep(a_mem.poll_delay);
        {
            float v[EPT];
            if (!take_tagged<EPT>(a_mem.x_tagged + (size_t)tid * EPT, tag, a_mem.spin_limit, a_mem.poll_gap, v))
                __hip_atomic_store(a_mem.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int e = 0; e < EPT; ++e) xs[tid * EPT + e] = v[e];
        }
        __syncthreads();
        STAGE_T(6);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NLO; ++i) acc += ao_dot16<BF16>(raw[i], xs + (i * 64 + lane) * VEC);
        acc = wave_sum(acc);
        if (lane == 0 && row < N) {
            const float hv = res + acc;  // src/ops/arithmetic.rs:48-51 via llama.rs:110
            a_mem.y[row] = hv;
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

int attn_oproj_workgroups(int N) { return (N + AO_WAVES - 1) / AO_WAVES; }

template <int D, bool BF16>
static int launch_ao(lumen_ctx *ctx, const AttnOprojArgs &a) {
    const int nlo = ao_nl(a.K, BF16);
    const int n_wg = a.attn.hq + attn_oproj_workgroups(a.N);
    dim3 grid(n_wg), block(AO_THREADS);
#define AO_LAUNCH(NLO)                                                                                                 \
    hipLaunchKernelGGL((attn_oproj_kernel<D, NLO, BF16>), grid, block, 0, ctx->stream, a.Wo, a.attn.k_cache, a.attn.v_cache, \
                       a.attn.q, a.attn.pos_dev, a.step_dev, a.attn.max_seq, a.attn.hq, a.attn.hkv, a.N, a)
    switch (nlo) {
        case 2: AO_LAUNCH(2); break;
        case 4: AO_LAUNCH(4); break;
        case 8: AO_LAUNCH(8); break;
        default: AO_LAUNCH(16); break;
    }
#undef AO_LAUNCH
    LUMEN_CHECK_LAUNCH();
    const int seg[2] = {a.attn.hq, n_wg};
    stage_times_report(ctx, "attention | o_proj chain", n_wg,
                       "start, (attention: rows done, merged, stored, acknowledged), o_proj: polls begin, input staged, acknowledged",
                       seg, 2);
    return LUMEN_OK;
}

int launch_attn_oproj(lumen_ctx *ctx, const AttnOprojArgs &a) {
    if (!attn_oproj_supported(a.attn.hq, a.attn.hkv, a.attn.d, a.N, a.K, a.w_bf16))
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "attention -> o_proj chain: %d/%d heads of %d, W_o [%d, %d] not covered", a.attn.hq,
                   a.attn.hkv, a.attn.d, a.N, a.K);
    if (!a.attn.pos_dev || !a.attn.pre_rotated || a.attn.b != 1 || !a.x_tagged || !a.step_dev || !a.err_dev || !a.attn.out_tagged)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "attention -> o_proj chain: needs a rotated q, a device position, batch 1 and a hand-over buffer");
    if ((((uintptr_t)a.Wo | (uintptr_t)a.attn.q | (uintptr_t)a.attn.k_cache | (uintptr_t)a.attn.v_cache) & 15) != 0)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "attention -> o_proj chain: operands must be 16-byte aligned");
    if ((size_t)a.attn.max_seq * a.attn.d * sizeof(float) >= ((size_t)1 << 32))
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "attention -> o_proj chain: a KV head of %d rows x %d exceeds 4 GiB", a.attn.max_seq, a.attn.d);
    if (a.attn.d == 64) return a.w_bf16 ? launch_ao<64, true>(ctx, a) : launch_ao<64, false>(ctx, a);
    return a.w_bf16 ? launch_ao<128, true>(ctx, a) : launch_ao<128, false>(ctx, a);
}
