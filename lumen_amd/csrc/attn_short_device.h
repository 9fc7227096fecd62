// The one-workgroup-per-query-head form of decode attention (short caches), shared by the stand-alone
// decode attention kernel (attention.hip) and the attention -> o_proj chain (attn_oproj.hip).
#pragma once
#include "internal.h"
#include "attn_device.h"
#include "stage_times.h"
#include "wave_reduce.h"

// A value handed from one workgroup to another INSIDE a launch travels as one 8-byte word {value bits, tag}: the
// writer stores it with a single agent-scope atomic store, the reader polls it with agent-scope atomic loads until
// the tag is the one it expects.  Value and tag are one atomic object, so a reader that sees the tag has the
// value: no fence, counter or ordering between different locations is involved.
__device__ __forceinline__ void tagged_store(unsigned long long *p, float v, unsigned tag) {
    const unsigned long long w = ((unsigned long long)tag << 32) | (unsigned long long)__float_as_uint(v);
    __hip_atomic_store(p, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long tagged_load(const unsigned long long *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void handover_pause(int n) {
    for (int i = 0; i < n; ++i) __builtin_amdgcn_s_sleep(4);  // 256 clocks each
}
// Pause until `tenths` x 0.1 us after `t0` (a wall_clock64() reading: 100 MHz, whatever the shader clock does --
// what the pauses are timed against is the memory system, which does not follow the shader clock either).
__device__ __forceinline__ void handover_pause_until(unsigned long long t0, int tenths) {
    const unsigned long long ticks = (unsigned long long)(tenths > 0 ? tenths : 0) * 10u;
    while (wall_clock64() - t0 < ticks) __builtin_amdgcn_s_sleep(1);
}
// the same against a 32-bit reading of the clock (differences survive the wrap)
__device__ __forceinline__ void handover_pause_until32(unsigned t0, int tenths) {
    const unsigned ticks = (unsigned)(tenths > 0 ? tenths : 0) * 10u;
    while ((unsigned)wall_clock64() - t0 < ticks) __builtin_amdgcn_s_sleep(1);
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
            handover_pause(gap);
        }
    } while (!ok);
#pragma unroll
    for (int e = 0; e < EPT; ++e) v[e] = __uint_as_float((unsigned)w[e]);
    return ok;
}

// Short contexts (up to ATTN_SHORT_ROWS cached rows; 256 for head_dim 128): one query head per
// workgroup over ALL rows, 8 row loads per lane in flight, so that nothing has to travel between
// workgroups -- at these lengths the hand-over of partial results through memory (an atomic and
// a round of agent-scope loads, each a trip to the memory side) costs more than reading the few
// hundred K/V rows once per query head instead of once per KV head.
#define ATTN_SHORT_ROWS 512
// row loads per lane in flight in one trip of the short form (256 rows per trip for head_dim 64, 128 for
// head_dim 128; 16 loads there would double the kernel's registers and halve the split form's occupancy)
template <int D>
struct ShortTrip {
    static constexpr int loads = 8;
};
// 16 bytes of row j of one KV head: a uniform base pointer and a 32-bit byte offset (a head of the
// cache stays below 4 GiB; the launcher checks), so that a row costs one address register
template <int D>
__device__ __forceinline__ v4f ld_row(const float *head, int j, unsigned c4) {
    return *(const v4f *)((const char *)head + ((unsigned)j * D + c4) * 4u);
}

// bit u set: row first + u * stride lies before `end`
template <int UB>
__device__ __forceinline__ unsigned rows_mask(int first, int stride, int end) {
    unsigned m = 0;
#pragma unroll
    for (int u = 0; u < UB; ++u) m |= (first + u * stride < end ? 1u : 0u) << u;
    return m;
}

// Where q and the new row come from (SRC):
//   ATTN_SRC_RAW     un-rotated projections in memory: this workgroup normalises and rotates its own query head and
//                    the group's new key itself (a few hundred flops, repeated by every head of the group so that
//                    nothing has to be exchanged), the first head of the group stores the new row, and every head
//                    takes that row from LDS (q_rot, k_new, v_new: D floats each);
//   ATTN_SRC_CACHE   q is rotated and cache row pos_new written already (an earlier launch did both);
//   ATTN_SRC_TAGGED  rotated q, new key and new value arrive as tagged words from other workgroups of THIS launch
//                    (which also store the row): they are polled for after the first trip of rows is requested, go to
//                    LDS, and the new row is taken from there;
//   ATTN_SRC_TAGGED_RAW  the same words hold the UN-rotated projections (q/k-norm models): ATTN_SRC_RAW with the
//                    tagged words in the place of the projections in memory.
//
// pos_new < 0: the position is not known yet.  The first trip of rows and the query are requested
// before it is read -- they do not depend on it: a row past the cached ones is only masked later --
// so the position's own trip to memory is off the critical path.  Returns false, having done
// nothing, when the position then turns out to lie past short_rows.
#define ATTN_SRC_RAW 0
#define ATTN_SRC_CACHE 1
#define ATTN_SRC_TAGGED 2
#define ATTN_SRC_TAGGED_RAW 3
//
// SLICED (the chained launch, which may run several workgroups per query head): this workgroup takes the rows
// [slice * R, (slice + 1) * R), R = 1 << a.slice_shift, a whole number of trips, walked trip by trip.  With `n` =
// position / R + 1 slices in use, a workgroup of a later slice returns at once; the slice the new token falls
// into adds the new row; with n == 1 the output is final as in the plain form, else the workgroup leaves its state
// (ctx[D], m, l) as tagged words in a.part_tagged [head][a.tslices][D + 2] for the workgroup that folds the slices
// of the head.
template <int D, int WAVES, int SRC, bool SLICED = false>
__device__ __forceinline__ bool attn_decode_short(const AttnDecodeArgs &a, int r, int nrep, int hk, int bb, int pos_new,
                                                  int short_rows, float *q_rot, float *k_new,
                                                  float *v_new, float *sm, float *sl, float *sacc, int slice = 0) {
    constexpr int LPR = D / 4, RPW = 64 / LPR, RPI = WAVES * RPW, UB = ShortTrip<D>::loads, THREADS = WAVES * 64;
    constexpr bool PRE = SRC == ATTN_SRC_CACHE;
    const int row0 = SLICED ? slice << a.slice_shift : 0;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int off = wave * RPW + lane / LPR, c = lane % LPR;
    const int hq = hk * nrep + r;
    const size_t head_base = ((size_t)bb * a.hkv + hk) * a.max_seq * D;
    // uniform head pointers plus one 32-bit element offset per row, shared by the K and the V load
    const float *Kb = a.k_cache + head_base, *Vb = a.v_cache + head_base;
    const unsigned c4 = c * 4;
    AttnState<1> st;
    state_init<1>(st);
    v4f q[1];
    bool have_q = false;
    // first trip: rows u * RPI + off, clamped to the cache (not to the position: see above)
    v4f kv0[UB], vv0[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        const int j = min(row0 + u * RPI + off, a.max_seq - 1);
        kv0[u] = ld_row<D>(Kb, j, c4);
        vv0[u] = ld_row<D>(Vb, j, c4);
    }
    if (PRE) {
        load_q_scaled<D, 1>(q, a.q + ((size_t)bb * a.hq + hq) * D, c, a.scale);
        have_q = true;
    }
    if (pos_new < 0) pos_new = a.pos_dev ? *a.pos_dev : a.pos_host;
    if (pos_new + 1 > short_rows) return false;
    const int nact = SLICED ? (pos_new >> a.slice_shift) + 1 : 1;  // slices in use
    if (SLICED && slice >= nact) return true;
    const bool owner = !SLICED || slice == nact - 1;  // the new token falls into this slice
    const int pos = SLICED ? min(PRE ? pos_new + 1 : pos_new, row0 + (1 << a.slice_shift)) : (PRE ? pos_new + 1 : pos_new);  // end of the cached rows read here
    auto get_q = [&]() __attribute__((always_inline)) {
        if (PRE) {
            load_q_scaled<D, 1>(q, a.q + ((size_t)bb * a.hq + hq) * D, c, a.scale);
        } else if constexpr (SRC == ATTN_SRC_TAGGED) {
            // wavefronts 0, 1, 2 wait for the query head, the new key and the new value (batch 1)
            constexpr int EPL = D >= 64 ? D / 64 : 1;  // (the chain takes head_dim 64 and 128 only)
            auto take = [&](float *dst, int vec) __attribute__((always_inline)) {
                float v[EPL];
                if (!take_tagged<EPL>(a.qkv_tagged + (size_t)vec * D + lane * EPL, a.tag, a.spin_limit, a.poll_gap, v))
                    __hip_atomic_store(a.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                for (int e = 0; e < EPL; ++e) dst[lane * EPL + e] = v[e];
            };
            if (wave == 0) take(q_rot, hq);
            else if (wave == 1 && owner) take(k_new, a.hq + hk);
            else if (wave == 2 && owner) take(v_new, a.hq + a.hkv + hk);
            __syncthreads();
            load_q_scaled<D, 1>(q, q_rot, c, a.scale);
        } else {
            // wavefront 0 takes the query head, wavefront 1 the new key, wavefront 2 copies the new value:
            // lane j holds the pair (j, j + D/2); everything they need from memory is requested at once
            constexpr int HALF = D / 2;
            constexpr bool WORDS = SRC == ATTN_SRC_TAGGED_RAW;
            const float *cs = a.cos_t + (size_t)pos_new * D, *sn = a.sin_t + (size_t)pos_new * D;
            auto word = [&](size_t i) __attribute__((always_inline)) {  // one tagged word of q | k | v (batch 1)
                float v[1];
                if (!take_tagged<1>(a.qkv_tagged + i, a.tag, a.spin_limit, a.poll_gap, v))
                    __hip_atomic_store(a.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return v[0];
            };
            if (wave == 0 || (wave == 1 && owner)) {
                const float *src = wave == 0 ? a.q + ((size_t)bb * a.hq + hq) * D : a.k_new + ((size_t)bb * a.hkv + hk) * D;
                const size_t wbase = (size_t)(wave == 0 ? hq : a.hq + hk) * D;
                const float *g = wave == 0 ? a.q_norm_w : a.k_norm_w;
                float x1 = 0.f, x2 = 0.f, cc = 0.f, ss_ = 0.f, g1 = 1.f, g2 = 1.f;
                if (lane < HALF) {
                    cc = cs[lane];
                    ss_ = sn[lane];
                    if (g) {
                        g1 = g[lane];
                        g2 = g[lane + HALF];
                    }
                    if (WORDS) {
                        x1 = word(wbase + lane);
                        x2 = word(wbase + lane + HALF);
                    } else {
                        x1 = src[lane];
                        x2 = src[lane + HALF];
                    }
                }
                if (g) {  // per-head RMSNorm before the rotation
                    float sq = x1 * x1 + x2 * x2;
                    sq = wave_sum(sq);
                    const float inv = 1.0f / sqrtf(sq / (float)D + a.norm_eps);
                    x1 = x1 * inv * g1;
                    x2 = x2 * inv * g2;
                }
                float o1, o2;
                {
#pragma clang fp contract(off)  // separate multiplies and add, like the reference's compiled code
                    o1 = x1 * cc - x2 * ss_;
                    o2 = x1 * ss_ + x2 * cc;
                }
                float *dst = wave == 0 ? q_rot : k_new;
                if (lane < HALF) {
                    dst[lane] = o1;
                    dst[lane + HALF] = o2;
                }
            } else if (wave == 2 && owner) {
                const float *v_src = a.v_new + ((size_t)bb * a.hkv + hk) * D;
                for (int i = lane; i < D; i += 64) v_new[i] = WORDS ? word((size_t)(a.hq + a.hkv + hk) * D + i) : v_src[i];
            }
            __syncthreads();
            if (r == 0 && owner) {  // self_attention.rs:161-176: rotated k and raw v go to cache row pos_new
                for (int i = threadIdx.x; i < D; i += THREADS) {
                    a.k_cache[head_base + (size_t)pos_new * D + i] = k_new[i];
                    a.v_cache[head_base + (size_t)pos_new * D + i] = v_new[i];
                }
            }
            load_q_scaled<D, 1>(q, q_rot, c, a.scale);
        }
        have_q = true;
    };
    if (!have_q && (SLICED || pos > 0)) get_q();
    attn_batch<D, UB>(st, q[0], kv0, vv0, rows_mask<UB>(row0 + off, RPI, pos));
    for (int base = row0 + RPI * UB; base < pos; base += RPI * UB) {
        v4f kv[UB], vv[UB];
#pragma unroll
        for (int u = 0; u < UB; ++u) {  // rows past the end are clamped here and masked in attn_batch
            const int j = min(base + u * RPI + off, pos - 1);
            kv[u] = ld_row<D>(Kb, j, c4);
            vv[u] = ld_row<D>(Vb, j, c4);
        }
        attn_batch<D, UB>(st, q[0], kv, vv, rows_mask<UB>(base + off, RPI, pos));
    }
    if (!PRE) {
        if (!have_q) get_q();  // empty cache: the new token attends to itself only
        if (wave == 0 && owner) {  // the new row, from LDS (lane group 0 of wavefront 0)
            const v4f kn = *(const v4f *)(k_new + c * 4), vn = *(const v4f *)(v_new + c * 4);
            attn_step<D, 1>(st, q, kn, vn, lane / LPR == 0);
        }
    }
    STAGE_T(1);
    wave_merge_publish<D, 1>(st, sm, sl, sacc);
    __syncthreads();
    STAGE_T(2);
    for (int dd = threadIdx.x; dd < D; dd += THREADS) {
        float mm, ls, cx;
        wave_fold<D, 1, WAVES>(sm, sl, sacc, 0, dd, mm, ls, cx);
        if (SLICED && nact > 1) {  // one of several slices: the state travels on
            unsigned long long *pt = a.part_tagged + (((size_t)bb * a.hq + hq) * a.tslices + slice) * (D + 2);
            tagged_store(pt + dd, cx, a.tag);
            if (dd == 0) {
                tagged_store(pt + D, mm, a.tag);
                tagged_store(pt + D + 1, ls, a.tag);
            }
        } else if (a.defer_merge) {  // the consumer divides
            float *part0 = a.part + ((size_t)bb * a.hq + hq) * a.nsplit * (D + 2);  // slice 0 of this head
            part0[dd] = cx;
            if (dd == 0) {
                part0[D] = mm;
                part0[D + 1] = ls;
            }
        } else {
            const float o = cx * (1.0f / (ls + 1e-9f));  // self_attention.rs:287-290
            if (a.out_tagged) tagged_store(a.out_tagged + ((size_t)bb * a.hq + hq) * D + dd, o, a.tag);
            else a.out[((size_t)bb * a.hq + hq) * D + dd] = o;
        }
    }
    STAGE_T(3);
    STAGE_T_STORES_DONE(4);
    return true;
}

