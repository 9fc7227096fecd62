// Static KV cache and GQA attention over it.
//
//  * decode (S == 1), src/layers/attention/self_attention.rs:125-297: one
//    workgroup per (query head, slice of the cached positions).  A K/V row is
//    read as 16-byte pieces (D/4 lanes per row), eight row loads per lane in
//    flight; each lane group keeps an online-softmax state (m, l, ctx),
//    merged across lane groups with shuffles and across wavefronts through
//    LDS.  The step is bound by latency, not by bytes (a few tens of KB per
//    compute unit), so the work is spread as widely as it goes: the n_rep
//    heads of a KV group run in workgroups of their own, placed on the same
//    XCD so that the group's rows come from HBM once and from that XCD's L2
//    for the other heads.  A short cache is one slice: nothing travels
//    between workgroups (attn_decode_short).  A long cache is cut into slices
//    of one trip of rows each; partial states go through a small global
//    scratch and the last workgroup of a head to finish folds them in a
//    fixed order, so results are reproducible run to run (attn_decode_slice).
//  * prefill (S > 1), self_attention.rs:308-419 + :519-678: rotate q/k and
//    append to the cache, then either the matrix-core kernel of
//    prefill_attention.hip (head_dim 64 / 128, long prompts) or one workgroup
//    per (query position, KV group) running the decode row loop over the
//    causal prefix.
#include "internal.h"
#include "attn_device.h"
#include "attn_short_device.h"
#include "wave_reduce.h"
#include "stage_times.h"

#define ATT_WAVES 4
#define ATT_THREADS (ATT_WAVES * 64)

// WAVES wavefronts per workgroup: 8, i.e. one trip covers 128 rows of D = 64; the step is ALU-bound
// (scores, exponentials and weighted sums for n_rep heads per row), so slices are kept short and
// spread over many compute units rather than packed into few large workgroups.
template <int D>
struct DecodeWaves {
    static constexpr int value = 8;
};

// Rows [0, pos) of a long cache are cut into nact slices of whole lane-group rounds, one trip of
// rows (ShortTrip loads per lane) each unless the cache is longer than nslices trips.
template <int D, int WAVES>
__device__ __forceinline__ void long_slices(int pos, int nslices, int &nact, int &chunk) {
    constexpr int RPI = WAVES * (64 / (D / 4)), TRIP = RPI * ShortTrip<D>::loads;
    nact = (pos + TRIP - 1) / TRIP;
    nact = nact < 1 ? 1 : (nact > nslices ? nslices : nact);
    chunk = (pos + nact - 1) / nact;
    chunk = (chunk + RPI - 1) / RPI * RPI;
}

// One query head (r of KV group hk) over slice `slice` of nact: rows [slice * chunk, ...) of the cache.
// The partial state (ctx[D], m, l) goes to a.part_tagged[head][slice] as tagged words; the workgroup of the
// last slice in use folds the nact partials: slice weights exp2(m_s - M) from wavefront 0
// (lane s takes slice s), the D context elements by THREADS / D thread groups that each take every
// (THREADS / D)-th slice, their sums added in group order.  !PRE: every workgroup rotates its own
// query head; the last slice also rotates the new key, takes the new row from LDS, and its first
// head stores the row into the cache (self_attention.rs:161-176).
template <int D, int WAVES, bool PRE>
__device__ __forceinline__ bool attn_decode_slice(const AttnDecodeArgs &a, int r, int nrep, int hk, int bb, int pos_new,
                                                  int slice, int nslices, bool fixed, int short_rows, float *q_rot,
                                                  float *k_new, float *v_new, float *sm, float *sl, float *sacc,
                                                  float *w_lds) {
    constexpr int LPR = D / 4, RPW = 64 / LPR, RPI = WAVES * RPW, UB = ShortTrip<D>::loads, THREADS = WAVES * 64;
    constexpr int TRIP = RPI * UB, GROUPS = THREADS / D, JMAX = (64 + GROUPS - 1) / GROUPS;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int off = wave * RPW + lane / LPR, c = lane % LPR;
    const int hq = hk * nrep + r;
    const size_t head_base = ((size_t)bb * a.hkv + hk) * a.max_seq * D;
    // uniform head pointers plus one 32-bit element offset per row, shared by the K and the V load
    const float *Kb = a.k_cache + head_base, *Vb = a.v_cache + head_base;
    const unsigned c4 = c * 4;
    // first trip of rows: requested before anything else, it does not depend on q -- nor, with fixed
    // slices, on the position: a row past the cached ones is only masked later
    v4f kv0[UB], vv0[UB];
    int nact = 0, chunk = TRIP, pos = 0;
    if (pos_new >= 0) {
        pos = PRE ? pos_new + 1 : pos_new;
        if (fixed) nact = max(1, (pos + TRIP - 1) / TRIP);
        else long_slices<D, WAVES>(pos, nslices, nact, chunk);
        if (slice >= nact) return true;
        const int first = min(pos, slice * chunk), last = min(pos, first + chunk) - 1;
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            const int j = max(min(first + u * RPI + off, last), 0);
            kv0[u] = ld_row<D>(Kb, j, c4);
            vv0[u] = ld_row<D>(Vb, j, c4);
        }
    } else {
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            const int j = min(slice * TRIP + u * RPI + off, a.max_seq - 1);
            kv0[u] = ld_row<D>(Kb, j, c4);
            vv0[u] = ld_row<D>(Vb, j, c4);
        }
        pos_new = *a.pos_dev;
        if (pos_new + 1 <= short_rows) return false;
        pos = PRE ? pos_new + 1 : pos_new;
        nact = max(1, (pos + TRIP - 1) / TRIP);
        if (slice >= nact) return true;
    }
    const int p0 = min(pos, slice * chunk), p1 = min(pos, p0 + chunk);
    const bool has_new = !PRE && slice == nact - 1;
    v4f q[1];
    if (PRE) {
        load_q_scaled<D, 1>(q, a.q + ((size_t)bb * a.hq + hq) * D, c, a.scale);
    } else {
        // wavefront 0 takes the query head; in the last slice wavefront 1 takes the new key and
        // wavefront 2 copies the new value: lane j holds the pair (j, j + D/2)
        constexpr int HALF = D / 2;
        const float *cs = a.cos_t + (size_t)pos_new * D, *sn = a.sin_t + (size_t)pos_new * D;
        if (wave == 0 || (wave == 1 && has_new)) {
            const float *src = wave == 0 ? a.q + ((size_t)bb * a.hq + hq) * D : a.k_new + ((size_t)bb * a.hkv + hk) * D;
            const float *g = wave == 0 ? a.q_norm_w : a.k_norm_w;
            float x1 = 0.f, x2 = 0.f, cc = 0.f, ss_ = 0.f, g1 = 1.f, g2 = 1.f;
            if (lane < HALF) {
                x1 = src[lane];
                x2 = src[lane + HALF];
                cc = cs[lane];
                ss_ = sn[lane];
                if (g) {
                    g1 = g[lane];
                    g2 = g[lane + HALF];
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
        } else if (wave == 2 && has_new) {
            const float *v_src = a.v_new + ((size_t)bb * a.hkv + hk) * D;
            for (int i = lane; i < D; i += 64) v_new[i] = v_src[i];
        }
        __syncthreads();
        if (has_new && r == 0) {
            for (int i = t; i < D; i += THREADS) {
                a.k_cache[head_base + (size_t)pos_new * D + i] = k_new[i];
                a.v_cache[head_base + (size_t)pos_new * D + i] = v_new[i];
            }
        }
        load_q_scaled<D, 1>(q, q_rot, c, a.scale);
    }
    AttnState<1> st;
    state_init<1>(st);
    attn_batch<D, UB>(st, q[0], kv0, vv0, rows_mask<UB>(p0 + off, RPI, p1));
    for (int base = p0 + RPI * UB; base < p1; base += RPI * UB) {  // caches longer than nslices trips
        v4f kv[UB], vv[UB];
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            const int j = min(base + u * RPI + off, p1 - 1);
            kv[u] = ld_row<D>(Kb, j, c4);
            vv[u] = ld_row<D>(Vb, j, c4);
        }
        attn_batch<D, UB>(st, q[0], kv, vv, rows_mask<UB>(base + off, RPI, p1));
    }
    if (has_new && wave == 0) {  // the new row, from LDS (lane group 0 of wavefront 0)
        const v4f kn = *(const v4f *)(k_new + c * 4), vn = *(const v4f *)(v_new + c * 4);
        attn_step<D, 1>(st, q, kn, vn, lane / LPR == 0);
    }
    wave_merge_publish<D, 1>(st, sm, sl, sacc);
    __syncthreads();
    float *out_head = a.out + ((size_t)bb * a.hq + hq) * D;
    const size_t part_off = ((size_t)bb * a.hq + hq) * nslices * (D + 2);
    // a slice's state travels as tagged 8-byte words {value, tag} (attn_short_device.h) unless the consumer is a
    // later launch (defer_merge: plain values in a.part)
    unsigned long long *part_head = a.part_tagged + part_off;
    const unsigned tag = (a.tag_dev ? *a.tag_dev : 0u) * a.tag_mul + a.tag_add;
    for (int dd = t; dd < D; dd += THREADS) {
        float mm, ls, cx;
        wave_fold<D, 1, WAVES>(sm, sl, sacc, 0, dd, mm, ls, cx);
        if (nact == 1 && !a.defer_merge) {
            out_head[dd] = cx * (1.0f / (ls + 1e-9f));  // self_attention.rs:287-290
        } else if (a.defer_merge) {
            float *pp = a.part + part_off + (size_t)slice * (D + 2);
            pp[dd] = cx;
            if (dd == 0) {
                pp[D] = mm;
                pp[D + 1] = ls;
            }
        } else {
            unsigned long long *pp = part_head + (size_t)slice * (D + 2);
            tagged_store(pp + dd, cx, tag);
            if (dd == 0) {
                tagged_store(pp + D, mm, tag);
                tagged_store(pp + D + 1, ls, tag);
            }
        }
    }
    if (nact == 1 || a.defer_merge) return true;  // one slice, or the consumer folds them
    // The workgroup of the last slice in use folds the slices of its head.  It has the highest index among them,
    // so it is dispatched last and the others are resident or finished while it waits; it polls their words (and
    // its own) until every one carries this launch's tag: a word that does has its value, whatever the order of
    // other accesses.  The wait is bounded (spin_limit polls, then *err_dev = 1 and the fold goes on with what it has).
    if (slice != nact - 1) return true;
    // fold: context partials of this thread's element and slices, and the slice weights' inputs by wavefront 0
    const int dd = t % D, grp = t / D;
    unsigned long long wv[JMAX], wm = 0, wl = 0;
    {
        unsigned spins = 0;
        bool ok;
        do {
            ok = true;
            if (grp < GROUPS) {
#pragma unroll
                for (int j = 0; j < JMAX; ++j) {
                    wv[j] = tagged_load(part_head + (size_t)min(grp + j * GROUPS, nact - 1) * (D + 2) + dd);
                    ok = ok && (unsigned)(wv[j] >> 32) == tag;
                }
            }
            if (wave == 0) {
                const unsigned long long *pp = part_head + (size_t)min(lane, nact - 1) * (D + 2);
                wm = tagged_load(pp + D);
                wl = tagged_load(pp + D + 1);
                ok = ok && (unsigned)(wm >> 32) == tag && (unsigned)(wl >> 32) == tag;
            }
            if (!ok) {
                if (++spins > a.spin_limit) break;  // never in a healthy launch: give up so that the wavefront exits
                __builtin_amdgcn_s_sleep(2);
            }
        } while (!ok);
        if (!ok && a.err_dev) __hip_atomic_store(a.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    float cv[JMAX];
#pragma unroll
    for (int j = 0; j < JMAX; ++j) cv[j] = __uint_as_float((unsigned)wv[j]);
    // ... then the slice weights, by wavefront 0
    if (wave == 0) {
        float m = __uint_as_float((unsigned)wm), l = __uint_as_float((unsigned)wl);
        if (lane >= nact) {
            m = -INFINITY;
            l = 0.f;
        }
        const float M = wave_max(m);
        const float w = (m > -INFINITY) ? fast_exp2(m - M) : 0.f;
        const float L = wave_sum(l * w);
        w_lds[lane] = w;
        if (lane == 0) w_lds[64] = 1.0f / (L + 1e-9f);
    }
    __syncthreads();
    if (grp < GROUPS) {
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < JMAX; ++j)
            if (grp + j * GROUPS < nact) acc = fmaf(cv[j], w_lds[grp + j * GROUPS], acc);
        sacc[grp * D + dd] = acc;  // sacc is free again: the wavefront states were consumed above
    }
    __syncthreads();
    if (t < D) {
        float acc = 0.f;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) acc += sacc[g * D + t];
        out_head[t] = acc * w_lds[64];
    }
    return true;
}

// PRE: q arrives rotated and cache row `pos` is already written (both done by the q|k|v GEMV's
// epilogue), so the kernel is only the row loop over [0, pos] and the merges.
// Grid: x = n_rep * nslices workgroups per KV head, y = KV head, z = batch.  NREP_T: the group size
// n_rep where it is one of the common ones (index arithmetic with constants), 0 for any other.
template <int D, int NREP_T, int WAVES, bool PRE>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(4, 4))) void attn_decode_kernel(
    float *k_cache_hot, float *v_cache_hot, const int *pos_dev_hot, const float *q_hot, int max_seq_hot, int hkv_hot,
    int start_short, int grid_x, int pos_host_hot, int hq_hot, AttnDecodeArgs a_mem) {
    typedef AttnGeom<D, WAVES> G;
    // The leading scalar arguments repeat the fields that the first trip of row loads depends on, and
    // start_short is the form to try first (decided by the launcher from the position, or from the hint
    // where the position sits in device memory): they are preloaded into scalar registers (see the
    // Makefile), so those loads go out without waiting for a read of the argument block.
    AttnDecodeArgs a = a_mem;
    a.k_cache = k_cache_hot;
    a.v_cache = v_cache_hot;
    a.pos_dev = pos_dev_hot;
    a.max_seq = max_seq_hot;
    a.hkv = hkv_hot;
    a.pos_host = pos_host_hot;
    a.q = q_hot;
    a.hq = hq_hot;
    __shared__ __align__(16) float q_rot[D];
    __shared__ __align__(16) float k_new[D];
    __shared__ __align__(16) float v_new[D];
    // wavefront states [WAVES][D]; the fold of a long cache reuses it for one partial sum per thread
    __shared__ __align__(16) float sacc[WAVES * (D > 64 ? D : 64)];
    __shared__ float sm[WAVES], sl[WAVES], w_lds[65];

    const int split = blockIdx.x, hk = blockIdx.y, bb = blockIdx.z;
    const int NREP = NREP_T ? NREP_T : a.hq / a.hkv;  // query heads per KV head
    // the short form walks the rows in trips, one after the other: two trips at most
    constexpr int SHORT_ROWS = (2 * ShortTrip<D>::loads * G::RPI < ATTN_SHORT_ROWS) ? 2 * ShortTrip<D>::loads * G::RPI : ATTN_SHORT_ROWS;
    // Short form: workgroup `split` takes query head r of the group.  Workgroups are dealt
    // round-robin over the 8 XCDs, each with an L2 of its own; with 32 or more workgroups per KV
    // head the heads of a group are placed 8 apart, four to an XCD, so that a group's K/V rows are
    // fetched into two L2s instead of eight (that placement is for groups of eight heads).
    int r = split;
    if (NREP == 8 && grid_x >= 32 && (grid_x & 7) == 0) r = (split & 7) < 2 && split < 32 ? (split >> 3) + 4 * (split & 7) : NREP;
    // Long form: workgroup `split` takes query head rr over slice `slice`.  With 8 or more slices
    // the heads of one (KV head, slice) sit 8 workgroups apart -- on one XCD -- so the slice's rows
    // reach that XCD's L2 once for all of them.
    const int nslices = grid_x / NREP;  // a power of two
    int slice, rr;
    if (nslices >= 8) {
        slice = (split & 7) | ((split / (8 * NREP)) << 3);
        rr = (split >> 3) % NREP;
    } else {
        slice = split % nslices;
        rr = split / nslices;
    }
    // slices of exactly one trip wherever the whole cache fits into nslices of them; then a
    // workgroup's rows do not depend on the position and are requested before it is read
    const bool fixed = a.max_seq <= nslices * ShortTrip<D>::loads * G::RPI;

    // The form follows the position: the launcher knows it (pos_host, or its own mirror of the device counter) and
    // passes the form to run, so the first trip of rows is requested before the position itself is read.  A form
    // that then finds the cache on the other side of the boundary has been launched wrongly: it writes nothing and
    // flags the launch as failed (*err_dev), which the next synchronising call reports.
    int pos_new = a.pos_dev ? -1 : a.pos_host;  // == past_len, the new token's position
    // (slices longer than a trip depend on the position: it is read first then)
    if (start_short == 0 && pos_new < 0 && !fixed) pos_new = *a.pos_dev;
    bool done;
    if (start_short != 0) {
        if (r >= NREP) return;  // not one of the short form's workgroups
        done = attn_decode_short<D, WAVES, PRE ? ATTN_SRC_CACHE : ATTN_SRC_RAW>(a, r, NREP, hk, bb, pos_new, SHORT_ROWS, q_rot, k_new,
                                                                                 v_new, sm, sl, sacc);
    } else {
        done = attn_decode_slice<D, WAVES, PRE>(a, rr, NREP, hk, bb, pos_new, slice, nslices, fixed, SHORT_ROWS, q_rot, k_new, v_new,
                                                sm, sl, sacc, w_lds);
    }
    if (!done && a.err_dev && threadIdx.x == 0) __hip_atomic_store(a.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// slices of a long cache: one trip of rows each (16384 / head_dim rows: eight 16-byte loads per lane,
// 8 wavefronts), a power of two, 64 at most (the fold takes one slice per lane)
int attn_decode_nsplit(int max_seq, int d) {
    const int trip = 16384 / d;
    int n = 1;
    while (n < 64 && n * trip < max_seq) n *= 2;
    return n;
}

size_t attn_decode_part_floats(int b, int hq, int d, int nsplit) { return (size_t)b * hq * nsplit * (d + 2); }

int attn_decode_trip_rows(int d) { return 16384 / d; }
int attn_decode_short_rows(int d) { return 2 * attn_decode_trip_rows(d) < ATTN_SHORT_ROWS ? 2 * attn_decode_trip_rows(d) : ATTN_SHORT_ROWS; }

template <int D>
static int launch_decode_d(lumen_ctx *ctx, const AttnDecodeArgs &a) {
    constexpr int WAVES = DecodeWaves<D>::value;
    const int nrep = a.hq / a.hkv;
    dim3 grid(nrep * a.nsplit, a.hkv, a.b);
    // the form the kernel tries first: known from the position, or the caller's hint
    const int start_short = a.pos_dev ? (a.expect_short != 0) : (a.pos_host + 1 <= attn_decode_short_rows(D));
    if ((size_t)a.max_seq * D * sizeof(float) >= ((size_t)1 << 32))  // 32-bit byte offsets inside a head
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "decode attention: a KV head of %d rows x %d exceeds 4 GiB", a.max_seq, D);
#define DECODE_HOT a.k_cache, a.v_cache, a.pos_dev, a.q, a.max_seq, a.hkv, start_short, (int)grid.x, a.pos_host, a.hq
#define LAUNCH_DECODE(NR)                                                                                          \
    do {                                                                                                           \
        if (a.pre_rotated)                                                                                         \
            hipLaunchKernelGGL((attn_decode_kernel<D, NR, WAVES, true>), grid, dim3(WAVES * 64), 0, ctx->stream, DECODE_HOT, a);  \
        else                                                                                                       \
            hipLaunchKernelGGL((attn_decode_kernel<D, NR, WAVES, false>), grid, dim3(WAVES * 64), 0, ctx->stream, DECODE_HOT, a); \
    } while (0)
    switch (nrep) {
        case 1: LAUNCH_DECODE(1); break;
        case 2: LAUNCH_DECODE(2); break;
        case 4: LAUNCH_DECODE(4); break;
        case 8: LAUNCH_DECODE(8); break;
        default: LAUNCH_DECODE(0); break;
    }
#undef LAUNCH_DECODE
#undef DECODE_HOT
    LUMEN_CHECK_LAUNCH();
    note_kernel(ctx, "attn_decode_kernel<%d, %d, %d, %s>", D, (nrep == 1 || nrep == 2 || nrep == 4 || nrep == 8) ? nrep : 0, WAVES,
                a.pre_rotated ? "true" : "false");
    return LUMEN_OK;
}

int launch_attn_decode(lumen_ctx *ctx, const AttnDecodeArgs &a) {
    if (a.hkv <= 0 || a.hq % a.hkv) LUMEN_FAIL(LUMEN_ERR_SHAPE, "heads %d not a multiple of kv heads %d", a.hq, a.hkv);
    if (a.defer_merge && (!a.pre_rotated || a.max_seq > a.nsplit * attn_decode_trip_rows(a.d)))
        LUMEN_FAIL(LUMEN_ERR_INVALID, "decode attention: a deferred merge needs a rotated q and one-trip slices");
    switch (a.d) {
        case 16: return launch_decode_d<16>(ctx, a);
        case 32: return launch_decode_d<32>(ctx, a);
        case 64: return launch_decode_d<64>(ctx, a);
        case 128: return launch_decode_d<128>(ctx, a);
        default: LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "decode attention: head_dim=%d (supported 16, 32, 64, 128)", a.d);
    }
}

// ------------------------------------------------------------------- prefill
// q/k-norm + RoPE + cache append for S new positions.
// q_rot [B,S,Hq,D] = rope(q); cache.k[b,hk,past+s,:] = rope(k); cache.v[...] = v
// (encoding.rs:56-123 at offset past_len; self_attention.rs:397-402)
template <int D>
__global__ __launch_bounds__(ATT_THREADS) void prefill_rope_kernel(AttnPrefillArgs a) {
    __shared__ __align__(16) float raw[8 * D];
    __shared__ __align__(16) float rot[8 * D];
    const int ss = blockIdx.x, bb = blockIdx.y;
    const int pos = a.past_len + ss;
    const float *cs = a.cos_t + (size_t)pos * D, *sn = a.sin_t + (size_t)pos * D;
    const float *qrow = a.q + ((size_t)bb * a.s + ss) * a.q_stride;
    const float *krow = a.k + ((size_t)bb * a.s + ss) * a.k_stride;
    const float *vrow = a.v + ((size_t)bb * a.s + ss) * a.v_stride;
    float *qo = a.q_rot + ((size_t)bb * a.s + ss) * (size_t)a.hq * D;
    for (int h0 = 0; h0 < a.hq; h0 += 8) {
        const int nh = min(8, a.hq - h0);
        __syncthreads();
        for (int i = threadIdx.x; i < nh * D; i += ATT_THREADS) raw[i] = qrow[(size_t)h0 * D + i];
        __syncthreads();
        norm_rope_heads<D>(raw, rot, nh, cs, sn, a.q_norm_w, a.norm_eps, ATT_THREADS);
        __syncthreads();
        for (int i = threadIdx.x; i < nh * D; i += ATT_THREADS) qo[(size_t)h0 * D + i] = rot[i];
    }
    for (int h0 = 0; h0 < a.hkv; h0 += 8) {
        const int nh = min(8, a.hkv - h0);
        __syncthreads();
        for (int i = threadIdx.x; i < nh * D; i += ATT_THREADS) raw[i] = krow[(size_t)h0 * D + i];
        __syncthreads();
        norm_rope_heads<D>(raw, rot, nh, cs, sn, a.k_norm_w, a.norm_eps, ATT_THREADS);
        __syncthreads();
        for (int i = threadIdx.x; i < nh * D; i += ATT_THREADS) {
            const int hk = h0 + i / D, dd = i % D;
            const size_t dst = (((size_t)bb * a.hkv + hk) * a.max_seq + pos) * D + dd;
            a.k_cache[dst] = rot[i];
            a.v_cache[dst] = vrow[(size_t)hk * D + dd];
        }
    }
}

// The same with 16-byte accesses: no LDS, no barriers, all heads of a position at once, four pairs (or four values of
// v) per thread; the sum of squares of a q/k norm is taken over the head's D / 8 neighbouring lanes.  The inputs may be the K splits of the
// q|k|v product, added here in split order (one launch and one pass over q|k|v less than a separate sum).
#define ROPE_MAX_SPLITS 16
template <int D, bool SPLIT, bool NORM>
__global__ __launch_bounds__(ATT_THREADS) void prefill_rope_sum_kernel(AttnPrefillArgs a) {
    constexpr int HALF = D / 2, UPH = HALF / 4, VPH = D / 4;  // units of four per head
    const int ss = blockIdx.x, bb = blockIdx.y;
    const int pos = a.past_len + ss;
    const float *cs = a.cos_t + (size_t)pos * D, *sn = a.sin_t + (size_t)pos * D;
    const size_t row = (size_t)bb * a.s + ss;
    const float *qrow = a.q + row * a.q_stride, *krow = a.k + row * a.k_stride, *vrow = a.v + row * a.v_stride;
    float *qo = a.q_rot + row * (size_t)a.hq * D;
    const int nq = a.hq * UPH, nk = a.hkv * UPH, nv = a.hkv * VPH;
    const int splits = a.in_splits > 1 ? a.in_splits : 1;
    const size_t sst = a.in_split_stride;
    // all splits are requested before the first is added: one trip to memory, not one per split
    auto sum4 = [&](const float *src) {
        if (!SPLIT) return *(const v4f *)src;
        v4f pv[ROPE_MAX_SPLITS];
#pragma unroll
        for (int i = 0; i < ROPE_MAX_SPLITS; ++i)
            if (i < splits) pv[i] = *(const v4f *)(src + (size_t)i * sst);
        v4f v = pv[0];
#pragma unroll
        for (int i = 1; i < ROPE_MAX_SPLITS; ++i)
            if (i < splits) v += pv[i];
        return v;
    };
    {
        const int u = blockIdx.z * ATT_THREADS + threadIdx.x;
        if (u >= nq + nk + nv) return;
        if (u < nq + nk) {
            const bool isq = u < nq;
            const int uu = isq ? u : u - nq, h = uu / UPH, j = (uu % UPH) * 4;
            const float *src = (isq ? qrow : krow) + (size_t)h * D + j;
            v4f x1 = sum4(src), x2 = sum4(src + HALF);
            if (NORM) {
                // q/k norm over the head (rms_norm.rs:45-58 on [.., D]): the head's D / 8 units are neighbouring lanes
                const float *g = isq ? a.q_norm_w : a.k_norm_w;
                if (g) {
                    float sq = x1.x * x1.x + x1.y * x1.y + x1.z * x1.z + x1.w * x1.w + x2.x * x2.x + x2.y * x2.y + x2.z * x2.z +
                               x2.w * x2.w;
#pragma unroll
                    for (int o = 1; o < UPH; o <<= 1) sq += __shfl_xor(sq, o, 64);
                    const float inv = 1.0f / sqrtf(sq / (float)D + a.norm_eps);
                    const v4f g1 = *(const v4f *)(g + j), g2 = *(const v4f *)(g + j + HALF);
                    x1 = x1 * inv * g1;
                    x2 = x2 * inv * g2;
                }
            }
            const v4f c = *(const v4f *)(cs + j), s = *(const v4f *)(sn + j);
            v4f r1, r2;
            {
#pragma clang fp contract(off)  // separate multiplies and add, like the reference's compiled code
                r1 = x1 * c - x2 * s;
                r2 = x1 * s + x2 * c;
            }
            float *dst = isq ? qo + (size_t)h * D + j : a.k_cache + (((size_t)bb * a.hkv + h) * a.max_seq + pos) * D + j;
            *(v4f *)dst = r1;
            *(v4f *)(dst + HALF) = r2;
        } else {
            const int uu = u - nq - nk, h = uu / VPH, j = (uu % VPH) * 4;
            *(v4f *)(a.v_cache + (((size_t)bb * a.hkv + h) * a.max_seq + pos) * D + j) = sum4(vrow + (size_t)h * D + j);
        }
    }
}

static bool prefill_rope_sum_ok(const AttnPrefillArgs &a) {
    if (a.d < 8) return false;
    const uintptr_t ptrs = (uintptr_t)a.q | (uintptr_t)a.k | (uintptr_t)a.v | (uintptr_t)a.q_rot | (uintptr_t)a.k_cache |
                           (uintptr_t)a.v_cache | (uintptr_t)a.cos_t | (uintptr_t)a.sin_t | (uintptr_t)a.q_norm_w |
                           (uintptr_t)a.k_norm_w;
    return (ptrs & 15) == 0 && ((a.q_stride | a.k_stride | a.v_stride) & 3) == 0 && (a.in_split_stride & 3) == 0 &&
           a.in_splits <= ROPE_MAX_SPLITS;
}

// One workgroup per (query position, KV group): scores over the causal prefix
// j <= past_len + i (softmax_inplace_view, self_attention.rs:643-678), ctx = P V,
// out [B,S,Hq,D] (BSHD, :534).
template <int D, int NREP>
__global__ __launch_bounds__(ATT_THREADS) void attn_prefill_kernel(AttnPrefillArgs a) {
    typedef AttnGeom<D, ATT_WAVES> G;
    __shared__ __align__(16) float sacc[ATT_WAVES * NREP * D];
    __shared__ float sm[ATT_WAVES * NREP], sl[ATT_WAVES * NREP];
    // blockIdx.y: KV head, or (NREP == 1 with a.kv_div = n_rep) query head of KV head blockIdx.y / n_rep
    const int i = blockIdx.x, hk = blockIdx.y, bb = blockIdx.z;
    const int L = a.past_len + a.s;
    const int q_abs = a.past_len + i;
    const int p1 = a.causal ? min(L, q_abs + 1) : L;
    const size_t head_base = ((size_t)bb * a.hkv + hk / a.kv_div) * a.max_seq * D;
    const int c = (threadIdx.x & 63) % G::LPR;
    const float *qr = a.q_rot + (((size_t)bb * a.s + i) * a.hq + (size_t)hk * NREP) * D;
    v4f q[NREP];
    load_q_scaled<D, NREP>(q, qr, c, a.scale);
    AttnState<NREP> st;
    state_init<NREP>(st);
    attn_rows<D, NREP, ATT_WAVES>(st, q, a.k_cache + head_base, a.v_cache + head_base, 0, p1);
    wave_merge_publish<D, NREP>(st, sm, sl, sacc);
    __syncthreads();
    for (int e = threadIdx.x; e < NREP * D; e += ATT_THREADS) {
        const int r = e / D, dd = e % D;
        float mm, ls, cx;
        wave_fold<D, NREP, ATT_WAVES>(sm, sl, sacc, r, dd, mm, ls, cx);
        a.out[(((size_t)bb * a.s + i) * a.hq + hk * NREP + r) * D + dd] = cx * (1.0f / (ls + 1e-9f));
    }
}

template <int D>
static int launch_prefill_d(lumen_ctx *ctx, const AttnPrefillArgs &a) {
    if (prefill_rope_sum_ok(a)) {
        const int units = (a.hq + a.hkv) * (D / 8) + a.hkv * (D / 4);  // of four pairs / four values of v
        const dim3 rgrid(a.s, a.b, (units + ATT_THREADS - 1) / ATT_THREADS);
        const bool norm = a.q_norm_w || a.k_norm_w;
        if (a.in_splits > 1) {
            if (norm) hipLaunchKernelGGL((prefill_rope_sum_kernel<D, true, true>), rgrid, dim3(ATT_THREADS), 0, ctx->stream, a);
            else hipLaunchKernelGGL((prefill_rope_sum_kernel<D, true, false>), rgrid, dim3(ATT_THREADS), 0, ctx->stream, a);
        } else {
            if (norm) hipLaunchKernelGGL((prefill_rope_sum_kernel<D, false, true>), rgrid, dim3(ATT_THREADS), 0, ctx->stream, a);
            else hipLaunchKernelGGL((prefill_rope_sum_kernel<D, false, false>), rgrid, dim3(ATT_THREADS), 0, ctx->stream, a);
        }
    } else {
        if (a.in_splits > 1) LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "prefill attention: split q|k|v inputs need 16-byte alignment");
        hipLaunchKernelGGL(prefill_rope_kernel<D>, dim3(a.s, a.b), dim3(ATT_THREADS), 0, ctx->stream, a);
    }
    LUMEN_CHECK_LAUNCH();
    if (attn_prefill_mfma_supported(a)) return launch_attn_prefill_mfma(ctx, a);  // head_dim 64 / 128: matrix cores
    dim3 grid(a.s, a.hkv, a.b), block(ATT_THREADS);
    const int nrep = a.hq / a.hkv;
    switch (nrep) {
        case 1: hipLaunchKernelGGL((attn_prefill_kernel<D, 1>), grid, block, 0, ctx->stream, a); break;
        case 2: hipLaunchKernelGGL((attn_prefill_kernel<D, 2>), grid, block, 0, ctx->stream, a); break;
        case 4: hipLaunchKernelGGL((attn_prefill_kernel<D, 4>), grid, block, 0, ctx->stream, a); break;
        case 8: hipLaunchKernelGGL((attn_prefill_kernel<D, 8>), grid, block, 0, ctx->stream, a); break;
        default: {  // any other group size: one query head per workgroup, its KV head = head / n_rep
            AttnPrefillArgs b = a;
            b.kv_div = nrep;
            hipLaunchKernelGGL((attn_prefill_kernel<D, 1>), dim3(a.s, a.hq, a.b), block, 0, ctx->stream, b);
        }
    }
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

int launch_attn_prefill(lumen_ctx *ctx, const AttnPrefillArgs &a_in) {
    AttnPrefillArgs a = a_in;
    a.kv_div = 1;
    if (a.hkv <= 0 || a.hq % a.hkv) LUMEN_FAIL(LUMEN_ERR_SHAPE, "heads %d not a multiple of kv heads %d", a.hq, a.hkv);
    if (a.s <= 0) return LUMEN_OK;
    switch (a.d) {
        case 16: return launch_prefill_d<16>(ctx, a);
        case 32: return launch_prefill_d<32>(ctx, a);
        case 64: return launch_prefill_d<64>(ctx, a);
        case 128: return launch_prefill_d<128>(ctx, a);
        default: LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "prefill attention: head_dim=%d (supported 16, 32, 64, 128)", a.d);
    }
}

// ------------------------------------------------------------------ KV cache
// legacy LlamaKVCache::update, src/kv_cache.rs:31-49: [B,Hkv,S,D] -> cache[.., start..start+S, ..]
__global__ __launch_bounds__(256) void kv_update_kernel(const float *__restrict__ src, float *__restrict__ dst, int s,
                                                        int d, int max_seq, int start, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const size_t dd = i % d, ss = (i / d) % s, bh = i / ((size_t)d * s);
        dst[(bh * max_seq + start + ss) * d + dd] = src[i];
    }
}

// legacy LlamaKVCache::get_view, src/kv_cache.rs:51-59: copy of the first cur positions
__global__ __launch_bounds__(256) void kv_view_kernel(const float *__restrict__ src, float *__restrict__ dst, int cur,
                                                      int d, int max_seq, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const size_t dd = i % d, ss = (i / d) % cur, bh = i / ((size_t)d * cur);
        dst[i] = src[(bh * max_seq + ss) * d + dd];
    }
}

static unsigned ew_blocks(lumen_ctx *ctx, size_t n) {
    size_t blocks = (n + 255) / 256;
    const size_t cap = (size_t)ctx->num_cus * 16;
    return (unsigned)(blocks > cap ? cap : (blocks ? blocks : 1));
}

extern "C" int lumen_kv_cache_create(lumen_ctx *ctx, int b, int h_kv, int max_seq, int d, lumen_kv_cache **out) {
    if (!ctx || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "kv_cache_create: null argument");
    if (b <= 0 || h_kv <= 0 || max_seq <= 0 || d <= 0)
        LUMEN_FAIL(LUMEN_ERR_SHAPE, "kv_cache_create: b=%d h_kv=%d max_seq=%d d=%d", b, h_kv, max_seq, d);
    lumen_kv_cache *c = new lumen_kv_cache();
    c->ctx = ctx; c->b = b; c->h_kv = h_kv; c->max_seq = max_seq; c->d = d; c->len = 0; c->owns = true;
    const size_t bytes = sizeof(float) * (size_t)b * h_kv * max_seq * d;
    if (hipMalloc((void **)&c->k, bytes) != hipSuccess || hipMalloc((void **)&c->v, bytes) != hipSuccess) {
        hipFree(c->k);
        delete c;
        LUMEN_FAIL(LUMEN_ERR_HIP, "kv_cache_create: hipMalloc of 2 x %zu bytes failed", bytes);
    }
    // zero-initialised like Array4::zeros (self_attention.rs:35-36); eager, never graph-captured
    if (hipMemsetAsync(c->k, 0, bytes, ctx->stream) != hipSuccess || hipMemsetAsync(c->v, 0, bytes, ctx->stream) != hipSuccess ||
        hipStreamSynchronize(ctx->stream) != hipSuccess) {
        hipFree(c->k);
        hipFree(c->v);
        delete c;
        LUMEN_FAIL(LUMEN_ERR_HIP, "kv_cache_create: clearing 2 x %zu bytes failed", bytes);
    }
    *out = c;
    return LUMEN_OK;
}

extern "C" int lumen_kv_cache_destroy(lumen_kv_cache *c) {
    if (!c) return LUMEN_OK;
    hipStreamSynchronize(c->ctx->stream);
    if (c->owns) {
        hipFree(c->k);
        hipFree(c->v);
    }
    hipFree(c->part_tagged);
    hipFree(c->q_rot);
    hipFree(c->d_pos);
    delete c;
    return LUMEN_OK;
}

extern "C" int lumen_kv_cache_reset(lumen_kv_cache *c) {
    if (!c) LUMEN_FAIL(LUMEN_ERR_INVALID, "kv_cache_reset: null");
    c->len = 0;  // self_attention.rs:41-43
    return LUMEN_OK;
}

extern "C" int lumen_kv_cache_len(const lumen_kv_cache *c, int *len_out) {
    if (!c || !len_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "kv_cache_len: null");
    *len_out = c->len;
    return LUMEN_OK;
}

extern "C" int lumen_kv_cache_set_len(lumen_kv_cache *c, int len) {
    if (!c) LUMEN_FAIL(LUMEN_ERR_INVALID, "kv_cache_set_len: null");
    if (len < 0 || len > c->max_seq) LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "kv_cache_set_len: %d outside [0, %d]", len, c->max_seq);
    c->len = len;
    return LUMEN_OK;
}

extern "C" int lumen_kv_cache_ptrs(const lumen_kv_cache *c, float **k_out, float **v_out) {
    if (!c || !k_out || !v_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "kv_cache_ptrs: null");
    *k_out = c->k;
    *v_out = c->v;
    return LUMEN_OK;
}

extern "C" int lumen_kv_cache_update(lumen_kv_cache *c, const float *k, const float *v, int s, int start_pos) {
    if (!c || !k || !v) LUMEN_FAIL(LUMEN_ERR_INVALID, "kv_cache_update: null");
    if (s < 0 || start_pos < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "kv_cache_update: negative argument");
    if (start_pos + s > c->max_seq)  // kv_cache.rs:33-36
        LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "KV Cache overflow! Max: %d, Current: %d", c->max_seq, start_pos + s);
    const size_t n = (size_t)c->b * c->h_kv * s * c->d;
    if (!n) return LUMEN_OK;
    hipLaunchKernelGGL(kv_update_kernel, dim3(ew_blocks(c->ctx, n)), dim3(256), 0, c->ctx->stream, k, c->k, s, c->d,
                       c->max_seq, start_pos, n);
    hipLaunchKernelGGL(kv_update_kernel, dim3(ew_blocks(c->ctx, n)), dim3(256), 0, c->ctx->stream, v, c->v, s, c->d,
                       c->max_seq, start_pos, n);
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

extern "C" int lumen_kv_cache_get_view(const lumen_kv_cache *c, int cur, float *k_out, float *v_out) {
    if (!c || !k_out || !v_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "kv_cache_get_view: null");
    if (cur < 0 || cur > c->max_seq) LUMEN_FAIL(LUMEN_ERR_SHAPE, "kv_cache_get_view: current_len %d outside [0,%d]", cur, c->max_seq);
    const size_t n = (size_t)c->b * c->h_kv * cur * c->d;
    if (!n) return LUMEN_OK;
    hipLaunchKernelGGL(kv_view_kernel, dim3(ew_blocks(c->ctx, n)), dim3(256), 0, c->ctx->stream, c->k, k_out, cur, c->d,
                       c->max_seq, n);
    hipLaunchKernelGGL(kv_view_kernel, dim3(ew_blocks(c->ctx, n)), dim3(256), 0, c->ctx->stream, c->v, v_out, cur, c->d,
                       c->max_seq, n);
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

static int ensure_split_scratch(lumen_kv_cache *c, int hq, int nsplit) {
    if (c->part_tagged && c->part_heads >= hq) return LUMEN_OK;
    hipStreamSynchronize(c->ctx->stream);
    hipFree(c->part_tagged);
    c->part_tagged = nullptr;
    const size_t bytes = sizeof(unsigned long long) * attn_decode_part_floats(c->b, hq, c->d, nsplit);
    HIP_TRY(hipMalloc((void **)&c->part_tagged, bytes));
    HIP_TRY(hipMemsetAsync(c->part_tagged, 0, bytes, c->ctx->stream));  // (no word carries a tag yet)
    c->part_heads = hq;
    return LUMEN_OK;
}

// The decode step of SelfAttention::forward behind both entry points: checks, launch, len += 1.
static int attn_decode_entry(lumen_kv_cache *c, lumen_rope *rope, const float *q3, const float *k3, const float *v3,
                             float *out, int h, float scale, unsigned long long *part_tagged, const unsigned *tag_dev,
                             unsigned tag_add, int nsplit) {
    const int past_len = c->len, new_len = past_len + 1;
    AttnDecodeArgs a = {};
    a.q = q3; a.k_new = k3; a.v_new = v3; a.out = out;
    a.k_cache = c->k; a.v_cache = c->v; a.cos_t = rope->cos_dev; a.sin_t = rope->sin_dev;
    a.pos_dev = nullptr; a.pos_host = past_len;
    a.b = c->b; a.hq = h; a.hkv = c->h_kv; a.d = c->d; a.max_seq = c->max_seq; a.scale = scale;
    a.q_norm_w = nullptr; a.k_norm_w = nullptr; a.norm_eps = 0.f;
    a.part_tagged = part_tagged; a.tag_dev = tag_dev; a.tag_mul = 1; a.tag_add = tag_add; a.nsplit = nsplit;
    a.spin_limit = HANDOVER_MAX_SPINS; a.err_dev = c->ctx->err_host;
    LUMEN_TRY(launch_attn_decode(c->ctx, a));
    c->len = new_len;
    return LUMEN_OK;
}

static int check_attn_decode(const lumen_kv_cache *c, const lumen_rope *rope, const float *q3, const float *k3,
                             const float *v3, const float *out, int h) {
    if (!c || !rope || !q3 || !k3 || !v3 || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "attn_decode: null argument");
    if (rope->dim != c->d) LUMEN_FAIL(LUMEN_ERR_SHAPE, "RoPE dimension mismatch: %d vs head_dim %d", rope->dim, c->d);
    if (h <= 0 || h % c->h_kv) LUMEN_FAIL(LUMEN_ERR_SHAPE, "attn_decode: %d heads over %d kv heads", h, c->h_kv);
    const int past_len = c->len, new_len = past_len + 1;
    if (new_len > c->max_seq)  // self_attention.rs:144-149
        LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "KV cache overflow: new_len=%d > max_seq=%d", new_len, c->max_seq);
    if (past_len >= rope->max_seq)  // encoding.rs:176-181
        LUMEN_FAIL(LUMEN_ERR_ROPE_RANGE, "RoPE index out of range: pos %d >= max %d", past_len, rope->max_seq);
    return LUMEN_OK;
}

extern "C" int lumen_attn_decode_f32(lumen_kv_cache *c, lumen_rope *rope, const float *q3, const float *k3,
                                     const float *v3, float *out, int h, float scale, int causal) {
    (void)causal;  // the causal test `j > past_len` never fires for S == 1 (self_attention.rs:256)
    LUMEN_TRY(check_attn_decode(c, rope, q3, k3, v3, out, h));
    const int nsplit = attn_decode_nsplit(c->max_seq, c->d);
    LUMEN_TRY(ensure_split_scratch(c, h, nsplit));
    // (the tag of this launch comes from the host: every call is a launch of its own with its own arguments)
    if (++c->merge_epoch == 0) c->merge_epoch = 1;
    return attn_decode_entry(c, rope, q3, k3, v3, out, h, scale, c->part_tagged, nullptr, c->merge_epoch, nsplit);
}

// ------------------------------------------------ the fused decode step of SelfAttention::forward, as two operators
__global__ void set_int_kernel(int *p, int v) { *p = v; }

// RMSNorm + q|k|v product + RoPE + cache append in one launch: what self_attention.rs:106-108 (projections),
// :161-176 (new row into the cache) and :220-227 (rotation of q) do for S == 1, with the input norm of
// llama.rs:107 on the way in.  W [(h + 2 h_kv) * d, K]: the rows of w_q, w_k, w_v one after the other.
// q comes back rotated; the cache length does NOT advance (lumen_attn_decode_prerotated_f32 does that).
extern "C" int lumen_qkv_rope_append_f32(lumen_kv_cache *c, lumen_rope *rope, const void *Wqkv, int w_bf16, const float *x,
                                         int K, const float *norm_w, float eps, float *q_rot_out, int h) {
    if (!c || !rope || !Wqkv || !x || !q_rot_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "qkv_rope_append: null argument");
    if (c->b != 1) LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "qkv_rope_append: batch 1 only (cache batch %d)", c->b);
    if (rope->dim != c->d) LUMEN_FAIL(LUMEN_ERR_SHAPE, "RoPE dimension mismatch: %d vs head_dim %d", rope->dim, c->d);
    if (h <= 0 || h % c->h_kv) LUMEN_FAIL(LUMEN_ERR_SHAPE, "qkv_rope_append: %d heads over %d kv heads", h, c->h_kv);
    if (c->d % 2 || K <= 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "qkv_rope_append: head_dim %d, K %d", c->d, K);
    if (c->len + 1 > c->max_seq)  // self_attention.rs:144-149
        LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "KV cache overflow: new_len=%d > max_seq=%d", c->len + 1, c->max_seq);
    if (c->len >= rope->max_seq)  // encoding.rs:176-181
        LUMEN_FAIL(LUMEN_ERR_ROPE_RANGE, "RoPE index out of range: pos %d >= max %d", c->len, rope->max_seq);
    lumen_ctx *ctx = c->ctx;
    HIP_TRY(hipSetDevice(ctx->device));
    if (!c->d_pos) HIP_TRY(hipMalloc(&c->d_pos, sizeof(int)));
    hipLaunchKernelGGL(set_int_kernel, dim3(1), dim3(1), 0, ctx->stream, c->d_pos, c->len);
    LUMEN_CHECK_LAUNCH();
    GemvArgs g = {};
    g.W = Wqkv; g.x = x; g.y = q_rot_out; g.N = (h + 2 * c->h_kv) * c->d; g.K = K; g.w_bf16 = w_bf16 ? 1 : 0;
    g.pro = norm_w ? PRO_RMSNORM : PRO_NONE; g.norm_w = norm_w; g.eps = eps;
    g.epi = EPI_ROPE_QKV; g.cos_t = rope->cos_dev; g.sin_t = rope->sin_dev; g.pos = c->d_pos;
    g.k_cache = c->k; g.v_cache = c->v; g.hq = h; g.hkv = c->h_kv; g.D = c->d; g.max_seq = c->max_seq;
    return launch_gemv(ctx, g);
}

// Decode attention over the cache INCLUDING the row lumen_qkv_rope_append_f32 just wrote, q rotated already
// (self_attention.rs:183-297); the cache length advances by one.
extern "C" int lumen_attn_decode_prerotated_f32(lumen_kv_cache *c, const float *q_rot, float *out, int h, float scale) {
    if (!c || !q_rot || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "attn_decode_prerotated: null argument");
    if (h <= 0 || h % c->h_kv) LUMEN_FAIL(LUMEN_ERR_SHAPE, "attn_decode: %d heads over %d kv heads", h, c->h_kv);
    if (c->len + 1 > c->max_seq)
        LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "KV cache overflow: new_len=%d > max_seq=%d", c->len + 1, c->max_seq);
    const int nsplit = attn_decode_nsplit(c->max_seq, c->d);
    LUMEN_TRY(ensure_split_scratch(c, h, nsplit));
    AttnDecodeArgs a = {};
    a.q = q_rot; a.out = out; a.k_cache = c->k; a.v_cache = c->v;
    a.pos_dev = nullptr; a.pos_host = c->len;
    a.b = c->b; a.hq = h; a.hkv = c->h_kv; a.d = c->d; a.max_seq = c->max_seq; a.scale = scale;
    if (++c->merge_epoch == 0) c->merge_epoch = 1;
    a.part_tagged = c->part_tagged; a.tag_mul = 1; a.tag_add = c->merge_epoch; a.nsplit = nsplit; a.pre_rotated = 1;
    a.spin_limit = HANDOVER_MAX_SPINS; a.err_dev = c->ctx->err_host;
    LUMEN_TRY(launch_attn_decode(c->ctx, a));
    c->len += 1;
    return LUMEN_OK;
}

// ------------------------------------------------ decode attention that allocates nothing
// The slices of a long cache hand their partial states (ctx[D], m, l per query head and slice, as tagged 8-byte
// words) from workgroup to workgroup through device memory.  lumen_attn_decode_f32 keeps that scratch on the cache
// object and allocates it at the first call; this variant takes it from a fixed array in the library's own device
// image instead, so it never calls an allocator.  Every GPU holds its own copy of the array for the life of the
// process; host code reaches it only through the address hipGetSymbolAddress gives on that GPU (the array's name in
// host code is a host-side stand-in, not a device address).  The first 256 bytes hold the count of launches the
// tags are made of -- in device memory, advanced by a one-thread kernel in front of every launch, so that a call
// recorded into a graph carries a new tag at every replay.
#define ATTN_STATIC_HEAD 256                         // the launch count (4 bytes used)
#define ATTN_STATIC_BYTES ((size_t)4 << 20)          // launch count + partial states
static __device__ __align__(256) unsigned char scratch[ATTN_STATIC_BYTES];

// called by lumen_ctx_create with the context's device current
int attn_static_scratch_init(lumen_ctx *ctx) {
    void *p = nullptr;
    HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p || ((uintptr_t)p & 255)) LUMEN_FAIL(LUMEN_ERR_HIP, "static attention scratch: bad device address %p", p);
    ctx->attn_static = (unsigned char *)p;
    ctx->attn_static_bytes = ATTN_STATIC_BYTES;
    return LUMEN_OK;
}

// the next launch's tag: 1, 2, ... (0 is what an untouched word carries)
__global__ void next_epoch_kernel(unsigned *epoch) {
    unsigned e = *epoch + 1u;
    *epoch = e ? e : 1u;
}

extern "C" int lumen_attn_decode_static_f32(lumen_kv_cache *c, lumen_rope *rope, const float *q3, const float *k3,
                                            const float *v3, float *out, int h, float scale, int causal) {
    (void)causal;
    LUMEN_TRY(check_attn_decode(c, rope, q3, k3, v3, out, h));
    lumen_ctx *ctx = c->ctx;
    if (!ctx->attn_static) LUMEN_FAIL(LUMEN_ERR_HIP, "attn_decode_static: the context holds no static scratch address");
    const int nsplit = attn_decode_nsplit(c->max_seq, c->d);
    const size_t need = ATTN_STATIC_HEAD + sizeof(unsigned long long) * attn_decode_part_floats(c->b, h, c->d, nsplit);
    if (need > ctx->attn_static_bytes)
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED,
                   "attn_decode_static: batch %d x %d heads x %d slices x head_dim %d needs %zu bytes of partial states; "
                   "the static scratch holds %zu bytes (use lumen_attn_decode_f32)",
                   c->b, h, nsplit, c->d, need, ctx->attn_static_bytes);
    unsigned *epoch = (unsigned *)ctx->attn_static;
    unsigned long long *part_tagged = (unsigned long long *)(ctx->attn_static + ATTN_STATIC_HEAD);
    // the array keeps what the last call left: words with older tags, which this launch's readers pass over
    hipLaunchKernelGGL(next_epoch_kernel, dim3(1), dim3(1), 0, ctx->stream, epoch);
    LUMEN_CHECK_LAUNCH();
    return attn_decode_entry(c, rope, q3, k3, v3, out, h, scale, part_tagged, epoch, 0, nsplit);
}

extern "C" int lumen_attn_prefill_f32(lumen_kv_cache *c, lumen_rope *rope, const float *q, const float *k,
                                      const float *v, float *out, int s, int h, float scale, int causal) {
    if (!c || !rope || !q || !k || !v || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "attn_prefill: null argument");
    if (rope->dim != c->d) LUMEN_FAIL(LUMEN_ERR_SHAPE, "RoPE dimension mismatch: %d vs head_dim %d", rope->dim, c->d);
    if (h <= 0 || h % c->h_kv || s < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "attn_prefill: s=%d, %d heads over %d kv heads", s, h, c->h_kv);
    const int past_len = c->len, new_len = past_len + s;
    if (past_len + s > rope->max_seq)  // encoding.rs:62-68
        LUMEN_FAIL(LUMEN_ERR_ROPE_RANGE, "RoPE index out of range: offset %d + len %d > max %d", past_len, s, rope->max_seq);
    if (new_len > c->max_seq)  // self_attention.rs:341-346
        LUMEN_FAIL(LUMEN_ERR_KV_OVERFLOW, "KV cache overflow: new_len=%d > max_seq=%d", new_len, c->max_seq);
    if (s == 0) return LUMEN_OK;
    // rotated queries: scratch kept on the cache, grown (with a stream synchronisation) only when a call needs more
    const size_t q_floats = (size_t)c->b * s * h * c->d;
    if (q_floats > c->q_rot_floats) {
        HIP_TRY(hipStreamSynchronize(c->ctx->stream));
        hipFree(c->q_rot);
        c->q_rot = nullptr;
        c->q_rot_floats = 0;
        HIP_TRY(hipMalloc((void **)&c->q_rot, sizeof(float) * q_floats));
        c->q_rot_floats = q_floats;
    }
    float *q_rot = c->q_rot;
    AttnPrefillArgs a = {};
    a.q = q; a.k = k; a.v = v; a.out = out; a.k_cache = c->k; a.v_cache = c->v;
    a.cos_t = rope->cos_dev; a.sin_t = rope->sin_dev;
    a.b = c->b; a.s = s; a.hq = h; a.hkv = c->h_kv; a.d = c->d; a.max_seq = c->max_seq; a.past_len = past_len;
    a.q_stride = h * c->d; a.k_stride = c->h_kv * c->d; a.v_stride = c->h_kv * c->d;
    a.scale = scale; a.causal = causal; a.q_rot = q_rot;
    const int rc = launch_attn_prefill(c->ctx, a);
    if (rc == LUMEN_OK) c->len = new_len;
    return rc;
}

LUMEN_DEFINE_WARM(attention)
