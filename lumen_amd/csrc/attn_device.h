// Device-side building blocks of GQA attention over the static KV cache,
// shared by the decode and the row-loop prefill attention kernels.
// WAVES = wavefronts per workgroup (64 lanes each).
//
// Lane mapping: a K/V row of D floats is covered by LPR = D/4 lanes holding
// 16 bytes each, so one 64-lane load instruction fetches 64/LPR rows.  Every
// lane group keeps an online-softmax state (m, l, ctx) for all NREP query
// heads of the KV group: each K/V byte is read once and used NREP times from
// registers.
#pragma once

#include <hip/hip_runtime.h>
#include <cmath>

typedef float v4f __attribute__((ext_vector_type(4)));

template <int NREP>
struct AttnState {
    float m[NREP], l[NREP];
    v4f acc[NREP];
};

template <int NREP>
__device__ __forceinline__ void state_init(AttnState<NREP> &st) {
#pragma unroll
    for (int r = 0; r < NREP; ++r) {
        st.m[r] = -INFINITY;
        st.l[r] = 0.f;
        st.acc[r] = (v4f){0.f, 0.f, 0.f, 0.f};
    }
}

// exp2 on the hardware transcendental unit (v_exp_f32, ~1 ulp; exp2(-inf) = 0).  Scores are kept in
// log2 units (q is pre-multiplied by scale * log2(e)), so softmax needs no other exponential.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

#define LUMEN_LOG2E 1.4426950408889634f

// Sum over the LPR lanes that share a K/V row; every lane of the group gets the total.  Groups of
// 16 lanes are one DPP row: four rotate-and-add steps on the VALU, no LDS crossbar traffic.
template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
    if (LPR >= 16) {
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));  // row_ror:8
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));  // row_ror:4
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));  // row_ror:2
        v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));  // row_ror:1
#pragma unroll
        for (int off = 16; off < LPR; off <<= 1) v += __shfl_xor(v, off, 64);
    } else {
#pragma unroll
        for (int off = LPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    }
    return v;
}

// One K/V row piece per lane: score for each of the NREP heads, online-softmax update (the
// reference's branchy form, self_attention.rs:252-285, computes the same quantities).  q holds the
// rotated query times scale * log2(e).  Every lane of the wavefront must call it (it shuffles).
template <int D, int NREP>
__device__ __forceinline__ void attn_step(AttnState<NREP> &st, const v4f (&q)[NREP], const v4f kv, const v4f vv,
                                          bool valid) {
    constexpr int LPR = D / 4;
#pragma unroll
    for (int r = 0; r < NREP; ++r) {
        float s = q[r].x * kv.x;
        s = fmaf(q[r].y, kv.y, s);
        s = fmaf(q[r].z, kv.z, s);
        s = fmaf(q[r].w, kv.w, s);
        s = group_sum<LPR>(s);
        s = valid ? s : -INFINITY;
        const float m_new = fmaxf(st.m[r], s);
        if (m_new > -INFINITY) {
            const float alpha = fast_exp2(st.m[r] - m_new);  // exp2(-inf) = 0 on the first row
            const float p = fast_exp2(s - m_new);
            st.l[r] = fmaf(st.l[r], alpha, p);
            st.acc[r].x = fmaf(st.acc[r].x, alpha, p * vv.x);
            st.acc[r].y = fmaf(st.acc[r].y, alpha, p * vv.y);
            st.acc[r].z = fmaf(st.acc[r].z, alpha, p * vv.z);
            st.acc[r].w = fmaf(st.acc[r].w, alpha, p * vv.w);
            st.m[r] = m_new;
        }
    }
}

// UB rows per lane group at once for one query head: the UB scores first (independent dot products
// and lane-group sums), then ONE online-softmax update for the batch -- one rescale of the running
// state and one exponential per row, instead of two exponentials and a rescale per row.  Rows
// whose bit in `valid` is clear get the weight exp2(-inf) = 0 (their loads were clamped to a row
// inside the cache, so the values multiplied by that zero are finite).
template <int D, int UB>
__device__ __forceinline__ void attn_batch(AttnState<1> &st, const v4f &q, const v4f (&kv)[UB], const v4f (&vv)[UB],
                                           unsigned valid) {
    constexpr int LPR = D / 4;
    float s[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        float d = q.x * kv[u].x;
        d = fmaf(q.y, kv[u].y, d);
        d = fmaf(q.z, kv[u].z, d);
        d = fmaf(q.w, kv[u].w, d);
        s[u] = d;
    }
    float mb = -INFINITY;
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        s[u] = group_sum<LPR>(s[u]);
        s[u] = (valid >> u) & 1u ? s[u] : -INFINITY;
        mb = fmaxf(mb, s[u]);
    }
    // no branch around the update (the compiler would sink the V loads into it, behind the wait for
    // the K rows): while nothing valid has been seen, m_new = -inf and every weight below is
    // exp2(-inf - 0) = 0
    const float m_new = fmaxf(st.m[0], mb);
    const float m_ref = m_new > -INFINITY ? m_new : 0.f;
    const float alpha = fast_exp2(st.m[0] - m_ref);  // exp2(-inf) = 0 on the first batch
    float l = st.l[0] * alpha;
    v4f acc = st.acc[0];
    acc.x *= alpha; acc.y *= alpha; acc.z *= alpha; acc.w *= alpha;
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        const float p = fast_exp2(s[u] - m_ref);
        l += p;
        acc.x = fmaf(p, vv[u].x, acc.x);
        acc.y = fmaf(p, vv[u].y, acc.y);
        acc.z = fmaf(p, vv[u].z, acc.z);
        acc.w = fmaf(p, vv[u].w, acc.w);
    }
    st.l[0] = l;
    st.acc[0] = acc;
    st.m[0] = m_new;
}

template <int D, int WAVES>
struct AttnGeom {
    static constexpr int LPR = D / 4;            // lanes per row
    static constexpr int RPW = 64 / LPR;         // rows per wavefront load
    static constexpr int RPI = WAVES * RPW;      // rows per workgroup iteration
    static constexpr int U = 2;                  // iterations whose loads are in flight together
    static constexpr int ROWS_PER_TRIP = RPI * U;
};

// Rows [p0, p1) of one KV head (Kb/Vb point at row 0) spread over the
// workgroup's WAVES x (64/LPR) lane groups.
// One trip = ROWS_PER_TRIP rows starting at `base`: issue all of this lane's K/V loads ...
template <int D, int WAVES>
__device__ __forceinline__ void attn_load_trip(const float *__restrict__ Kb, const float *__restrict__ Vb, int base,
                                               int p1, v4f (&kv)[AttnGeom<D, WAVES>::U],
                                               v4f (&vv)[AttnGeom<D, WAVES>::U]) {
    typedef AttnGeom<D, WAVES> G;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int off = wave * G::RPW + lane / G::LPR, c = lane % G::LPR;
#pragma unroll
    for (int u = 0; u < G::U; ++u) {
        // unconditional loads (straight-line code keeps them all in flight): a row past the slice is
        // clamped to a row inside the cache and masked out in attn_step (weight exp(-inf) = 0)
        const int j = max(min(base + u * G::RPI + off, p1 - 1), 0);
        kv[u] = *(const v4f *)(Kb + (size_t)j * D + c * 4);
        vv[u] = *(const v4f *)(Vb + (size_t)j * D + c * 4);
    }
}

// ... and fold them into the running state.
template <int D, int NREP, int WAVES>
__device__ __forceinline__ void attn_compute_trip(AttnState<NREP> &st, const v4f (&q)[NREP],
                                                  const v4f (&kv)[AttnGeom<D, WAVES>::U],
                                                  const v4f (&vv)[AttnGeom<D, WAVES>::U], int base, int p1) {
    typedef AttnGeom<D, WAVES> G;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int off = wave * G::RPW + lane / G::LPR;
#pragma unroll
    for (int u = 0; u < G::U; ++u) {
        // uniform test: every lane of the wavefront takes the step (it shuffles), rows past p1 are masked
        if (base + u * G::RPI < p1) attn_step<D, NREP>(st, q, kv[u], vv[u], base + u * G::RPI + off < p1);
    }
}

template <int D, int NREP, int WAVES>
__device__ __forceinline__ void attn_rows(AttnState<NREP> &st, const v4f (&q)[NREP], const float *__restrict__ Kb,
                                          const float *__restrict__ Vb, int p0, int p1) {
    typedef AttnGeom<D, WAVES> G;
    for (int base = p0; base < p1; base += G::ROWS_PER_TRIP) {  // trip count is uniform over the workgroup
        v4f kv[G::U], vv[G::U];
        attn_load_trip<D, WAVES>(Kb, Vb, base, p1, kv, vv);
        attn_compute_trip<D, NREP, WAVES>(st, q, kv, vv, base, p1);
    }
}

// Merge the lane-group states of each wavefront and publish one state per
// wavefront in LDS (sm, sl [WAVES][NREP]; sacc [WAVES][NREP][D]).  The caller
// puts a workgroup barrier between this and wave_fold().
template <int D, int NREP>
__device__ __forceinline__ void wave_merge_publish(AttnState<NREP> &st, float *sm, float *sl, float *sacc) {
    constexpr int LPR = D / 4;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int slot = lane / LPR, c = lane % LPR;
#pragma unroll
    for (int r = 0; r < NREP; ++r) {
#pragma unroll
        for (int off = LPR; off < 64; off <<= 1) {
            const float mo = __shfl_xor(st.m[r], off, 64);
            const float lo = __shfl_xor(st.l[r], off, 64);
            v4f ao;
            ao.x = __shfl_xor(st.acc[r].x, off, 64);
            ao.y = __shfl_xor(st.acc[r].y, off, 64);
            ao.z = __shfl_xor(st.acc[r].z, off, 64);
            ao.w = __shfl_xor(st.acc[r].w, off, 64);
            const float mn = fmaxf(st.m[r], mo);
            const float a = (mn > -INFINITY) ? fast_exp2(st.m[r] - mn) : 0.f;
            const float b = (mn > -INFINITY) ? fast_exp2(mo - mn) : 0.f;
            st.l[r] = st.l[r] * a + lo * b;
            st.acc[r].x = st.acc[r].x * a + ao.x * b;
            st.acc[r].y = st.acc[r].y * a + ao.y * b;
            st.acc[r].z = st.acc[r].z * a + ao.z * b;
            st.acc[r].w = st.acc[r].w * a + ao.w * b;
            st.m[r] = mn;
        }
        if (slot == 0) {
            if (c == 0) {
                sm[wave * NREP + r] = st.m[r];
                sl[wave * NREP + r] = st.l[r];
            }
            *(v4f *)(sacc + ((size_t)(wave * NREP + r)) * D + c * 4) = st.acc[r];
        }
    }
}

// (max, sum, ctx) of head r, dim dd over the wavefront states in LDS
template <int D, int NREP, int WAVES>
__device__ __forceinline__ void wave_fold(const float *sm, const float *sl, const float *sacc, int r, int dd,
                                          float &mm, float &ls, float &cx) {
    mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, sm[w * NREP + r]);
    ls = 0.f;
    cx = 0.f;
    if (mm > -INFINITY) {
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float ex = fast_exp2(sm[w * NREP + r] - mm);
            ls = fmaf(sl[w * NREP + r], ex, ls);
            cx = fmaf(sacc[((size_t)(w * NREP + r)) * D + dd], ex, cx);
        }
    }
}

// This lane's 16-byte piece of each rotated query head, times scale * log2(e)
template <int D, int NREP>
__device__ __forceinline__ void load_q_scaled(v4f (&q)[NREP], const float *q_rot, int c, float scale) {
    const float f = scale * LUMEN_LOG2E;
#pragma unroll
    for (int r = 0; r < NREP; ++r) {
        q[r] = *(const v4f *)(q_rot + r * D + c * 4);
        q[r].x *= f; q[r].y *= f; q[r].z *= f; q[r].w *= f;
    }
}

// Optional per-head RMSNorm (gain g) then half-split RoPE of nh contiguous
// heads held raw in LDS `raw` ([nh][D]) into `rot`.  cs/sn: table rows at the
// token's position.  q: (x1*c - x2*s, x1*s + x2*c), self_attention.rs:220-227;
// k: same values, encoding.rs:196-203.
template <int D>
__device__ __forceinline__ void norm_rope_heads(const float *raw, float *rot, int nh, const float *__restrict__ cs,
                                                const float *__restrict__ sn, const float *__restrict__ g,
                                                float eps, int nthreads) {
    constexpr int HALF = D / 2;
    for (int p = threadIdx.x; p < nh * HALF; p += nthreads) {
        const int r = p / HALF, j = p % HALF;
        float x1 = raw[r * D + j], x2 = raw[r * D + j + HALF];
        if (g) {
            float ss = 0.f;
            for (int i = 0; i < D; ++i) ss = fmaf(raw[r * D + i], raw[r * D + i], ss);
            const float inv = 1.0f / sqrtf(ss / (float)D + eps);
            x1 = x1 * inv * g[j];
            x2 = x2 * inv * g[j + HALF];
        }
        const float c = cs[j], s = sn[j];
        {
#pragma clang fp contract(off)  // separate multiplies and add, like the reference's compiled code
            rot[r * D + j] = x1 * c - x2 * s;
            rot[r * D + j + HALF] = x1 * s + x2 * c;
        }
    }
}
