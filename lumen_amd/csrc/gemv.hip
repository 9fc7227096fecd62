// Memory-bound vector-matrix product y = W x for the M == 1 branch of
// ops::matmul::matmul (src/ops/matmul.rs:42-69), W [N, K] row-major f32 or
// bf16 bits, x and y f32, f32 accumulation.
//
// Mapping: x is staged once per workgroup in LDS (optionally RMS-normalised
// on the way in).  One 64-lane wavefront owns R whole rows at a time; each
// lane streams 16-byte pieces of the rows (a wavefront covers 1 KiB of a row
// per load instruction, fully coalesced), multiplies them with its slice of x
// from LDS and the 64 partial sums are folded with cross-lane shuffles.  A
// wavefront's rows are walked in pieces of 8 independent 16-byte loads per
// lane and two pieces are kept in flight (16 loads per lane).
#include "internal.h"
#include "wave_reduce.h"
#include "stage_times.h"

typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

#define GEMV_THREADS 256                  // default workgroup: 4 wavefronts
#define GEMV_WAVES (GEMV_THREADS / 64)
#define GEMV_MAX_WAVES 8                  // the launcher picks 4 to 8 wavefronts per workgroup

__device__ __forceinline__ float silu_f(float g) {
    // x * (1 / (1 + exp(-x))), src/layers/activation.rs:143-146
    float sig = 1.0f / (1.0f + expf(-g));
    return g * sig;
}

// 16 bytes of weights times the matching slice of x
template <bool BF16>
__device__ __forceinline__ float dot16(const v4u raw, const float *xs) {
    if (BF16) {
        // eight bf16 values; widening is a 16-bit shift (src/loader.rs:58)
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

// Stages x (optionally RMS-normalised: (x * inv_rms) * g, src/layers/norm/rms_norm.rs:45-58)
// into LDS, zero-padded to kpad.  x is read from memory once: the raw values go to LDS while the
// sum of squares is taken, then every thread scales the elements it staged itself.  All threads
// of the workgroup must call it.
template <int PRO, int XB>
__device__ __forceinline__ void stage_x(float *xs, const float *__restrict__ x, const float *__restrict__ g,
                                        float eps, int K, int kpad, int nwaves) {
    __shared__ float red[GEMV_MAX_WAVES];
    const int tid = threadIdx.x, nthreads = nwaves * 64;
    float ss = 0.f;
    // XB loads per thread are requested before the first one is waited for: taken one by one, each is a
    // trip to memory of its own (eleven in a row for K = 11008 with 256 threads).  The launcher asks for
    // XB = 4 where a thread has more than two pieces to stage; the registers this takes cost the
    // K = 2048 kernels more than the trips (gate|up 16.1 -> 16.8 us), so those keep XB = 1.
    
    for (int k0 = tid * 4; k0 < kpad; k0 += nthreads * 4 * XB) {
        v4f v[XB];
#pragma unroll
        for (int i = 0; i < XB; ++i) {
            const int k = k0 + i * nthreads * 4;
            v[i] = v4f{0.f, 0.f, 0.f, 0.f};
            if (k < K) v[i] = *(const v4f *)(x + k);
        }
#pragma unroll
        for (int i = 0; i < XB; ++i) {
            const int k = k0 + i * nthreads * 4;
            if (k < kpad) {
                ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
                *(v4f *)(xs + k) = v[i];
            }
        }
    }
    if (PRO == PRO_RMSNORM) {
        ss = wave_sum(ss);
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        float tot = 0.f;
        for (int w = 0; w < nwaves; ++w) tot += red[w];
        const float rms = sqrtf(tot / (float)K + eps);
        const float inv = 1.0f / rms;
        for (int k = tid * 4; k < K; k += nthreads * 4) {
            v4f v = *(const v4f *)(xs + k);
            const v4f gg = *(const v4f *)(g + k);
            v.x = v.x * inv * gg.x;
            v.y = v.y * inv * gg.y;
            v.z = v.z * inv * gg.z;
            v.w = v.w * inv * gg.w;
            *(v4f *)(xs + k) = v;
        }
    }
    __syncthreads();
}

// Latency-bound launches (every wavefront has a single unit whose loads all go out at once): the first
// GEMV_EARLY pieces of x of a thread -- and of the norm gains -- are requested BEFORE the weights.  Loads
// return in the order they were issued, so x queued behind the weights would arrive after them, and the
// staging, the sum of squares and the gains (two dependent trips more in the plain loop) would all sit
// between the arrival of the weights and the first multiply.  Requested first, they are staged while the
// weights are still on their way.
#define GEMV_EARLY 2
template <int PRO>
__device__ __forceinline__ void request_early(v4f (&xe)[GEMV_EARLY], v4f (&ge)[GEMV_EARLY], const float *__restrict__ x,
                                              const float *__restrict__ g, int K, int nthreads) {
#pragma unroll
    for (int i = 0; i < GEMV_EARLY; ++i) {
        const int k = ((int)threadIdx.x + i * nthreads) * 4;
        xe[i] = v4f{0.f, 0.f, 0.f, 0.f};
        ge[i] = v4f{0.f, 0.f, 0.f, 0.f};
        if (k < K) {
            xe[i] = *(const v4f *)(x + k);
            if (PRO == PRO_RMSNORM) ge[i] = *(const v4f *)(g + k);
        }
    }
}

// stage_x for a launch whose first GEMV_EARLY pieces per thread were requested by request_early; pieces
// beyond those (none for the shapes the launcher sends here) take the plain loops.
template <int PRO>
__device__ __forceinline__ void stage_x_early(float *xs, const float *__restrict__ x, const float *__restrict__ g,
                                              float eps, int K, int kpad, int nwaves, const v4f (&xe)[GEMV_EARLY],
                                              const v4f (&ge)[GEMV_EARLY]) {
    __shared__ float red_e[GEMV_MAX_WAVES];
    const int tid = threadIdx.x, nthreads = nwaves * 64;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < GEMV_EARLY; ++i) {
        const int k = (tid + i * nthreads) * 4;
        if (k < kpad) {
            ss += xe[i].x * xe[i].x + xe[i].y * xe[i].y + xe[i].z * xe[i].z + xe[i].w * xe[i].w;
            if (PRO != PRO_RMSNORM) *(v4f *)(xs + k) = xe[i];
        }
    }
    for (int k = (tid + GEMV_EARLY * nthreads) * 4; k < kpad; k += nthreads * 4) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        if (k < K) v = *(const v4f *)(x + k);
        ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        *(v4f *)(xs + k) = v;
    }
    if (PRO == PRO_RMSNORM) {
        // the early pieces stay in registers until the sum of squares is known and go to LDS scaled
        ss = wave_sum(ss);
        if ((tid & 63) == 0) red_e[tid >> 6] = ss;
        __syncthreads();
        float tot = 0.f;
        for (int w = 0; w < nwaves; ++w) tot += red_e[w];
        const float rms = sqrtf(tot / (float)K + eps);
        const float inv = 1.0f / rms;
#pragma unroll
        for (int i = 0; i < GEMV_EARLY; ++i) {
            const int k = (tid + i * nthreads) * 4;
            if (k < kpad) {
                v4f v = xe[i];
                v.x = v.x * inv * ge[i].x;
                v.y = v.y * inv * ge[i].y;
                v.z = v.z * inv * ge[i].z;
                v.w = v.w * inv * ge[i].w;
                *(v4f *)(xs + k) = v;
            }
        }
        for (int k = (tid + GEMV_EARLY * nthreads) * 4; k < K; k += nthreads * 4) {
            v4f v = *(const v4f *)(xs + k);
            const v4f gg = *(const v4f *)(g + k);
            v.x = v.x * inv * gg.x;
            v.y = v.y * inv * gg.y;
            v.z = v.z * inv * gg.z;
            v.w = v.w * inv * gg.w;
            *(v4f *)(xs + k) = v;
        }
    }
    __syncthreads();
}

// Stages the decode attention output from the attention kernel's partial states: head h, element d is
// sum_s w_s ctx_s[d] / (sum_s w_s l_s + 1e-9) with w_s = exp2(m_s - max m) over the slices in use
// (self_attention.rs:287-290 after the merge of the slices' online-softmax states).  A thread's loads
// are independent of each other: one trip to memory after the position is known.  Slices not in use
// hold whatever an earlier step left there: they are never read (the index is clamped to the last one
// in use and its weight forced to zero).  All threads of the workgroup must call it.
typedef float v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void stage_attn_fold(float *xs, const GemvArgs &a, int K, int kpad, int nwaves) {
    const int tid = threadIdx.x, nthreads = nwaves * 64;
    const int D = a.attn_d, S = a.attn_nslices, stride = D + 2;
    const int rows = *a.attn_pos + 1;
    int nact = 1;
    if (rows > a.attn_short_rows) nact = min(S, (rows + a.attn_trip - 1) / a.attn_trip);
    for (int k = tid * 4; k < kpad; k += nthreads * 4) {
        v4f v = {0.f, 0.f, 0.f, 0.f};
        if (k < K) {
            const float *ph = a.attn_part + (size_t)(k / D) * S * stride;
            const int d = k % D;
            float m[GEMV_FOLD_MAX_SLICES], l[GEMV_FOLD_MAX_SLICES];
            v2f c0[GEMV_FOLD_MAX_SLICES], c1[GEMV_FOLD_MAX_SLICES];
#pragma unroll
            for (int s = 0; s < GEMV_FOLD_MAX_SLICES; ++s) {
                const float *pp = ph + (size_t)min(s, nact - 1) * stride;
                m[s] = pp[D];
                l[s] = pp[D + 1];
                c0[s] = *(const v2f *)(pp + d);  // rows of D + 2 floats: 8-byte aligned
                c1[s] = *(const v2f *)(pp + d + 2);
            }
            float M = -INFINITY;
#pragma unroll
            for (int s = 0; s < GEMV_FOLD_MAX_SLICES; ++s)
                if (s < nact) M = fmaxf(M, m[s]);
            float L = 0.f;
#pragma unroll
            for (int s = 0; s < GEMV_FOLD_MAX_SLICES; ++s) {
                const float w = (s < nact && m[s] > -INFINITY) ? __builtin_amdgcn_exp2f(m[s] - M) : 0.f;
                L = fmaf(l[s], w, L);
                v.x = fmaf(c0[s].x, w, v.x);
                v.y = fmaf(c0[s].y, w, v.y);
                v.z = fmaf(c1[s].x, w, v.z);
                v.w = fmaf(c1[s].y, w, v.w);
            }
            const float inv = 1.0f / (L + 1e-9f);
            v.x *= inv; v.y *= inv; v.z *= inv; v.w *= inv;
        }
        *(v4f *)(xs + k) = v;
    }
    __syncthreads();
}

template <bool BF16, int R, int PRO, int EPI, int XB, bool KA>
__global__ __launch_bounds__(GEMV_MAX_WAVES * 64) void gemv_kernel(const void *W_hot, const float *x_hot,
                                                                  const float *norm_w_hot, const int *row_sel_hot,
                                                                  int N_hot, int K_hot, int D_hot, int nblocks,
                                                                  int nwaves, GemvArgs a) {
    // The leading scalar arguments repeat what the first loads need (a.W, a.x, a.norm_w, a.row_sel, a.N,
    // a.K, a.D, the grid and workgroup size): the file is compiled with kernel-argument preloading, so they
    // are in scalar registers when a wavefront starts and its first loads do not wait for a read of the
    // argument block.  XB: how x is staged -- 1 piece at a time, 4 at a time, or 0: requested ahead of the
    // weights (request_early).
    LUMEN_DYNAMIC_LDS(float, xs);
    constexpr int VEC = BF16 ? 8 : 4;          // elements per 16-byte load
    constexpr int SWEEP = 64 * VEC;            // elements one wavefront covers per load
    constexpr int U = 8 / R;                   // loads in flight per lane per row
    constexpr int PIECE = SWEEP * U;           // elements of a row one piece covers
    constexpr int ESZ = BF16 ? 2 : 4;
    const int K = K_hot, N = N_hot, D = D_hot;
    const int kpad = (K + PIECE - 1) / PIECE * PIECE;  // xs is zero from K to kpad

    STAGE_T(0);
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * nwaves + (threadIdx.x >> 6);
    const int nw = nblocks * nwaves;
    const int nunits = (N + R - 1) / R;
    const char *Wb = (const char *)W_hot;
    const size_t row_bytes = (size_t)K * ESZ;
    const int half_d = D >> 1;

    // row r of unit u: consecutive rows, or the RoPE pair (j, j + D/2) of one head
    auto unit_row = [&](int u, int r) {
        if (EPI == EPI_ROPE_QKV) return (u / half_d) * D + (u % half_d) + r * half_d;
        return u * R + r;
    };

    // 8 x 16 bytes per lane of unit u from element k0 on.  Every load is issued unconditionally:
    // positions past the end of the row are clamped to its last 16 bytes (they meet the zero
    // padding of xs), a row past N to row N-1 (discarded in the epilogue).
    auto load_piece = [&](int u, int k0, v4u (&raw)[R][U]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = min(unit_row(u, r), N - 1);
            const char *rp = Wb + (size_t)row * row_bytes;
#pragma unroll
            for (int uu = 0; uu < U; ++uu) {
                // KA: K is a whole number of pieces, no position lies past the end of the row -- the eight
                // addresses are then one base plus constant offsets
                const int kk = KA ? k0 + uu * SWEEP + lane * VEC : min(k0 + uu * SWEEP + lane * VEC, K - VEC);
                raw[r][uu] = __builtin_nontemporal_load((const v4u *)(rp + (size_t)kk * ESZ));
            }
        }
    };

    // A wavefront's work is a sequence of pieces: np pieces per unit, units gw, gw + nw, ...  Two
    // pieces (2 x 8 loads per lane) are kept in flight: while one is multiplied the next one is
    // already on its way and the one after is requested as soon as its registers are free.
    const int np = kpad / PIECE;
    int lu = gw, lk = 0;  // unit / element offset of the next piece to load
    auto advance_load = [&]() {
        lk += PIECE;
        if (lk >= kpad) {
            lk = 0;
            lu += nw;
        }
    };

    constexpr bool EARLY = XB == 0 && PRO != PRO_ATTN_FOLD;
    v4f xe[GEMV_EARLY], ge[GEMV_EARLY];
    // (with a row selector -- the first layer's gather -- the address of x needs a trip to memory itself:
    // then the weights go first)
    if (EARLY && !row_sel_hot) request_early<PRO>(xe, ge, x_hot, norm_w_hot, K, nwaves * 64);

    // the first weights of this wavefront start streaming before x is staged: they do not depend on it
    v4u rawA[R][U], rawB[R][U];
    load_piece(min(lu, nunits - 1), lk, rawA);
    advance_load();
    // a second piece exists: the unit has one, or the wavefront a second unit (the count of pieces, which
    // takes a division, is left until both requests are out)
    if ((kpad > PIECE && gw < nunits) || gw + nw < nunits) {
        load_piece(lu, lk, rawB);
        advance_load();
    }
    const int my_units = (nunits > gw) ? (nunits - gw + nw - 1) / nw : 0;
    const int T = my_units * np;

    long sel_off = 0;
    const float *xin = x_hot;
    if (row_sel_hot) {
        sel_off = (long)(*row_sel_hot) * a.row_stride;
        if (a.x_sel) xin += sel_off;
        if (EARLY) request_early<PRO>(xe, ge, xin, norm_w_hot, K, nwaves * 64);
    }
    const float *residual = a.residual + (a.residual_sel ? sel_off : 0);
    // What a unit's epilogue needs from memory is requested a unit ahead -- the first one here,
    // before x is staged -- so that no load sits between the last multiply and the store:
    // cos / sin of the unit's RoPE pair, or the residual of its rows.
    const int pos = (EPI == EPI_ROPE_QKV) ? *a.pos : 0;
    float pre0 = 0.f, pre1 = 0.f;
    auto preload = [&](int un) {
        if (EPI == EPI_ROPE_QKV && un < nunits) {
            const int j = un % half_d;
            pre0 = a.cos_t[(size_t)pos * D + j];
            pre1 = a.sin_t[(size_t)pos * D + j];
        }
        if (EPI == EPI_RESIDUAL) {
            if (un * R < N) pre0 = residual[un * R];
            if (R == 2 && un * R + 1 < N) pre1 = residual[un * R + 1];
        }
    };
    preload(gw);
    STAGE_T(1);
    if (PRO == PRO_ATTN_FOLD) stage_attn_fold(xs, a, K, kpad, nwaves);
    else if (EARLY) stage_x_early<PRO>(xs, xin, norm_w_hot, a.eps, K, kpad, nwaves, xe, ge);
    else stage_x<PRO, (XB > 0 ? XB : 1)>(xs, xin, norm_w_hot, a.eps, K, kpad, nwaves);
    STAGE_T(2);
    float best = -INFINITY;
    int best_idx = 0xffffff;  // (rows are below 2^24: the launcher checks)

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;
    int u = gw, k0 = 0;  // unit / element offset of the piece being multiplied
    auto consume = [&](const v4u (&raw)[R][U]) {
#pragma unroll
        for (int uu = 0; uu < U; ++uu) {
            const float *xp = xs + k0 + uu * SWEEP + lane * VEC;
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] += dot16<BF16>(raw[r][uu], xp);
        }
        k0 += PIECE;
        if (k0 >= kpad) {  // unit complete
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
            if (EPI == EPI_ARGMAX) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int row = u * R + r;
                    if (row < N && (acc[r] > best || (acc[r] == best && row < best_idx))) {
                        best = acc[r];
                        best_idx = row;
                    }
                }
            }
            if (lane == 0) {
                if (EPI == EPI_SWIGLU) {
                    // rows (2u, 2u+1) hold (gate_u, up_u): silu(gate) * up, src/models/llama.rs:60-63
                    a.y[u] = silu_f(acc[0]) * acc[R - 1];
                } else if (EPI == EPI_ROPE_QKV) {
                    // half-split rotation at the token's position (src/layers/attention/encoding.rs:196-203,
                    // self_attention.rs:220-227); k and v land in cache row pos (self_attention.rs:161-176)
                    const int head = u / half_d, j = u % half_d;
                    const float c = pre0, sn = pre1;
                    const float x1 = acc[0], x2 = acc[R - 1];
                    float o1, o2;
                    {
#pragma clang fp contract(off)
                        o1 = x1 * c - x2 * sn;
                        o2 = x1 * sn + x2 * c;
                    }
                    if (head < a.hq) {
                        a.y[head * D + j] = o1;
                        a.y[head * D + j + half_d] = o2;
                    } else if (head < a.hq + a.hkv) {
                        float *dst = a.k_cache + ((size_t)(head - a.hq) * a.max_seq + pos) * D;
                        dst[j] = o1;
                        dst[j + half_d] = o2;
                    } else {
                        float *dst = a.v_cache + ((size_t)(head - a.hq - a.hkv) * a.max_seq + pos) * D;
                        dst[j] = x1;
                        dst[j + half_d] = x2;
                    }
                } else {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const int row = u * R + r;
                        if (row < N) {
                            // residual: x + y, src/ops/arithmetic.rs:48-51 via src/models/llama.rs:110,115
                            a.y[row] = (EPI == EPI_RESIDUAL) ? (r == 0 ? pre0 : pre1) + acc[r] : acc[r];
                        }
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = 0.f;
            k0 = 0;
            u += nw;
            preload(u);
        }
    };
    for (int t = 0; t < T; t += 2) {
        consume(rawA);
        if (t == 0) STAGE_T(3);
        if (t + 2 < T) {
            load_piece(lu, lk, rawA);
            advance_load();
        }
        if (t + 1 < T) {
            consume(rawB);
            if (t + 3 < T) {
                load_piece(lu, lk, rawB);
                advance_load();
            }
        }
    }

    STAGE_T(4);
    STAGE_T_STORES_DONE(5);
    if (EPI == EPI_ARGMAX) {
        // Greedy pick fused into the lm_head product.  Every workgroup leaves its candidate as ONE 8-byte word
        // {value bits, tag << 24 | row}, stored with a single agent-scope atomic store; the workgroup with the highest
        // index -- dispatched last, so every other one is resident or finished when it starts to wait -- polls the
        // words of all workgroups until each carries this launch's tag, and folds them (lowest row wins ties).
        // Value, row and tag are one atomic object: a reader that sees the tag has the candidate, whatever the order
        // of other accesses (no counter, no fence).  The tag is 1 + (*epoch mod 255); every workgroup writes its word
        // in every launch and the folding workgroup advances *epoch when it is done, so a word left by the launch
        // before never carries the tag of this one.  The wait is bounded: after spin_limit polls the workgroup flags
        // the failure in *err_dev, folds what it has and exits.
        __shared__ float am_v[GEMV_MAX_WAVES];
        __shared__ int am_i[GEMV_MAX_WAVES];
        const int wave = threadIdx.x >> 6;
        const unsigned tag = 1u + *a.amax_epoch % 255u;
        if (lane == 0) {
            am_v[wave] = best;
            am_i[wave] = best_idx;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < nwaves; ++w)
                if (am_v[w] > best || (am_v[w] == best && am_i[w] < best_idx)) {
                    best = am_v[w];
                    best_idx = am_i[w];
                }
            // (a workgroup without a row, or with NaNs only, leaves the row 0xffffff: never picked)
            const unsigned long long word = ((unsigned long long)((tag << 24) | ((unsigned)best_idx & 0xffffffu)) << 32) |
                                            (unsigned long long)__float_as_uint(best);
            __hip_atomic_store(a.amax_word + blockIdx.x, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if ((int)blockIdx.x != nblocks - 1) return;
        float bv = -INFINITY;
        int bi = 0xffffff;
        bool gave_up = false;
        for (int i = threadIdx.x; i < nblocks; i += nwaves * 64) {
            unsigned long long w;
            unsigned spins = 0;
            for (;;) {
                w = __hip_atomic_load(a.amax_word + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((unsigned)(w >> 56) == tag) break;
                if (++spins > a.spin_limit) {  // never in a healthy launch
                    gave_up = true;
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
            if ((unsigned)(w >> 56) != tag) continue;
            const float v = __uint_as_float((unsigned)w);
            const int ix = (int)((unsigned)(w >> 32) & 0xffffffu);
            if (v > bv || (v == bv && ix < bi)) {
                bv = v;
                bi = ix;
            }
        }
        if (gave_up) __hip_atomic_store(a.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (ov > bv || (ov == bv && oi < bi)) {
                bv = ov;
                bi = oi;
            }
        }
        __syncthreads();
        if (lane == 0) {
            am_v[wave] = bv;
            am_i[wave] = bi;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < nwaves; ++w)
                if (am_v[w] > bv || (am_v[w] == bv && am_i[w] < bi)) {
                    bv = am_v[w];
                    bi = am_i[w];
                }
            if (bi >= N) bi = 0;  // all NaN: index 0 like a sequential scan
            *a.tok_out = bi;
            if (a.pos_inc) {
                const int pos = *a.pos_inc;
                if (a.tok_hist) a.tok_hist[pos + 1] = bi;  // the pick is the token of the next position
                *a.pos_inc = pos + 1;
            }
            if (a.step_inc) *a.step_inc += 1;
            *a.amax_epoch += 1;
        }
    }
}

// Any K, any alignment: one wavefront per row, scalar loads, x from global memory.
template <bool BF16>
__global__ __launch_bounds__(GEMV_THREADS) void gemv_generic_kernel(GemvArgs a) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * GEMV_WAVES + (threadIdx.x >> 6);
    const int nw = gridDim.x * GEMV_WAVES;
    for (int row = gw; row < a.N; row += nw) {
        float acc = 0.f;
        for (int k = lane; k < a.K; k += 64) {
            float w;
            if (BF16)
                w = __uint_as_float((unsigned int)((const uint16_t *)a.W)[(size_t)row * a.K + k] << 16);
            else
                w = ((const float *)a.W)[(size_t)row * a.K + k];
            acc = fmaf(w, a.x[k], acc);
        }
        acc = wave_sum(acc);
        if (lane == 0) a.y[row] = acc;
    }
}

template <bool BF16, int R, int PRO, int XB, bool KA>
static void launch_epi(const GemvArgs &a, dim3 grid, int threads, size_t lds, hipStream_t s) {
    switch (a.epi) {
        case EPI_STORE:
            hipLaunchKernelGGL((gemv_kernel<BF16, R, PRO, EPI_STORE, XB, KA>), grid, dim3(threads), lds, s, a.W, a.x, a.norm_w, a.row_sel, a.N, a.K, a.D, (int)grid.x, threads >> 6, a);
            break;
        case EPI_RESIDUAL:
            hipLaunchKernelGGL((gemv_kernel<BF16, R, PRO, EPI_RESIDUAL, XB, KA>), grid, dim3(threads), lds, s, a.W, a.x, a.norm_w, a.row_sel, a.N, a.K, a.D, (int)grid.x, threads >> 6, a);
            break;
        case EPI_ARGMAX:
            hipLaunchKernelGGL((gemv_kernel<BF16, R, PRO, EPI_ARGMAX, XB, KA>), grid, dim3(threads), lds, s, a.W, a.x, a.norm_w, a.row_sel, a.N, a.K, a.D, (int)grid.x, threads >> 6, a);
            break;
        case EPI_ROPE_QKV:
            hipLaunchKernelGGL((gemv_kernel<BF16, 2, PRO, EPI_ROPE_QKV, XB, KA>), grid, dim3(threads), lds, s, a.W, a.x, a.norm_w, a.row_sel, a.N, a.K, a.D, (int)grid.x, threads >> 6, a);
            break;
        default:
            hipLaunchKernelGGL((gemv_kernel<BF16, 2, PRO, EPI_SWIGLU, XB, KA>), grid, dim3(threads), lds, s, a.W, a.x, a.norm_w, a.row_sel, a.N, a.K, a.D, (int)grid.x, threads >> 6, a);
            break;
    }
}

template <bool BF16, int R, int XB, bool KA>
static void launch_pro(const GemvArgs &a, dim3 grid, int threads, size_t lds, hipStream_t s) {
    if (a.pro == PRO_ATTN_FOLD)  // o_proj only (launch_gemv checks): one row per unit, residual epilogue
        hipLaunchKernelGGL((gemv_kernel<BF16, 1, PRO_ATTN_FOLD, EPI_RESIDUAL, XB, KA>), grid, dim3(threads), lds, s, a.W, a.x, a.norm_w, a.row_sel, a.N, a.K, a.D, (int)grid.x, threads >> 6, a);
    else if (a.pro == PRO_RMSNORM)
        launch_epi<BF16, R, PRO_RMSNORM, XB, KA>(a, grid, threads, lds, s);
    else
        launch_epi<BF16, R, PRO_NONE, XB, KA>(a, grid, threads, lds, s);
}

// Grid of the fused kernel for an [N, K] product: workgroups and threads per workgroup.
static int gemv_grid_cus(int num_cus, int N, int K, int w_bf16, int epi, int *threads_out) {
    const int vec = w_bf16 ? 8 : 4;
    const int R = (epi == EPI_SWIGLU || epi == EPI_ROPE_QKV || N >= 8192) ? 2 : 1;
    const int piece = 64 * vec * (8 / R);
    const int kpad = (K + piece - 1) / piece * piece;
    const size_t lds = (size_t)kpad * sizeof(float);
    const int nunits = (N + R - 1) / R;
    // Wavefronts per workgroup: when the units divide into exactly one workgroup of 5 to 8 wavefronts
    // per compute unit, take that shape -- every compute unit gets the same share and stages x once
    // (q|k|v of a 2048-wide model: 1280 pairs = 256 x 5; its o_proj and down: 2048 rows = 256 x 8).
    int waves = GEMV_WAVES;
    if (nunits % num_cus == 0) {
        const int w = nunits / num_cus;
        if (w > GEMV_WAVES && w <= GEMV_MAX_WAVES) waves = w;
        else if (w > GEMV_MAX_WAVES && w % GEMV_MAX_WAVES == 0) waves = GEMV_MAX_WAVES;  // several units per wavefront, x staged once per compute unit
    }
    const int threads = waves * 64;
    int blocks = (nunits + waves - 1) / waves;
    // one wave of workgroups: at most 4 per compute unit, fewer when their staged x would not fit the
    // compute unit's 160 KiB of LDS side by side (a second, partial wave of workgroups costs more
    // than longer row loops: 4.0 -> 4.7 TB/s at K = 11008 with bf16 weights)
    int per_cu = (int)((size_t)(160 * 1024) / (lds + 256));
    const int max_per_cu = 16 / waves > 1 ? 16 / waves : 1;  // 16 wavefronts per compute unit
    if (per_cu > max_per_cu) per_cu = max_per_cu;
    if (per_cu < 1) per_cu = 1;
    const int cap = num_cus * per_cu;
    if (blocks > cap) {
        // every wavefront the same number of units: with the grid simply cut at the cap some wavefronts
        // would take one unit more than the others, and those late, dependent requests are the kernel's tail
        const int per_wave = (nunits + cap * waves - 1) / (cap * waves);
        blocks = (nunits + waves * per_wave - 1) / (waves * per_wave);
    }
    if (threads_out) *threads_out = threads;
    return blocks;
}

int gemv_grid(const lumen_ctx *ctx, int N, int K, int w_bf16, int epi, int *threads_out) {
    return gemv_grid_cus(ctx->num_cus, N, K, w_bf16, epi, threads_out);
}

GemvPick gemv_pick(int num_cus, int N, int K, int w_bf16, int pro, int epi, bool aligned) {
    GemvPick p = {};
    const int vec = w_bf16 ? 8 : 4;
    p.R = (epi == EPI_SWIGLU || epi == EPI_ROPE_QKV || N >= 8192) ? 2 : 1;
    const int piece = 64 * vec * (8 / p.R);  // x is staged zero-padded to whole pieces
    const int kpad = (K + piece - 1) / piece * piece;
    p.lds = (size_t)kpad * sizeof(float);
    p.fast = (K % vec == 0) && aligned && p.lds <= 64 * 1024;
    p.pro = pro;
    p.epi = pro == PRO_ATTN_FOLD ? (int)EPI_RESIDUAL : epi;
    if (!p.fast) {
        p.threads = GEMV_THREADS;
        p.blocks = (N + GEMV_WAVES - 1) / GEMV_WAVES;
        if (p.blocks > num_cus * 8) p.blocks = num_cus * 8;
        return p;
    }
    p.blocks = gemv_grid_cus(num_cus, N, K, w_bf16, epi, &p.threads);
    // How x is staged (see stage_x, request_early): ahead of the weights where every wavefront has a
    // single unit of at most two pieces -- all of its loads go out at once and the prologue is what the
    // multiplies wait for -- and a thread stages at most GEMV_EARLY pieces; else in the loop, four pieces
    // at a time from three pieces per thread on.
    const int x_pieces = (kpad + p.threads * 4 - 1) / (p.threads * 4);
    const int nunits = (N + p.R - 1) / p.R;
    const bool early_x = pro != PRO_ATTN_FOLD && x_pieces <= GEMV_EARLY && kpad / piece <= 2 &&
                         nunits <= p.blocks * (p.threads / 64);
    p.xb = early_x ? 0 : x_pieces > 2 ? 4 : 1;
    p.ka = K % piece == 0;  // whole pieces: no clamped load positions
    return p;
}

int gemv_kernel_name(const GemvPick &p, int w_bf16, char *buf, int buf_len) {
    if (!p.fast) return snprintf(buf, buf_len, "gemv_generic_kernel<%s>", w_bf16 ? "true" : "false");
    return snprintf(buf, buf_len, "gemv_kernel<%s, %d, %d, %d, %d, %s>", w_bf16 ? "true" : "false", p.R, p.pro, p.epi, p.xb,
                    p.ka ? "true" : "false");
}

int gemv_max_blocks(const lumen_ctx *ctx) { return ctx->num_cus * 4; }

int launch_gemv(lumen_ctx *ctx, const GemvArgs &a) {
    if (a.N <= 0 || a.K <= 0) return LUMEN_OK;
    const int vec = a.w_bf16 ? 8 : 4;
    const bool aligned = (((uintptr_t)a.W | (uintptr_t)a.x) & 15) == 0 && (((uintptr_t)a.attn_part) & 7) == 0 &&
                         (a.pro != PRO_RMSNORM || ((uintptr_t)a.norm_w & 15) == 0);
    const GemvPick p = gemv_pick(ctx->num_cus, a.N, a.K, a.w_bf16, a.pro, a.epi, aligned);
    if (ctx->note_kernels) gemv_kernel_name(p, a.w_bf16, ctx->last_kernel, sizeof ctx->last_kernel);
    if (!p.fast) {
        if (a.pro != PRO_NONE || a.epi != EPI_STORE || a.row_sel)
            LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "fused GEMV needs K %% %d == 0, 16-byte alignment and K <= %d (K=%d)", vec,
                       16384, a.K);
        if (a.w_bf16)
            hipLaunchKernelGGL(gemv_generic_kernel<true>, dim3(p.blocks), dim3(p.threads), 0, ctx->stream, a);
        else
            hipLaunchKernelGGL(gemv_generic_kernel<false>, dim3(p.blocks), dim3(p.threads), 0, ctx->stream, a);
        LUMEN_CHECK_LAUNCH();
        return LUMEN_OK;
    }
    if (a.pro == PRO_ATTN_FOLD) {
        if (a.epi != EPI_RESIDUAL || p.R != 1 || !a.attn_part || !a.attn_pos || a.attn_d <= 0 || a.attn_d % 4 ||
            a.K % a.attn_d || a.attn_nslices < 1 || a.attn_nslices > GEMV_FOLD_MAX_SLICES)
            LUMEN_FAIL(LUMEN_ERR_INVALID, "GEMV over attention partials: one row per unit, residual epilogue, at most %d slices (got %d)",
                       GEMV_FOLD_MAX_SLICES, a.attn_nslices);
    }
    if ((a.epi == EPI_SWIGLU || a.epi == EPI_ROPE_QKV) && (a.N & 1))
        LUMEN_FAIL(LUMEN_ERR_SHAPE, "paired-row epilogue needs an even row count, got %d", a.N);
    if (a.epi == EPI_ARGMAX) {
        if (!a.amax_word || !a.amax_epoch || !a.err_dev || !a.tok_out || ((uintptr_t)a.amax_word & 7))
            LUMEN_FAIL(LUMEN_ERR_INVALID, "arg-max epilogue: needs a candidate buffer, a launch counter and an error flag");
        if (a.N >= (1 << 24))  // a candidate's row shares a word with its tag
            LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "arg-max epilogue: %d rows (at most %d)", a.N, (1 << 24) - 1);
        if (a.spin_limit > HANDOVER_MAX_SPINS) LUMEN_FAIL(LUMEN_ERR_INVALID, "arg-max epilogue: poll limit %u", a.spin_limit);
    }
    const int threads = p.threads, blocks = p.blocks;
    const size_t lds = p.lds;
    dim3 grid(blocks);
#define LAUNCH_GEMV_K(BF, RR, KAV)                                                       \
    do {                                                                                 \
        if (p.xb == 0) launch_pro<BF, RR, 0, KAV>(a, grid, threads, lds, ctx->stream);      \
        else if (p.xb == 4) launch_pro<BF, RR, 4, KAV>(a, grid, threads, lds, ctx->stream); \
        else launch_pro<BF, RR, 1, KAV>(a, grid, threads, lds, ctx->stream);             \
    } while (0)
#define LAUNCH_GEMV(BF, RR)                  \
    do {                                     \
        if (p.ka) LAUNCH_GEMV_K(BF, RR, true); \
        else LAUNCH_GEMV_K(BF, RR, false);   \
    } while (0)
    if (a.w_bf16) {
        if (p.R == 2) LAUNCH_GEMV(true, 2);
        else LAUNCH_GEMV(true, 1);
    } else {
        if (p.R == 2) LAUNCH_GEMV(false, 2);
        else LAUNCH_GEMV(false, 1);
    }
#undef LAUNCH_GEMV
#undef LAUNCH_GEMV_K
    LUMEN_CHECK_LAUNCH();
    {
        char what[96];
        snprintf(what, sizeof what, "gemv N=%d K=%d pro=%d epi=%d threads=%d", a.N, a.K, a.pro, a.epi, threads);
        stage_times_report(ctx, what, blocks, "start, requests out, x staged, first piece done, rows done, stores acknowledged");
    }
    return LUMEN_OK;
}

// --------------------------------------------------------------------- C ABI
static int check_gemv(lumen_ctx *ctx, const void *W, const float *x, float *y, int N, int K) {
    if (!ctx || !W || !x || !y) LUMEN_FAIL(LUMEN_ERR_INVALID, "gemv: null argument");
    if (N < 0 || K < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "gemv: negative dimension N=%d K=%d", N, K);
    return LUMEN_OK;
}

extern "C" int lumen_gemv_f32(lumen_ctx *ctx, const float *W, const float *x, float *y, int N, int K) {
    LUMEN_TRY(check_gemv(ctx, W, x, y, N, K));
    GemvArgs a = {};
    a.W = W; a.x = x; a.y = y; a.N = N; a.K = K; a.w_bf16 = 0; a.pro = PRO_NONE; a.epi = EPI_STORE;
    return launch_gemv(ctx, a);
}

extern "C" int lumen_gemv_bf16w(lumen_ctx *ctx, const uint16_t *W, const float *x, float *y, int N, int K) {
    LUMEN_TRY(check_gemv(ctx, W, x, y, N, K));
    GemvArgs a = {};
    a.W = W; a.x = x; a.y = y; a.N = N; a.K = K; a.w_bf16 = 1; a.pro = PRO_NONE; a.epi = EPI_STORE;
    return launch_gemv(ctx, a);
}

// The fused forms the decode step is made of, as an operator: optional RMSNorm on the way in (x is read from memory
// once), the epilogue on the way out.
extern "C" int lumen_gemv_fused_f32(lumen_ctx *ctx, const void *W, int w_bf16, const float *x, float *y, int N, int K,
                                    const float *norm_w, float eps, int epilogue, const float *residual) {
    LUMEN_TRY(check_gemv(ctx, W, x, y, N, K));
    if (epilogue != LUMEN_GEMV_EPI_STORE && epilogue != LUMEN_GEMV_EPI_RESIDUAL && epilogue != LUMEN_GEMV_EPI_SWIGLU)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "gemv_fused: unknown epilogue %d", epilogue);
    if (epilogue == LUMEN_GEMV_EPI_RESIDUAL && !residual) LUMEN_FAIL(LUMEN_ERR_INVALID, "gemv_fused: residual epilogue without a residual");
    GemvArgs a = {};
    a.W = W; a.x = x; a.y = y; a.N = N; a.K = K; a.w_bf16 = w_bf16 ? 1 : 0;
    a.pro = norm_w ? PRO_RMSNORM : PRO_NONE; a.norm_w = norm_w; a.eps = eps;
    a.epi = epilogue == LUMEN_GEMV_EPI_RESIDUAL ? EPI_RESIDUAL : epilogue == LUMEN_GEMV_EPI_SWIGLU ? EPI_SWIGLU : EPI_STORE;
    a.residual = residual;
    return launch_gemv(ctx, a);
}

// out row 2i = a row i, out row 2i + 1 = b row i: the layout the SwiGLU epilogue wants of gate_proj / up_proj
extern "C" int lumen_interleave_rows(lumen_ctx *ctx, const void *a, const void *b, void *out, int rows, size_t row_bytes) {
    if (!ctx || !a || !b || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "interleave_rows: null argument");
    if (rows < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "interleave_rows: negative row count");
    if (rows == 0 || row_bytes == 0) return LUMEN_OK;
    HIP_TRY(hipMemcpy2DAsync(out, 2 * row_bytes, a, row_bytes, row_bytes, (size_t)rows, hipMemcpyDeviceToDevice, ctx->stream));
    HIP_TRY(hipMemcpy2DAsync((char *)out + row_bytes, 2 * row_bytes, b, row_bytes, row_bytes, (size_t)rows, hipMemcpyDeviceToDevice,
                             ctx->stream));
    return LUMEN_OK;
}

extern "C" int lumen_gemv_kernel_name(int num_cus, int N, int K, int w_bf16, int rmsnorm, int epilogue, char *buf, int buf_len) {
    if (!buf || buf_len <= 0 || num_cus <= 0 || N <= 0 || K <= 0) LUMEN_FAIL(LUMEN_ERR_INVALID, "gemv_kernel_name: bad argument");
    if (epilogue < LUMEN_GEMV_EPI_STORE || epilogue > LUMEN_GEMV_EPI_ROPE_QKV)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "gemv_kernel_name: unknown epilogue %d", epilogue);
    const GemvPick p = gemv_pick(num_cus, N, K, w_bf16, rmsnorm ? PRO_RMSNORM : PRO_NONE, epilogue, true);
    gemv_kernel_name(p, w_bf16, buf, buf_len);
    return LUMEN_OK;
}

extern "C" int lumen_matmul_f32(lumen_ctx *ctx, const float *A, const float *W, float *C, int M, int N, int K_a,
                                int K_w) {
    if (!ctx || !A || !W || !C) LUMEN_FAIL(LUMEN_ERR_INVALID, "matmul: null argument");
    if (K_a != K_w)  // src/ops/matmul.rs:33-38
        LUMEN_FAIL(LUMEN_ERR_SHAPE, "MatMul shape mismatch: a (K=%d) vs b (K=%d)", K_a, K_w);
    if (M < 0 || N < 0 || K_a < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "matmul: negative dimension");
    if (M == 1) return lumen_gemv_f32(ctx, W, A, C, N, K_a);  // src/ops/matmul.rs:42
    return lumen_gemm_f32(ctx, A, W, C, M, N, K_a);
}

// Measurement aid: `iters` GEMVs back to back on the ctx stream, cycling through `ncopies` weight
// matrices `stride_elems` apart so that every launch streams its weights from HBM rather than from
// the L2 / memory-side cache; returns the HIP-event time of the whole run.
extern "C" int lumen_gemv_bench(lumen_ctx *ctx, const void *W_base, size_t stride_elems, int ncopies, int w_bf16,
                                const float *x, float *y, int N, int K, int iters, float *ms_out) {
    if (!ctx || !W_base || !x || !y || !ms_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "gemv_bench: null argument");
    if (ncopies <= 0 || iters <= 0 || N <= 0 || K <= 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "gemv_bench: non-positive argument");
    const size_t esz = w_bf16 ? 2 : 4;
    GemvArgs a = {};
    a.x = x; a.y = y; a.N = N; a.K = K; a.w_bf16 = w_bf16; a.pro = PRO_NONE; a.epi = EPI_STORE;
    LUMEN_TRY(lumen_timer_start(ctx));
    for (int i = 0; i < iters; ++i) {
        a.W = (const char *)W_base + (size_t)(i % ncopies) * stride_elems * esz;
        LUMEN_TRY(launch_gemv(ctx, a));
    }
    return lumen_timer_stop(ctx, ms_out);
}

LUMEN_DEFINE_WARM(gemv)
