// Causal GQA attention for a prompt (S > 1) on the matrix cores:
// self_attention.rs:308-419 with gqa_attention_no_repeat_bshd_view (:519-641)
// and softmax_inplace_view (:643-678) -- scores = Q K^T * scale, mask
// j > past_len + i, softmax with divisor (sum + 1e-9), ctx = P V, output BSHD.
//
// The reference materialises the S x L score matrix per head; here a
// workgroup keeps 128 (position, query head) rows of one KV group in
// registers and walks the cached keys in tiles of 32 with an online softmax,
// so scores never leave the compute unit and every K/V tile read from the
// cache serves all n_rep heads of the group and 128 / n_rep positions at once.
//
// The products run on the bf16 matrix cores at f32 accuracy, as in the prompt-pass GEMM: an f32
// value is the exact sum of three bf16 values, a product the sum of the six part products whose
// orders add up to at most four, accumulated in f32 by v_mfma_f32_32x32x16_bf16 (for head_dim 64:
// 24 + 24 instructions of 8 passes per key tile and wavefront; the f32 instruction would take
// 32 + 32 of 16 passes).
//
// Per wavefront (32 rows) and key tile, everything transposed so that a lane owns one query row:
//   S^T = K Q^T       K from LDS ([part][key][element], split on its way in) is the A operand, Q
//                     (split once, in registers) the B operand; two accumulators take turns so
//                     that consecutive instructions do not wait.  A lane then holds 16 of the
//                     tile's 32 scores of ITS row, lane ^ 32 the other 16
//   softmax           row max and sum in the lane (one exchange with lane ^ 32 for the max, one at
//                     the very end for the sum); scores in log2 units (Q pre-multiplied by
//                     scale * log2 e), P = exp2(S - m)
//   O^T += V^T P^T    V is staged transposed ([part][element][key position]) as the A operand; the
//                     lane's 16 weights are the B operand as they stand (split in the lane), no
//                     trip through LDS; the rescale by alpha is a per-lane scalar
#include "internal.h"
#include "attn_device.h"

typedef float v16f __attribute__((ext_vector_type(16)));

#define FA_ROWS 128  // (position, head) rows per workgroup
#define FA_KEYS 32   // keys per tile
#define FA_THREADS 256

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

__device__ __forceinline__ unsigned fa_pack_hi(float odd, float even) {
    return __builtin_amdgcn_perm(__float_as_uint(odd), __float_as_uint(even), 0x07060302u);
}
// x[0..3] -> three parts of 4 bf16 (2 dwords each)
__device__ __forceinline__ void fa_split4(const v4f x, v2u (&part)[3]) {
    float r[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int p = 0; p < 3; ++p) {
        part[p].x = fa_pack_hi(r[1], r[0]);
        part[p].y = fa_pack_hi(r[3], r[2]);
        if (p < 2) {
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] -= __uint_as_float(__float_as_uint(r[e]) & 0xffff0000u);
        }
    }
}
// KT: key tiles of 32 per trip of the loop (2 for head_dim 64: one barrier pair, one row maximum and one rescale of
// O per 64 keys; 1 for head_dim 128, whose K and V tiles fill LDS twice as fast).
template <int D, int NREP, int KT>
__global__ __launch_bounds__(FA_THREADS, (D == 64 ? 2 : 1)) void attn_prefill_bf16x3_kernel(AttnPrefillArgs a) {
    constexpr int BQ = FA_ROWS / NREP;  // positions per workgroup
    constexpr int KEYS = FA_KEYS * KT;   // keys per trip
    constexpr int DT = D / 32;          // 32-wide tiles of the head dimension
    constexpr int PIECES = D * KEYS / 4 / FA_THREADS;  // 16-byte pieces of a K (or V) tile per thread
    // rows of 4 words more than a multiple of 32: the 16-byte reads of 8 neighbouring rows hit distinct banks
    constexpr int LDK = D + 8, LDV = KEYS + 8;
    __shared__ __align__(16) uint16_t Ks[3][KEYS][LDK];  // [part][key][element]
    __shared__ __align__(16) uint16_t Vt[3][D][LDV];        // [part][element][key position]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 31, half = lane >> 5;
    // workgroups are dealt in index order: the blocks of late positions (most keys) go first
    const int q0 = (int)(gridDim.x - 1 - blockIdx.x) * BQ, hk = blockIdx.y, bb = blockIdx.z;
    const int L = a.past_len + a.s;
    const size_t head_base = ((size_t)bb * a.hkv + hk / a.kv_div) * a.max_seq * D;  // kv_div > 1: grid row = query head
    const float *Kc = a.k_cache + head_base, *Vc = a.v_cache + head_base;

    // This lane's query row (the COLUMN it owns in S^T and O^T): (position, head) row wave * 32 + c of the workgroup
    const int my_row = wave * 32 + c;
    const int my_i = min(q0 + my_row / NREP, a.s - 1);  // clamped: rows past S are computed and dropped
    const int my_pos = a.past_len + q0 + my_row / NREP;  // absolute position: keys up to it are visible
    const float *qrow = a.q_rot + (((size_t)bb * a.s + my_i) * a.hq + (size_t)hk * NREP + my_row % NREP) * D;
    const float qf_scale = a.scale * LUMEN_LOG2E;
    // Q as the B operand of S^T = K Q^T: lane (column c, half g) holds elements ks * 16 + g * 8 .. + 7 of its row
    v4u qp[D / 16][3];
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks) {
        v2u lo[3], hi[3];
        v4f x = *(const v4f *)(qrow + ks * 16 + half * 8);
        x.x *= qf_scale; x.y *= qf_scale; x.z *= qf_scale; x.w *= qf_scale;
        fa_split4(x, lo);
        x = *(const v4f *)(qrow + ks * 16 + half * 8 + 4);
        x.x *= qf_scale; x.y *= qf_scale; x.z *= qf_scale; x.w *= qf_scale;
        fa_split4(x, hi);
#pragma unroll
        for (int p = 0; p < 3; ++p) qp[ks][p] = (v4u){lo[p].x, lo[p].y, hi[p].x, hi[p].y};
    }

    const int q_last = min(q0 + BQ, a.s) - 1;
    const int kmax = a.causal ? min(L, a.past_len + q_last + 1) : L;
    const int wave_i_last = min(q0 + (wave * 32 + 31) / NREP, a.s - 1);
    const int wave_kmax = a.causal ? min(L, a.past_len + wave_i_last + 1) : L;
    // keys [0, wave_kfull) are visible to every row of this wavefront: no mask needed below it
    const int wave_kfull = a.causal ? min(L, a.past_len + q0 + (wave * 32) / NREP + 1) : L;

    // O^T: register r of tile t belongs to element 32 t + 8 (r / 4) + 4 half + r % 4 of this lane's row
    v16f O[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) O[t][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;  // of this lane's row; l over this lane's half of the keys

    // V^T is staged with bits 2 and 3 of the key index exchanged: the 8 keys a lane holds of S^T (4 + 4,
    // eight apart) then sit next to each other for the 16-byte operand read.  A thread takes 4 elements
    // (v_k4 ..) of the 4 keys that land on positions 4 v_g .. 4 v_g + 3 -- consecutive keys from v_key on --
    // so that one element of the four keys is one 8-byte LDS write.
    static_assert(PIECES == 4, "a thread stages four keys of V");
    constexpr int NG = KEYS / 4;  // groups of four key positions
    const int v_g = (tid >> 2) % NG, v_k4 = ((tid / (4 * NG)) * 4 + (tid & 3)) * 4;
    const int v_key = 4 * ((v_g & ~3) | ((v_g & 1) << 1) | ((v_g >> 1) & 1));
    v4f kreg[PIECES], vreg[PIECES];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int idx = tid + p * FA_THREADS;
            const int key = idx / (D / 4), k4 = (idx % (D / 4)) * 4;
            const int j = min(j0 + key, L - 1);  // keys past L are masked below
            kreg[p] = *(const v4f *)(Kc + (size_t)j * D + k4);
            vreg[p] = *(const v4f *)(Vc + (size_t)min(j0 + v_key + p, L - 1) * D + v_k4);
        }
    };

    constexpr int PA_[6] = {2, 0, 1, 1, 0, 0}, PB_[6] = {0, 2, 1, 0, 1, 0};  // part products by ascending size
    if (kmax > 0) fetch(0);
    for (int j0 = 0; j0 < kmax; j0 += KEYS) {
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int idx = tid + p * FA_THREADS;
            const int key = idx / (D / 4), k4 = (idx % (D / 4)) * 4;
            v2u kp[3];
            fa_split4(kreg[p], kp);
#pragma unroll
            for (int q = 0; q < 3; ++q) *(v2u *)&Ks[q][key][k4] = kp[q];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v2u vp[3];
            fa_split4((v4f){vreg[0][e], vreg[1][e], vreg[2][e], vreg[3][e]}, vp);
#pragma unroll
            for (int q = 0; q < 3; ++q) *(v2u *)&Vt[q][v_k4 + e][4 * v_g] = vp[q];
        }
        __syncthreads();
        if (j0 + KEYS < kmax) fetch(j0 + KEYS);  // in flight during the matrix instructions below

        if (j0 < wave_kmax) {  // uniform per wavefront: tiles wholly above the causal diagonal are skipped
            // S^T = K Q^T: register r of tile kt holds key 32 kt + 8 (r / 4) + 4 half + r % 4 against this lane's row
            v16f Sa[KT], Sb[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) Sa[kt][r] = Sb[kt][r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks) {
                bf16x8 qf[3];
#pragma unroll
                for (int p = 0; p < 3; ++p) qf[p] = __builtin_bit_cast(bf16x8, qp[ks][p]);
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    bf16x8 kf[3];
#pragma unroll
                    for (int p = 0; p < 3; ++p)
                        kf[p] = __builtin_bit_cast(bf16x8, *(const v4u *)&Ks[p][32 * kt + c][ks * 16 + half * 8]);
#pragma unroll
                    for (int q = 0; q < 6; q += 2) {
                        Sa[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[PA_[q]], qf[PB_[q]], Sa[kt], 0, 0, 0);
                        Sb[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[PA_[q + 1]], qf[PB_[q + 1]], Sb[kt], 0, 0, 0);
                    }
                }
            }

            // softmax of this lane's row, in the lane: half of the trip's keys here, half in lane ^ 32
            float sc[16 * KT];
            float m_tile = -INFINITY;
            if (j0 + KEYS <= wave_kfull) {  // uniform per wavefront: every key of the trip is visible to every row
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        sc[16 * kt + r] = Sa[kt][r] + Sb[kt][r];
                        m_tile = fmaxf(m_tile, sc[16 * kt + r]);
                    }
            } else {
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int j = j0 + 32 * kt + 8 * (r >> 2) + 4 * half + (r & 3);
                        const bool valid = j < L && (!a.causal || j <= my_pos);
                        sc[16 * kt + r] = valid ? Sa[kt][r] + Sb[kt][r] : -INFINITY;
                        m_tile = fmaxf(m_tile, sc[16 * kt + r]);
                    }
            }
            m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
            const float m_new = fmaxf(m_run, m_tile);
            const float m_ref = m_new > -INFINITY ? m_new : 0.f;  // nothing visible yet: every weight below is exp2(-inf) = 0
            const float alpha = fast_exp2(m_run - m_ref);
            m_run = m_new;
            float psum = 0.f;
#pragma unroll
            for (int r = 0; r < 16 * KT; ++r) {
                sc[r] = fast_exp2(sc[r] - m_ref);
                psum += sc[r];
            }
            l_run = fmaf(l_run, alpha, psum);
#pragma unroll
            for (int t = 0; t < DT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) O[t][r] *= alpha;

            // O^T += V^T P^T: P^T is this lane's weights, already where the B operand wants them
            // (registers 8 ks .. 8 ks + 7 are the keys at positions 16 ks + 8 half .. + 7 of V^T)
#pragma unroll
            for (int ks = 0; ks < KEYS / 16; ++ks) {
                bf16x8 pf[3];
                {
                    v2u lo[3], hi[3];
                    fa_split4((v4f){sc[8 * ks], sc[8 * ks + 1], sc[8 * ks + 2], sc[8 * ks + 3]}, lo);
                    fa_split4((v4f){sc[8 * ks + 4], sc[8 * ks + 5], sc[8 * ks + 6], sc[8 * ks + 7]}, hi);
#pragma unroll
                    for (int p = 0; p < 3; ++p) pf[p] = __builtin_bit_cast(bf16x8, (v4u){lo[p].x, lo[p].y, hi[p].x, hi[p].y});
                }
                bf16x8 vf[DT][3];
#pragma unroll
                for (int t = 0; t < DT; ++t)
#pragma unroll
                    for (int p = 0; p < 3; ++p)
                        vf[t][p] = __builtin_bit_cast(bf16x8, *(const v4u *)&Vt[p][32 * t + c][ks * 16 + half * 8]);
#pragma unroll
                for (int q = 0; q < 6; ++q)
#pragma unroll
                    for (int t = 0; t < DT; ++t)
                        O[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[t][PA_[q]], pf[PB_[q]], O[t], 0, 0, 0);
            }
        }
        __syncthreads();
    }

    // out = ctx / (sum + 1e-9), self_attention.rs:670-676; [B,S,Hq,D]
    const float inv = 1.0f / ((l_run + __shfl_xor(l_run, 32, 64)) + 1e-9f);
    const int i = q0 + my_row / NREP;
    if (i < a.s) {
        float *o = a.out + (((size_t)bb * a.s + i) * a.hq + (size_t)hk * NREP + my_row % NREP) * D;
#pragma unroll
        for (int t = 0; t < DT; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                v4f v = {O[t][4 * g] * inv, O[t][4 * g + 1] * inv, O[t][4 * g + 2] * inv, O[t][4 * g + 3] * inv};
                *(v4f *)(o + 32 * t + 8 * g + 4 * half) = v;
            }
    }
}

template <int D>
static int launch_fa_d(lumen_ctx *ctx, const AttnPrefillArgs &a) {
    const int nrep = a.hq / a.hkv;
    dim3 block(FA_THREADS);
#define LAUNCH_FA(NR)                                                                                    \
    hipLaunchKernelGGL((attn_prefill_bf16x3_kernel<D, NR, (D == 64 ? 2 : 1)>), dim3((a.s + FA_ROWS / NR - 1) / (FA_ROWS / NR), a.hkv, a.b), \
                       block, 0, ctx->stream, a)
    switch (nrep) {
        case 1: LAUNCH_FA(1); break;
        case 2: LAUNCH_FA(2); break;
        case 4: LAUNCH_FA(4); break;
        case 8: LAUNCH_FA(8); break;
        default: {  // any other group size: one query head per grid row, its KV head = head / n_rep
            AttnPrefillArgs b = a;
            b.kv_div = nrep;
            hipLaunchKernelGGL((attn_prefill_bf16x3_kernel<D, 1, (D == 64 ? 2 : 1)>), dim3((a.s + FA_ROWS - 1) / FA_ROWS, a.hq, a.b), block, 0,
                               ctx->stream, b);
        }
    }
#undef LAUNCH_FA
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

// Worth it from a few hundred positions on: below that the tile loop of the few workgroups is
// longer than the row loop of one workgroup per position.
bool attn_prefill_mfma_supported(const AttnPrefillArgs &a) { return (a.d == 64 || a.d == 128) && a.s >= 96; }

int launch_attn_prefill_mfma(lumen_ctx *ctx, const AttnPrefillArgs &a) {
    if (a.d == 64) return launch_fa_d<64>(ctx, a);
    if (a.d == 128) return launch_fa_d<128>(ctx, a);
    LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "matrix-core prefill attention: head_dim=%d (supported 64, 128)", a.d);
}

LUMEN_DEFINE_WARM(prefill_attention)
