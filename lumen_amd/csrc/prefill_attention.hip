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
// Per wavefront (32 rows) and key tile:
//   S  = Q K^T        Q split once into registers, K on its way into LDS ([part][key][element]);
//                     an operand is one 16-byte LDS read of 8 consecutive elements; two
//                     accumulators take turns so that consecutive instructions do not wait
//   row max           across the 32 lanes that hold a row's 32 keys (DPP + one permlane swap)
//   P  = exp2(S - m)  scores are kept in log2 units (Q is pre-multiplied by scale * log2 e);
//                     the row sums stay per lane and are folded across lanes once at the end
//   O  = alpha O + P V   P goes through a per-wavefront LDS patch (f32) to become an A operand
//                     and is split after that read; V is staged transposed ([part][element][key])
#include "internal.h"
#include "attn_device.h"

typedef float v16f __attribute__((ext_vector_type(16)));

#define FA_ROWS 128  // (position, head) rows per workgroup
#define FA_KEYS 32   // keys per tile
#define FA_THREADS 256

// Last step of a reduction over 32 lanes: combine lane l with lane l ^ 16.  v_permlane16_swap
// exchanges the odd 16-lane rows of one register with the even rows of another on the vector ALU
// (no trip through the LDS crossbar): with both operands v it leaves (row0,row0,row2,row2) and
// (row1,row1,row3,row3).
__device__ __forceinline__ float fmaxf16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float add16(float v) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// max over the 32 lanes of a half-wavefront; every lane gets the result
__device__ __forceinline__ float half_max(float v) {
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false)));  // row_ror:8
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false)));  // row_ror:4
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false)));  // row_ror:2
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false)));  // row_ror:1
    return fmaxf16(v);
}

__device__ __forceinline__ float half_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));
    return add16(v);
}

// ---- the same tile loop on the bf16 matrix cores at f32 accuracy (head_dim 64) ----
// As in the prompt-pass GEMM: an f32 value is the exact sum of three bf16 values, a product the sum
// of the six part products whose orders add up to at most four, accumulated in f32 by
// v_mfma_f32_32x32x16_bf16 -- 24 + 24 instructions of 8 passes per key tile and wavefront instead
// of 32 + 32 of 16 passes with the f32 instruction.  Q is split once into registers, K and V on
// their way into LDS ([part][key][element] and, transposed, [part][element][key]), P after the
// transposing trip through the per-wavefront LDS patch; K and V operands are single 16-byte LDS
// reads of 8 consecutive elements (keys).  Two accumulators take turns under Q K^T so that consecutive matrix
// instructions do not wait on each other.
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
// one value -> its three parts
__device__ __forceinline__ void fa_split1(float x, uint16_t (&part)[3]) {
#pragma unroll
    for (int p = 0; p < 3; ++p) {
        part[p] = (uint16_t)(__float_as_uint(x) >> 16);
        if (p < 2) x -= __uint_as_float(__float_as_uint(x) & 0xffff0000u);
    }
}

template <int D, int NREP>
__global__ __launch_bounds__(FA_THREADS) void attn_prefill_bf16x3_kernel(AttnPrefillArgs a) {
    constexpr int BQ = FA_ROWS / NREP;  // positions per workgroup
    constexpr int DT = D / 32;          // 32-wide output tiles per row
    constexpr int PIECES = D * FA_KEYS / 4 / FA_THREADS;  // 16-byte pieces of a K (or V) tile per thread
    // rows of 4 words more than a multiple of 32: the 16-byte reads of 8 neighbouring rows hit distinct banks
    constexpr int LDK = D + 8, LDV = FA_KEYS + 8;
    __shared__ __align__(16) uint16_t Ks[3][FA_KEYS][LDK];            // [part][key][element]
    __shared__ __align__(16) uint16_t Vt[3][D][LDV];                  // [part][element][key]
    __shared__ __align__(16) float Ps[FA_THREADS / 64][32][FA_KEYS + 4];  // [wavefront][row][key], f32: split after the transposing read

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 31, half = lane >> 5;
    // workgroups are dealt in index order: the blocks of late positions (most keys) go first
    const int q0 = (int)(gridDim.x - 1 - blockIdx.x) * BQ, hk = blockIdx.y, bb = blockIdx.z;
    const int L = a.past_len + a.s;
    const size_t head_base = ((size_t)bb * a.hkv + hk / a.kv_div) * a.max_seq * D;  // kv_div > 1: grid row = query head
    const float *Kc = a.k_cache + head_base, *Vc = a.v_cache + head_base;
    auto row_of = [&](int r) { return 8 * (r >> 2) + 4 * half + (r & 3); };

    // Q operand: lane (row c, half g) holds elements ks * 16 + g * 8 .. + 7 of its row for every 16-deep step
    const int my_row = wave * 32 + c;
    const int my_i = min(q0 + my_row / NREP, a.s - 1);  // clamped: rows past S are computed and dropped
    const float *qrow = a.q_rot + (((size_t)bb * a.s + my_i) * a.hq + (size_t)hk * NREP + my_row % NREP) * D;
    const float qf_scale = a.scale * LUMEN_LOG2E;
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

    v16f O[DT];
    float m_run[16], l_run[16];
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) O[t][r] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        m_run[r] = -INFINITY;
        l_run[r] = 0.f;
    }
    int pos_r[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) pos_r[r] = a.past_len + q0 + (wave * 32 + row_of(r)) / NREP;

    v4f kreg[PIECES], vreg[PIECES];
    auto fetch = [&](int j0) {
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int idx = tid + p * FA_THREADS;
            const int key = idx / (D / 4), k4 = (idx % (D / 4)) * 4;
            const int j = min(j0 + key, L - 1);  // keys past L are masked below
            kreg[p] = *(const v4f *)(Kc + (size_t)j * D + k4);
            vreg[p] = *(const v4f *)(Vc + (size_t)j * D + k4);
        }
    };

    constexpr int PA_[6] = {2, 0, 1, 1, 0, 0}, PB_[6] = {0, 2, 1, 0, 1, 0};  // part products by ascending size
    if (kmax > 0) fetch(0);
    for (int j0 = 0; j0 < kmax; j0 += FA_KEYS) {
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int idx = tid + p * FA_THREADS;
            const int key = idx / (D / 4), k4 = (idx % (D / 4)) * 4;
            v2u kp[3];
            fa_split4(kreg[p], kp);
#pragma unroll
            for (int q = 0; q < 3; ++q) *(v2u *)&Ks[q][key][k4] = kp[q];
            const float ve[4] = {vreg[p].x, vreg[p].y, vreg[p].z, vreg[p].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                uint16_t vp[3];
                fa_split1(ve[e], vp);
#pragma unroll
                for (int q = 0; q < 3; ++q) Vt[q][k4 + e][key] = vp[q];
            }
        }
        __syncthreads();
        if (j0 + FA_KEYS < kmax) fetch(j0 + FA_KEYS);  // in flight during the matrix instructions below

        if (j0 < wave_kmax) {  // uniform per wavefront: tiles wholly above the causal diagonal are skipped
            v16f Sa, Sb;
#pragma unroll
            for (int r = 0; r < 16; ++r) Sa[r] = Sb[r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < D / 16; ++ks) {
                bf16x8 kf[3], qf[3];
#pragma unroll
                for (int p = 0; p < 3; ++p) {
                    kf[p] = __builtin_bit_cast(bf16x8, *(const v4u *)&Ks[p][c][ks * 16 + half * 8]);
                    qf[p] = __builtin_bit_cast(bf16x8, qp[ks][p]);
                }
#pragma unroll
                for (int q = 0; q < 6; q += 2) {
                    Sa = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[PA_[q]], kf[PB_[q]], Sa, 0, 0, 0);
                    Sb = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[PA_[q + 1]], kf[PB_[q + 1]], Sb, 0, 0, 0);
                }
            }

            const int j = j0 + c;  // this lane's key
            float alpha[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const bool valid = j < L && (!a.causal || j <= pos_r[r]);
                const float s = valid ? Sa[r] + Sb[r] : -INFINITY;
                const float m_new = fmaxf(m_run[r], half_max(s));
                float p = 0.f;
                alpha[r] = 1.0f;
                if (m_new > -INFINITY) {
                    alpha[r] = fast_exp2(m_run[r] - m_new);  // exp2(-inf) = 0 on the row's first live tile
                    p = fast_exp2(s - m_new);
                }
                l_run[r] = fmaf(l_run[r], alpha[r], p);
                m_run[r] = m_new;
                Ps[wave][row_of(r)][c] = p;
            }
#pragma unroll
            for (int t = 0; t < DT; ++t)
#pragma unroll
                for (int r = 0; r < 16; ++r) O[t][r] *= alpha[r];
            __builtin_amdgcn_wave_barrier();  // P: written above by this wavefront, read below in another lane order
#pragma unroll
            for (int ks = 0; ks < FA_KEYS / 16; ++ks) {
                bf16x8 pf[3];
                {
                    v2u lo[3], hi[3];
                    fa_split4(*(const v4f *)&Ps[wave][c][ks * 16 + half * 8], lo);
                    fa_split4(*(const v4f *)&Ps[wave][c][ks * 16 + half * 8 + 4], hi);
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
                        O[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[PA_[q]], vf[t][PB_[q]], O[t], 0, 0, 0);
            }
        }
        __syncthreads();
    }

    // out = ctx / (sum + 1e-9), self_attention.rs:670-676; [B,S,Hq,D]
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const float inv = 1.0f / (half_sum(l_run[r]) + 1e-9f);
        const int row = wave * 32 + row_of(r);
        const int i = q0 + row / NREP;
        if (i < a.s) {
            float *o = a.out + (((size_t)bb * a.s + i) * a.hq + (size_t)hk * NREP + row % NREP) * D;
#pragma unroll
            for (int t = 0; t < DT; ++t) o[32 * t + c] = O[t][r] * inv;
        }
    }
}

template <int D>
static int launch_fa_d(lumen_ctx *ctx, const AttnPrefillArgs &a) {
    const int nrep = a.hq / a.hkv;
    dim3 block(FA_THREADS);
#define LAUNCH_FA(NR)                                                                                    \
    hipLaunchKernelGGL((attn_prefill_bf16x3_kernel<D, NR>), dim3((a.s + FA_ROWS / NR - 1) / (FA_ROWS / NR), a.hkv, a.b), \
                       block, 0, ctx->stream, a)
    switch (nrep) {
        case 1: LAUNCH_FA(1); break;
        case 2: LAUNCH_FA(2); break;
        case 4: LAUNCH_FA(4); break;
        case 8: LAUNCH_FA(8); break;
        default: {  // any other group size: one query head per grid row, its KV head = head / n_rep
            AttnPrefillArgs b = a;
            b.kv_div = nrep;
            hipLaunchKernelGGL((attn_prefill_bf16x3_kernel<D, 1>), dim3((a.s + FA_ROWS - 1) / FA_ROWS, a.hq, a.b), block, 0,
                               ctx->stream, b);
        }
    }
#undef LAUNCH_FA
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

// Worth it from a few hundred positions on: below that the tile loop of the few workgroups is
// longer than the row loop of one workgroup per position.
bool attn_prefill_mfma_supported(const AttnPrefillArgs &a) { return (a.d == 64 || a.d == 128) && a.s >= 192; }

int launch_attn_prefill_mfma(lumen_ctx *ctx, const AttnPrefillArgs &a) {
    if (a.d == 64) return launch_fa_d<64>(ctx, a);
    if (a.d == 128) return launch_fa_d<128>(ctx, a);
    LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "matrix-core prefill attention: head_dim=%d (supported 64, 128)", a.d);
}
