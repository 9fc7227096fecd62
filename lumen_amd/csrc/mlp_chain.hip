// The MLP of a decoder layer for one token as ONE launch, for models whose products are latency rather than bytes.
//
// Reference path: LlamaMLP::forward (src/models/llama.rs:59-65): down(silu(gate(x)) * up(x)), with the
// post-attention RMSNorm in front and the residual add behind (LlamaDecoderLayer::forward_infer, llama.rs:113-115).
//
// As two launches (RMSNorm + gate|up + SwiGLU, then down + residual) a narrow model pays the ~2.2 us of start, first
// touch and tail twice for a few microseconds of streaming.  Here they are one grid of 512-thread workgroups with
// two roles, dispatched in this order:
//
//   [0, I / 8)    RMSNorm + gate|up + SwiGLU: one (gate_i, up_i) pair of rows per wavefront, both rows' weights in
//                 registers; act_i = silu(gate) * up leaves as a tagged word;
//   next N / 8    down: one row per wavefront, all of its I weights requested into registers at once, then the I tagged
//                 words are taken (each thread its own few), staged in LDS, multiplied, the residual added.
//
// The hand-over is the one of attn_oproj.hip: a value travels as one 8-byte word {bits, tag}, written and read
// atomically, the tag changing with every decode step and layer; producers have lower workgroup indices than their
// consumers, so they are resident or finished before a consumer waits; waits are bounded (spin_limit polls, then
// *err_dev = 1 and the wavefront goes on and exits).
#include "internal.h"
#include "attn_short_device.h"
#include "wave_reduce.h"
#include "stage_times.h"

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

#define MC_WAVES 8
#define MC_THREADS (MC_WAVES * 64)

template <bool BF16>
__device__ __forceinline__ float mc_dot16(const v4u raw, const float *xs) {
    const v4f xa = *(const v4f *)xs;
    if (BF16) {  // eight bf16 values, widened by a shift (src/loader.rs:58)
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

// NLH / NLD: 16-byte weight loads per lane and row of the gate|up / the down product (row length = loads * 64 *
// elements per load: hidden / intermediate).
template <int NLH, int NLD, bool BF16>
__global__ __launch_bounds__(MC_THREADS) void mlp_chain_kernel(const void *Wgu_hot, const float *h_hot, const float *norm_hot,
                                                               const void *Wdown_hot, const unsigned *step_dev_hot, int N_hot,
                                                               MlpChainArgs a_mem) {
    constexpr int VEC = BF16 ? 8 : 4;
    constexpr int ESZ = BF16 ? 2 : 4;
    constexpr int KH = NLH * 64 * VEC;  // hidden
    constexpr int KD = NLD * 64 * VEC;  // intermediate
    constexpr int EPT = KD / MC_THREADS;
    static_assert(KD % MC_THREADS == 0 && EPT >= 1, "the intermediate size must be a multiple of the workgroup size");
    __shared__ __align__(16) float xs[KD > KH ? KD : KH];
    __shared__ float sm[MC_WAVES];
    STAGE_T(0);
    const unsigned long long t_start = wall_clock64();
    const int N = N_hot;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ngu = KD / MC_WAVES;
    int blk = blockIdx.x;
    if (blk < ngu) {
        // ---- RMSNorm + gate|up + SwiGLU: rows (2u, 2u + 1) = (gate_u, up_u)
        constexpr int XP = (KH / 4 + MC_THREADS - 1) / MC_THREADS;
        const int unit = blk * MC_WAVES + wave;
        // x and the gains first: what is requested first arrives first, and the norm is what the multiplies wait for
        v4f xe[XP], ge[XP];
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int k = (tid + i * MC_THREADS) * 4;
            xe[i] = v4f{0.f, 0.f, 0.f, 0.f};
            ge[i] = xe[i];
            if (k < KH) {
                xe[i] = *(const v4f *)(h_hot + k);
                ge[i] = *(const v4f *)(norm_hot + k);
            }
        }
        v4u raw[2][NLH];
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const char *rp = (const char *)Wgu_hot + ((size_t)(2 * unit + r) * KH + (size_t)lane * VEC) * ESZ;
#pragma unroll
            for (int i = 0; i < NLH; ++i) raw[r][i] = __builtin_nontemporal_load((const v4u *)(rp + (size_t)i * 64 * VEC * ESZ));
        }
        const unsigned tag = *step_dev_hot * a_mem.tag_mul + a_mem.tag_add;
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
        for (int w = 0; w < MC_WAVES; ++w) tot += sm[w];
        const float inv = 1.0f / sqrtf(tot / (float)KH + a_mem.eps);
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            const int k = (tid + i * MC_THREADS) * 4;
            if (k < KH) {
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
        float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
        for (int i = 0; i < NLH; ++i) {
            acc0 += mc_dot16<BF16>(raw[0][i], xs + (i * 64 + lane) * VEC);
            acc1 += mc_dot16<BF16>(raw[1][i], xs + (i * 64 + lane) * VEC);
        }
        acc0 = wave_sum(acc0);
        acc1 = wave_sum(acc1);
        if (lane == 0) {
            // silu(gate) * up: x * (1 / (1 + exp(-x))), src/layers/activation.rs:143-146, llama.rs:60-63
            const float sig = 1.0f / (1.0f + expf(-acc0));
            tagged_store(a_mem.act_tagged + unit, (acc0 * sig) * acc1, tag);
        }
        STAGE_T_STORES_DONE(3);
        return;
    }
    blk -= ngu;
    {
        // ---- down + residual: one row per wavefront (rows past N: clamped, not stored)
        const int row = blk * MC_WAVES + wave;
        handover_pause_until(t_start, a_mem.pre_sleep);  // (the requests of the role before go first)
        v4u raw[NLD];
        {
            const char *rp = (const char *)Wdown_hot + ((size_t)min(row, N - 1) * KD + (size_t)lane * VEC) * ESZ;
#pragma unroll
            for (int i = 0; i < NLD; ++i) raw[i] = __builtin_nontemporal_load((const v4u *)(rp + (size_t)i * 64 * VEC * ESZ));
        }
        const unsigned tag = *step_dev_hot * a_mem.tag_mul + a_mem.tag_add;
        const float res = h_hot[min(row, N - 1)];
        STAGE_T(5);
        handover_pause_until(wall_clock64(), a_mem.poll_delay);
        {
            float v[EPT];
            if (!take_tagged<EPT>(a_mem.act_tagged + (size_t)tid * EPT, tag, a_mem.spin_limit, a_mem.poll_gap, v))
                __hip_atomic_store(a_mem.err_dev, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int e = 0; e < EPT; ++e) xs[tid * EPT + e] = v[e];
        }
        __syncthreads();
        STAGE_T(6);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < NLD; ++i) acc += mc_dot16<BF16>(raw[i], xs + (i * 64 + lane) * VEC);
        acc = wave_sum(acc);
        if (lane == 0 && row < N) a_mem.y[row] = res + acc;  // src/ops/arithmetic.rs:48-51 via llama.rs:115
        STAGE_T_STORES_DONE(7);
    }
}

static int mc_nl(int K, int w_bf16) {
    const int vec = w_bf16 ? 8 : 4;
    if (K <= 0 || K % (64 * vec)) return 0;
    return K / (64 * vec);
}

// hidden: two rows fit a wavefront's registers; intermediate: one row does, and divides among the 512 threads
bool mlp_chain_supported(int hidden, int inter, int w_bf16) {
    const int nlh = mc_nl(hidden, w_bf16), nld = mc_nl(inter, w_bf16);
    if (nlh != 2 && nlh != 4 && nlh != 8) return false;
    if (nld != 4 && nld != 8 && nld != 12 && nld != 16) return false;
    return inter % MC_THREADS == 0 && hidden % 8 == 0;
}

int mlp_chain_workgroups(int hidden, int inter) { return inter / MC_WAVES + (hidden + MC_WAVES - 1) / MC_WAVES; }

template <bool BF16>
static int launch_mc(lumen_ctx *ctx, const MlpChainArgs &a) {
    const int nlh = mc_nl(a.N, BF16), nld = mc_nl(a.I, BF16);
    const int n_wg = mlp_chain_workgroups(a.N, a.I);
    dim3 grid(n_wg), block(MC_THREADS);
    bool launched = false;
#define MC_LAUNCH(NLH, NLD)                                                                                                    \
    do {                                                                                                                       \
        if (nlh == NLH && nld == NLD) {                                                                                        \
            hipLaunchKernelGGL((mlp_chain_kernel<NLH, NLD, BF16>), grid, block, 0, ctx->stream, a.Wgu, a.h, a.norm_w, a.Wdown, \
                               a.step_dev, a.N, a);                                                                            \
            launched = true;                                                                                                   \
        }                                                                                                                      \
    } while (0)
#define MC_ROWS(NLH)    \
    do {                \
        MC_LAUNCH(NLH, 4);  \
        MC_LAUNCH(NLH, 8);  \
        MC_LAUNCH(NLH, 12); \
        MC_LAUNCH(NLH, 16); \
    } while (0)
    MC_ROWS(2);
    MC_ROWS(4);
    MC_ROWS(8);
#undef MC_ROWS
#undef MC_LAUNCH
    if (!launched) LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "MLP chain: no instance for hidden %d, intermediate %d", a.N, a.I);
    LUMEN_CHECK_LAUNCH();
    note_kernel(ctx, "mlp_chain_kernel<%d, %d, %s>", nlh, nld, BF16 ? "true" : "false");
    const int seg[2] = {a.I / MC_WAVES, n_wg};
    stage_times_report(ctx, "gate|up | down chain", n_wg,
                       "start, then gate|up: [1] requests out, [2] x staged, [3] acknowledged; down: [5] polls begin, "
                       "[6] input staged, [7] acknowledged", seg, 2);
    return LUMEN_OK;
}

int launch_mlp_chain(lumen_ctx *ctx, const MlpChainArgs &a) {
    if (!mlp_chain_supported(a.N, a.I, a.w_bf16))
        LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "MLP chain: hidden %d, intermediate %d not covered", a.N, a.I);
    if (!a.Wgu || !a.Wdown || !a.h || !a.norm_w || !a.y || !a.act_tagged || !a.step_dev || !a.err_dev)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "MLP chain: null argument");
    if ((((uintptr_t)a.Wgu | (uintptr_t)a.Wdown | (uintptr_t)a.h | (uintptr_t)a.norm_w) & 15) != 0)
        LUMEN_FAIL(LUMEN_ERR_INVALID, "MLP chain: operands must be 16-byte aligned");
    if (!handover_timing_ok(a.spin_limit, a.pre_sleep, a.poll_delay, a.poll_gap))
        LUMEN_FAIL(LUMEN_ERR_INVALID, "MLP chain: wait limits out of range (%u polls, pauses %d / %d / %d)", a.spin_limit,
                   a.pre_sleep, a.poll_delay, a.poll_gap);
    return a.w_bf16 ? launch_mc<true>(ctx, a) : launch_mc<false>(ctx, a);
}

LUMEN_DEFINE_WARM(mlp_chain)
