// Internal declarations shared by the translation units of liblumen_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <string>
#include <vector>

#include "../../include/lumen_hip.h"

// The dynamically sized LDS array of a kernel (one per kernel, sized by the launch)
#ifndef LUMEN_DYNAMIC_LDS
#define LUMEN_DYNAMIC_LDS(type, name) extern __shared__ __align__(16) type name[]
#endif

// ---------------------------------------------------------------- errors
void lumen_set_error(const char *fmt, ...);

#define LUMEN_FAIL(code, ...)           \
    do {                                \
        lumen_set_error(__VA_ARGS__);   \
        return (code);                  \
    } while (0)

#define HIP_TRY(expr)                                                                      \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess)                                                              \
            LUMEN_FAIL(LUMEN_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), \
                       __FILE__, __LINE__);                                                \
    } while (0)

#define LUMEN_TRY(expr)              \
    do {                             \
        int rc_ = (expr);            \
        if (rc_ != LUMEN_OK) return rc_; \
    } while (0)

#define LUMEN_CHECK_LAUNCH() HIP_TRY(hipGetLastError())

// ---------------------------------------------------------------- objects
#define LUMEN_BOUNCE_BYTES ((size_t)1 << 20)
struct lumen_ctx {
    int device = 0;
    int num_cus = 0;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    int *d_scratch_int = nullptr;  // small device scratch (argmax result etc.)
    void *bounce = nullptr;        // pinned host memory that small downloads travel through (LUMEN_BOUNCE_BYTES)
    // one int of pinned host memory the GPU can write: set to 1 by an operator-level launch whose bounded wait for
    // another workgroup's values ran out; lumen_ctx_synchronize and lumen_download report and clear it
    int *err_host = nullptr;
    float *gemm_ws = nullptr;      // split-K workspace of the prefill GEMM, grown on demand
    size_t gemm_ws_bytes = 0;
    // this device's address of the fixed scratch array behind lumen_attn_decode_static_f32
    unsigned char *attn_static = nullptr;
    size_t attn_static_bytes = 0;
    // name of the kernel instance the decode-path launchers started last (template arguments as a profiler prints
    // them), kept while note_kernels is set: the per-class profile hands these names out
    bool note_kernels = false;
    char last_kernel[160] = {0};
};
void note_kernel(lumen_ctx *ctx, const char *fmt, ...);
int attn_static_scratch_init(lumen_ctx *ctx);

struct lumen_rope {
    lumen_ctx *ctx = nullptr;
    int dim = 0, max_seq = 0;
    float theta = 0.f;
    float *cos_dev = nullptr, *sin_dev = nullptr;  // [max_seq, dim]
    std::vector<float> cos_host, sin_host;
};

struct lumen_kv_cache {
    lumen_ctx *ctx = nullptr;
    int b = 0, h_kv = 0, max_seq = 0, d = 0;
    int len = 0;            // host mirror of the position counter
    float *k = nullptr, *v = nullptr;
    bool owns = true;       // false when k/v are slices of a model-wide slab
    // decode attention, sliced long cache: the slices' states on their way to the workgroup that folds them,
    // tagged words [b*h_q_max, nsplit, d + 2], and the count of launches their tags are made of
    unsigned long long *part_tagged = nullptr;
    unsigned merge_epoch = 0;
    int part_heads = 0;
    int *d_pos = nullptr;    // device copy of len for lumen_qkv_rope_append_f32, allocated at its first call
    float *q_rot = nullptr;  // rotated queries of the prefill entry point, grown on demand
    size_t q_rot_floats = 0;
};

// ---------------------------------------------------------------- launchers
// Every launcher validates nothing: callers check shapes first.

enum GemvPro { PRO_NONE = 0, PRO_RMSNORM = 1, PRO_ATTN_FOLD = 2 };
enum GemvEpi { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2, EPI_ARGMAX = 3, EPI_ROPE_QKV = 4 };

struct GemvArgs {
    const void *W;        // [N, K] f32 or bf16 bits
    const float *x;       // [K]
    float *y;             // [N] (EPI_SWIGLU: [N/2])
    int N, K;
    int w_bf16;
    int pro, epi;
    const float *norm_w;  // PRO_RMSNORM: gain [K]
    float eps;
    const float *residual;  // EPI_RESIDUAL: [N]
    // x (and, with residual_sel, the residual) is row *row_sel of a [rows, row_stride] table:
    // the embedding gather folded into the first layer's GEMVs
    const int *row_sel;
    long row_stride;
    int x_sel, residual_sel;
    // EPI_ARGMAX (N < 2^24): y still receives the N values; the index of the first maximum goes to *tok_out and
    // *pos_inc is incremented, by the workgroup with the highest index, which waits for the others' candidates
    unsigned long long *amax_word;  // [gridDim.x] candidates {value, tag << 24 | row}, zero before the first launch
    unsigned *amax_epoch;           // launches so far (the tag is made of it; advanced by the kernel)
    int *err_dev;                   // set to 1 when the wait for the candidates ran into spin_limit
    unsigned spin_limit;
    int *tok_out, *pos_inc;
    int *tok_hist;     // optional [max_seq + 1]: the pick is also stored at index *pos_inc + 1
    unsigned *step_inc;  // optional: decode step counter, incremented together with *pos_inc
    // EPI_ROPE_QKV: rows are q|k|v heads of D; a unit is the RoPE pair (j, j + D/2) of one head.
    // q is rotated into y, k rotated and v as is go to row *pos of the KV cache.
    const float *cos_t, *sin_t;
    const int *pos;
    float *k_cache, *v_cache;  // [hkv, max_seq, D]
    int hq, hkv, D, max_seq;
    // PRO_ATTN_FOLD: x is the decode attention output [attn_hq * attn_d], still in the kernel's partial
    // states attn_part [attn_hq][attn_nslices][attn_d + 2] (ctx, m, l).  With *attn_pos + 1 cached rows,
    // slice 0 alone is in use up to attn_short_rows, else one slice per attn_trip rows.
    const float *attn_part;
    const int *attn_pos;
    int attn_nslices, attn_d, attn_trip, attn_short_rows;
};
#define GEMV_FOLD_MAX_SLICES 16  // PRO_ATTN_FOLD reads this many slice states per element, whatever the count in use
int launch_gemv(lumen_ctx *ctx, const GemvArgs &a);
int gemv_max_blocks(const lumen_ctx *ctx);
// grid of the fused GEMV kernel for an [N, K] product (workgroups; threads per workgroup in *threads_out)
int gemv_grid(const lumen_ctx *ctx, int N, int K, int w_bf16, int epi, int *threads_out);
// The template instance and launch shape the fused GEMV takes for a product: ONE function decides, the launcher
// and the name report (lumen_gemv_kernel_name) both read it.
struct GemvPick {
    bool fast;         // the fused kernel (else the generic one: K not a multiple of the load width, unaligned, K > 16384)
    int R;             // rows per unit
    int pro, epi;      // template prologue / epilogue
    int xb;            // 0: x requested ahead of the weights, 1: staged piece by piece, 4: four pieces at a time
    bool ka;           // K is a whole number of pieces
    int threads, blocks;
    size_t lds;
};
GemvPick gemv_pick(int num_cus, int N, int K, int w_bf16, int pro, int epi, bool aligned);
int gemv_kernel_name(const GemvPick &p, int w_bf16, char *buf, int buf_len);

struct GemmArgs {
    const float *A;   // [M, K]
    const void *W;    // [N, K]
    float *C;         // [M, N] (EPI_SWIGLU: [M, N/2])
    int M, N, K;
    int w_bf16;
    int epi;
    const float *residual;  // [M, N]
    float *part;            // split-K partial tiles [splits, M, N] (set by the launcher)
    // optional, with EPI_RESIDUAL: the RMSNorm of the finished rows as well, norm_out [M, N] = (C * inv_rms) * norm_w
    // (src/layers/norm/rms_norm.rs:45-58): where K is split the pass that adds the splits takes it along (one
    // launch instead of two), else a launch of its own follows
    const float *norm_w;    // [N] or null
    float *norm_out;
    float norm_eps;
    // optional, with EPI_STORE: where K is split, leave the partial products [splits, M, N] in the workspace for a
    // consumer that adds them itself (in split order) and report how many there are; 1 = C holds the product
    int keep_splits;
    int *splits_used;
};
int launch_gemm(lumen_ctx *ctx, const GemmArgs &a);
int gemm_reserve_workspace(lumen_ctx *ctx, size_t bytes);  // grows the split-K workspace (synchronises the stream when it does)
size_t gemm_workspace_bytes(const lumen_ctx *ctx, int M, int N, int K, int w_bf16);

// One empty kernel per translation unit with kernels.  The runtime loads a translation unit's device code at the first
// launch of one of its kernels (milliseconds for the larger ones); lumen_ctx_create launches these so that the first
// prompt does not pay for it.
#define LUMEN_DEFINE_WARM(name)                                                                  \
    __global__ void warm_##name##_kernel() {}                                                    \
    void lumen_warm_##name(hipStream_t s) { hipLaunchKernelGGL(warm_##name##_kernel, dim3(1), dim3(1), 0, s); }
void lumen_warm_attention(hipStream_t s);
void lumen_warm_attn_oproj(hipStream_t s);
void lumen_warm_elementwise(hipStream_t s);
void lumen_warm_gemm(hipStream_t s);
void lumen_warm_gemv(hipStream_t s);
void lumen_warm_mlp_chain(hipStream_t s);
void lumen_warm_prefill_attention(hipStream_t s);


int launch_rmsnorm(lumen_ctx *ctx, const float *x, const float *w, float *out, int rows, int dim, float eps);
int launch_silu(lumen_ctx *ctx, const float *x, float *out, size_t n);
int launch_add(lumen_ctx *ctx, const float *a, const float *b, float *out, size_t n);
int launch_mul(lumen_ctx *ctx, const float *a, const float *b, float *out, size_t n);
int launch_swiglu(lumen_ctx *ctx, const float *g, const float *u, float *out, size_t n);
// ids_dev int32 [n]; out [n, dim]
int launch_embedding(lumen_ctx *ctx, const float *W, const int *ids_dev, int n, int dim, int vocab, float *out);
// writes the index of the first maximum to *out_dev; if next_id/pos are given
// (device ints) also stores the index there and increments *pos by one
int launch_argmax(lumen_ctx *ctx, const float *x, int n, int *out_dev, int *pos_inc_dev);
// x, out [B, H, S, D], positions offset..offset+S-1
int launch_rope_bhsd(lumen_ctx *ctx, const float *x, float *out, const float *cos_t, const float *sin_t,
                     int b, int h, int s, int d, int offset);

struct AttnDecodeArgs {
    const float *q;     // [B, Hq, D] un-rotated (row stride q_stride floats per batch)
    const float *k_new; // [B, Hkv, D] un-rotated
    const float *v_new; // [B, Hkv, D]
    float *out;         // [B, Hq, D]
    float *k_cache, *v_cache;  // [B, Hkv, max_seq, D]
    const float *cos_t, *sin_t;
    const int *pos_dev; // device int: position of the new token (== past_len), or null
    int pos_host;       // used when pos_dev is null
    int b, hq, hkv, d, max_seq;
    float scale;
    const float *q_norm_w, *k_norm_w;  // per-head RMSNorm gains [D] or null
    float norm_eps;
    float *part;        // slice states for a consumer in a LATER launch (defer_merge), plain floats [b*hq][nsplit][d + 2]
    int nsplit;         // slices a long cache is cut into (attn_decode_nsplit)
    // slices merged inside the launch: their states travel as tagged words in part_tagged [b*hq][nsplit][d + 2]
    // (zero before the first launch); the tag is (*tag_dev, or 0 without one) * tag_mul + tag_add and must differ
    // from launch to launch on one buffer and never be 0
    const unsigned *tag_dev;
    unsigned tag_mul, tag_add;
    int pre_rotated;    // q is already rotated and row pos of the cache already written (fused QKV GEMV)
    int expect_short;   // hint: the cache is short (a few hundred rows); a wrong hint only costs time
    // Leave the merge of a long cache's slices to the consumer: every workgroup stores its partial state
    // (ctx[D], m, l) in `part` -- the short form in slice 0 -- and `out` is not written.  The o_proj GEMV
    // folds the partials while it stages its input (PRO_ATTN_FOLD).  Needs pre_rotated and one-trip slices.
    int defer_merge;
    // the output goes out as tagged 8-byte words {value, tag} instead of plain floats (the short form inside the
    // attention -> o_proj chain, attn_oproj.hip); null everywhere else
    unsigned long long *out_tagged;
    unsigned tag;
    // q, the new key and the new value ARRIVE as tagged words, [hq + 2 hkv, D] rotated (the q|k|v -> attention ->
    // o_proj chain): the cache row of the new token is not read, nothing is rotated or stored here; null everywhere else
    const unsigned long long *qkv_tagged;
    // the chained launch with several workgroups per query head: slices launched, and where a slice leaves its
    // state for the workgroup that folds them, [hq][tslices][d + 2] tagged words (part_tagged, as above)
    int tslices, slice_shift;  // (a slice covers 1 << slice_shift rows)
    unsigned long long *part_tagged;
    unsigned spin_limit;  // polls before a wait for tagged words gives up (then *err_dev = 1)
    int poll_gap;         // pause between polls, units of 256 clocks
    int *err_dev;
};
int launch_attn_decode(lumen_ctx *ctx, const AttnDecodeArgs &a);

// Decode attention and the o_proj product chained inside ONE launch (attn_oproj.hip): the first hq workgroups
// are the short-form attention (one query head each), the others the o_proj rows; the attention output travels
// between them as tagged words.  q rotated, cache row *pos_dev written already.
struct AttnOprojArgs {
    AttnDecodeArgs attn;          // q, caches, pos_dev, scale, hq, hkv, d, max_seq (b = 1, pre_rotated)
    const void *Wo;               // [N, K] f32 or bf16 bits, K = hq * d
    const float *residual;        // [N]: y = residual + Wo attn (src/models/llama.rs:110)
    float *y;                     // [N]
    int N, K, w_bf16;
    const int *row_sel;           // the residual is row *row_sel of a [rows, row_stride] table (first layer), or null
    long row_stride;
    unsigned long long *x_tagged; // [K] attention output on its way to the o_proj workgroups, zero at start
    const unsigned *step_dev;     // decode step counter of the model: the tag is *step_dev * tag_mul + tag_add
    unsigned tag_mul, tag_add;
    int *err_dev;                 // set to 1 when a wait ran into spin_limit
    unsigned spin_limit;          // polls before a waiting workgroup gives up
    int pre_sleep, poll_delay, poll_gap;  // timing of the o_proj workgroups (units of 256 clocks), see attn_oproj.hip
    // With Wqkv set the launch starts one step earlier: its first workgroups are RMSNorm + the q|k|v product + RoPE
    // + KV append (src/models/llama.rs:107, self_attention.rs:106-108, :161-176, :220-227) on `residual` (the layer
    // input), and q / new key / new value travel to the attention workgroups as tagged words -- un-rotated when
    // attn.q_norm_w / attn.k_norm_w are set (per-head norm, rotation and cache write then happen in the attention role).
    const void *Wqkv;             // [(hq + 2 hkv) * d, N] f32 or bf16 bits, or null
    const float *in_norm_w;       // [N] gains of the input RMSNorm
    float norm_eps;
    unsigned long long *qkv_tagged;  // [(hq + 2 hkv) * d]
    // Attention workgroups per query head (1 to ATTN_CHAIN_MAX_SLICES): slice s takes the cached rows
    // [s R, (s + 1) R), R = slice_rows (a power of two, a multiple of attn_decode_trip_rows(d)); with more
    // than one, hq further workgroups fold the slices of a head (part_tagged [hq][nslices][d + 2]) and hand the
    // result to the o_proj workgroups.  The position must lie below nslices * slice_rows.
    int nslices, slice_rows;
    unsigned long long *part_tagged;
    unsigned long long *t0_tagged;  // one word: the first workgroup's clock reading at its start
};
#define ATTN_CHAIN_MAX_SLICES 16
// Limits of the waits inside the chained launches, enforced by lumen_llama_set_handover and by the launchers: a
// pause is at most 100 us, a wait at most 2^22 polls of at most 16 x 256 clocks plus a trip to memory each -- about
// 10 s in the worst case, a few seconds with the default settings -- after which the waiting workgroup flags the
// failure and exits.
#define HANDOVER_MAX_TENTHS 1000
#define HANDOVER_MAX_GAP 16
#define HANDOVER_MAX_SPINS (1u << 22)
static inline bool handover_timing_ok(unsigned spin_limit, int pre_sleep, int poll_delay, int poll_gap) {
    return spin_limit <= HANDOVER_MAX_SPINS && pre_sleep >= 0 && pre_sleep <= HANDOVER_MAX_TENTHS && poll_delay >= 0 &&
           poll_delay <= HANDOVER_MAX_TENTHS && poll_gap >= 0 && poll_gap <= HANDOVER_MAX_GAP;
}
bool attn_oproj_supported(int hq, int hkv, int d, int N, int K, int w_bf16);
bool qkv_attn_oproj_supported(int hq, int hkv, int d, int N, int K, int w_bf16, int qk_norm);
int launch_attn_oproj(lumen_ctx *ctx, const AttnOprojArgs &a);

// RMSNorm + gate|up + SwiGLU and down + residual chained inside ONE launch (mlp_chain.hip); act travels between the
// roles as tagged words.
struct MlpChainArgs {
    const void *Wgu;     // [2 I, N] gate / up rows interleaved, f32 or bf16 bits
    const float *h;      // [N] layer-internal input: normalised for gate|up, added to the down product
    const float *norm_w; // [N] gains of the post-attention RMSNorm
    float eps;
    const void *Wdown;   // [N, I]
    float *y;            // [N]
    int N, I, w_bf16;    // hidden, intermediate
    unsigned long long *act_tagged;  // [I]
    const unsigned *step_dev;        // the tag is *step_dev * tag_mul + tag_add
    unsigned tag_mul, tag_add;
    int *err_dev;
    unsigned spin_limit;
    int pre_sleep, poll_delay, poll_gap;  // timing of the down workgroups (units of 256 clocks)
};
bool mlp_chain_supported(int hidden, int inter, int w_bf16);
int mlp_chain_workgroups(int hidden, int inter);
int launch_mlp_chain(lumen_ctx *ctx, const MlpChainArgs &a);

struct AttnPrefillArgs {
    const float *q;  // [B, S, Hq, D] un-rotated
    const float *k;  // [B, S, Hkv, D] un-rotated
    const float *v;  // [B, S, Hkv, D]
    float *out;      // [B, S, Hq, D]
    float *k_cache, *v_cache;
    const float *cos_t, *sin_t;
    int b, s, hq, hkv, d, max_seq, past_len;
    int q_stride, k_stride, v_stride;  // floats between consecutive positions
    float scale;
    int causal;
    int kv_div;  // set by the launcher: KV head of grid row y is y / kv_div (1 unless one query head per row)
    const float *q_norm_w, *k_norm_w;
    float norm_eps;
    float *q_rot;    // scratch [B, S, Hq, D]
    // q, k and v may arrive as in_splits partial sums (a GEMM's K splits), copy i at pointer + i * in_split_stride
    // floats, to be added in index order; 0 or 1 = plain values.
    int in_splits;
    size_t in_split_stride;
};
int launch_attn_prefill(lumen_ctx *ctx, const AttnPrefillArgs &a);
// the scores / softmax / context part on the matrix cores (q_rot and the cache rows already written)
bool attn_prefill_mfma_supported(const AttnPrefillArgs &a);
int launch_attn_prefill_mfma(lumen_ctx *ctx, const AttnPrefillArgs &a);

int attn_decode_nsplit(int max_seq, int d);
size_t attn_decode_part_floats(int b, int hq, int d, int nsplit);
// rows of one slice of a long cache, and the longest cache the one-workgroup-per-head form takes
int attn_decode_trip_rows(int d);
int attn_decode_short_rows(int d);

void rope_tables_host(std::vector<float> &cos_t, std::vector<float> &sin_t, int dim, int max_seq, float theta);
