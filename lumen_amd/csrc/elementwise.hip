// Small HBM-bound kernels of the path: RMSNorm, SiLU / add / mul / SwiGLU,
// embedding gather, greedy argmax and the tensor form of RoPE.
#include "internal.h"
#include "wave_reduce.h"

#include <cmath>

typedef float v4f __attribute__((ext_vector_type(4)));


// ------------------------------------------------------------------ RMSNorm
// One workgroup per row: sum of squares, rms = sqrt(ss/dim + eps), out = (x * inv) * w.
// src/layers/norm/rms_norm.rs:45-58
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                      float *__restrict__ out, int dim, float eps) {
    __shared__ float red[4];
    const float *xr = x + (size_t)blockIdx.x * dim;
    float *o = out + (size_t)blockIdx.x * dim;
    const int tid = threadIdx.x;
    float ss = 0.f;
    for (int i = tid; i < dim; i += 256) {
        const float v = xr[i];
        ss = fmaf(v, v, ss);
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    const float rms = sqrtf(tot / (float)dim + eps);
    const float inv = 1.0f / rms;
    for (int i = tid; i < dim; i += 256) o[i] = xr[i] * inv * w[i];
}

// The same for rows of up to 1024 * VPT floats that are 16-byte aligned: a thread requests all of its
// pieces of the row and of the gains at once (the scalar loop above takes a trip to memory per element
// and pass) and keeps the row in registers between the two passes.
template <int VPT>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                          float *__restrict__ out, int dim, float eps) {
    __shared__ float red[4];
    const float *xr = x + (size_t)blockIdx.x * dim;
    float *o = out + (size_t)blockIdx.x * dim;
    const int tid = threadIdx.x;
    v4f v[VPT], g[VPT];
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int k = (tid + i * 256) * 4;
        v[i] = v4f{0.f, 0.f, 0.f, 0.f};
        g[i] = v4f{0.f, 0.f, 0.f, 0.f};
        if (k < dim) {
            v[i] = *(const v4f *)(xr + k);
            g[i] = *(const v4f *)(w + k);
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        ss = fmaf(v[i].x, v[i].x, ss);
        ss = fmaf(v[i].y, v[i].y, ss);
        ss = fmaf(v[i].z, v[i].z, ss);
        ss = fmaf(v[i].w, v[i].w, ss);
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    const float rms = sqrtf(tot / (float)dim + eps);
    const float inv = 1.0f / rms;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int k = (tid + i * 256) * 4;
        if (k < dim) {
            v4f r;
            r.x = v[i].x * inv * g[i].x;
            r.y = v[i].y * inv * g[i].y;
            r.z = v[i].z * inv * g[i].z;
            r.w = v[i].w * inv * g[i].w;
            *(v4f *)(o + k) = r;
        }
    }
}

int launch_rmsnorm(lumen_ctx *ctx, const float *x, const float *w, float *out, int rows, int dim, float eps) {
    if (rows <= 0 || dim <= 0) return LUMEN_OK;
    const bool vec = dim % 4 == 0 && ((((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) & 15) == 0);
    if (vec && dim <= 2048)
        hipLaunchKernelGGL(rmsnorm_vec_kernel<2>, dim3(rows), dim3(256), 0, ctx->stream, x, w, out, dim, eps);
    else if (vec && dim <= 4096)
        hipLaunchKernelGGL(rmsnorm_vec_kernel<4>, dim3(rows), dim3(256), 0, ctx->stream, x, w, out, dim, eps);
    else
        hipLaunchKernelGGL(rmsnorm_kernel, dim3(rows), dim3(256), 0, ctx->stream, x, w, out, dim, eps);
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

// -------------------------------------------------------------- elementwise
enum { OP_SILU, OP_ADD, OP_MUL, OP_SWIGLU, OP_COPY };

template <int OP>
__global__ __launch_bounds__(256) void ew_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                 float *__restrict__ out, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const float x = a[i];
        float r;
        if (OP == OP_SILU) {
            const float sig = 1.0f / (1.0f + expf(-x));  // src/layers/activation.rs:143-146
            r = x * sig;
        } else if (OP == OP_COPY) {
            r = x;
        } else if (OP == OP_ADD) {
            r = x + b[i];
        } else if (OP == OP_MUL) {
            r = x * b[i];
        } else {
            const float sig = 1.0f / (1.0f + expf(-x));
            r = (x * sig) * b[i];  // src/models/llama.rs:60-63
        }
        out[i] = r;
    }
}

template <int OP>
static int launch_ew(lumen_ctx *ctx, const float *a, const float *b, float *out, size_t n) {
    if (n == 0) return LUMEN_OK;
    size_t blocks = (n + 255) / 256;
    const size_t cap = (size_t)ctx->num_cus * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(ew_kernel<OP>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a, b, out, n);
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

int launch_silu(lumen_ctx *ctx, const float *x, float *out, size_t n) { return launch_ew<OP_SILU>(ctx, x, x, out, n); }
int launch_add(lumen_ctx *ctx, const float *a, const float *b, float *out, size_t n) { return launch_ew<OP_ADD>(ctx, a, b, out, n); }
int launch_mul(lumen_ctx *ctx, const float *a, const float *b, float *out, size_t n) { return launch_ew<OP_MUL>(ctx, a, b, out, n); }
int launch_swiglu(lumen_ctx *ctx, const float *g, const float *u, float *out, size_t n) { return launch_ew<OP_SWIGLU>(ctx, g, u, out, n); }
static int launch_copy(lumen_ctx *ctx, const float *x, float *out, size_t n) { return launch_ew<OP_COPY>(ctx, x, x, out, n); }

// ---------------------------------------------------------------- embedding
// out[t, :] = W[ids[t], :], src/layers/basic/embedding.rs:47-57.  ids were
// range-checked on the host; the device clamps so that a stale id can never
// read outside the table.
__global__ __launch_bounds__(256) void embedding_kernel(const float *__restrict__ W, const int *__restrict__ ids,
                                                        int dim, int vocab, float *__restrict__ out) {
    int id = ids[blockIdx.x];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const float *src = W + (size_t)id * dim;
    float *dst = out + (size_t)blockIdx.x * dim;
    for (int i = threadIdx.x; i < dim; i += 256) dst[i] = src[i];
}

int launch_embedding(lumen_ctx *ctx, const float *W, const int *ids_dev, int n, int dim, int vocab, float *out) {
    if (n <= 0) return LUMEN_OK;
    hipLaunchKernelGGL(embedding_kernel, dim3(n), dim3(256), 0, ctx->stream, W, ids_dev, dim, vocab, out);
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

// ------------------------------------------------------------------- argmax
// Single workgroup; first index of the maximum (lowest index wins ties).
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ x, int n, int *__restrict__ out,
                                                      int *__restrict__ pos_inc) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    const int tid = threadIdx.x;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int i = tid; i < n; i += 1024) {
        const float v = x[i];
        if (v > best || (v == best && i < idx)) {
            best = v;
            idx = i;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(idx, off, 64);
        if (ov > best || (ov == best && oi < idx)) {
            best = ov;
            idx = oi;
        }
    }
    if ((tid & 63) == 0) {
        bv[tid >> 6] = best;
        bi[tid >> 6] = idx;
    }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < 16; ++w)
            if (bv[w] > best || (bv[w] == best && bi[w] < idx)) {
                best = bv[w];
                idx = bi[w];
            }
        if (idx == 0x7fffffff) idx = 0;  // all NaN / -inf: index 0 like a sequential scan
        *out = idx;
        if (pos_inc) *pos_inc += 1;
    }
}

int launch_argmax(lumen_ctx *ctx, const float *x, int n, int *out_dev, int *pos_inc_dev) {
    hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(1024), 0, ctx->stream, x, n, out_dev, pos_inc_dev);
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

// --------------------------------------------------------------------- RoPE
// freq = 1 / theta^(2j/dim), val = pos * freq, cos/sin in f32, both halves
// alike: src/layers/attention/encoding.rs:29-54.  Computed on the host with
// libm so that the table holds the same values as the reference's.
void rope_tables_host(std::vector<float> &cos_t, std::vector<float> &sin_t, int dim, int max_seq, float theta) {
    const int half = dim / 2;
    cos_t.assign((size_t)max_seq * dim, 0.f);
    sin_t.assign((size_t)max_seq * dim, 0.f);
    std::vector<float> freq(half);
    for (int j = 0; j < half; ++j) freq[j] = 1.0f / powf(theta, ((float)j * 2.0f) / (float)dim);
    for (int i = 0; i < max_seq; ++i) {
        const float pos = (float)i;
        for (int j = 0; j < half; ++j) {
            const float val = pos * freq[j];
            const float c = cosf(val), s = sinf(val);
            cos_t[(size_t)i * dim + j] = c;
            cos_t[(size_t)i * dim + j + half] = c;
            sin_t[(size_t)i * dim + j] = s;
            sin_t[(size_t)i * dim + j + half] = s;
        }
    }
}

// x, out [B*H, S, D]: out[j] = x1*c - x2*s, out[j+half] = x2*c + x1*s (encoding.rs:103-116)
__global__ __launch_bounds__(256) void rope_bhsd_kernel(const float *__restrict__ x, float *__restrict__ out,
                                                        const float *__restrict__ cos_t,
                                                        const float *__restrict__ sin_t, int s, int d, int offset,
                                                        size_t npairs) {
    const int half = d / 2;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x; p < npairs; p += stride) {
        const int j = (int)(p % half);
        const size_t row = p / half;  // (b*h, s) flattened
        const int ss = (int)(row % s);
        const float *xr = x + row * d;
        const float x1 = xr[j], x2 = xr[j + half];
        const float c = cos_t[(size_t)(offset + ss) * d + j];
        const float sv = sin_t[(size_t)(offset + ss) * d + j];
        {
#pragma clang fp contract(off)  // separate multiplies and add, like the reference's compiled code
            out[row * d + j] = x1 * c - x2 * sv;
            out[row * d + j + half] = x2 * c + x1 * sv;
        }
    }
}

int launch_rope_bhsd(lumen_ctx *ctx, const float *x, float *out, const float *cos_t, const float *sin_t, int b, int h,
                     int s, int d, int offset) {
    const size_t npairs = (size_t)b * h * s * (d / 2);
    if (npairs == 0) return LUMEN_OK;
    size_t blocks = (npairs + 255) / 256;
    const size_t cap = (size_t)ctx->num_cus * 16;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL(rope_bhsd_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, x, out, cos_t, sin_t, s, d,
                       offset, npairs);
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

// ---------------------------------------------------------------------- C ABI
extern "C" int lumen_rmsnorm_f32(lumen_ctx *ctx, const float *x, const float *w, float *out, int rows, int dim,
                                 float eps) {
    if (!ctx || !x || !w || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "rmsnorm: null argument");
    if (rows < 0 || dim < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "rmsnorm: negative dimension");
    return launch_rmsnorm(ctx, x, w, out, rows, dim, eps);
}

#define EW_ABI1(name, fn)                                                                 \
    extern "C" int name(lumen_ctx *ctx, const float *x, float *out, size_t n) {           \
        if (!ctx || ((!x || !out) && n)) LUMEN_FAIL(LUMEN_ERR_INVALID, #name ": null argument"); \
        return fn(ctx, x, out, n);                                                        \
    }
#define EW_ABI2(name, fn)                                                                         \
    extern "C" int name(lumen_ctx *ctx, const float *a, const float *b, float *out, size_t n) {   \
        if (!ctx || ((!a || !b || !out) && n)) LUMEN_FAIL(LUMEN_ERR_INVALID, #name ": null argument"); \
        return fn(ctx, a, b, out, n);                                                             \
    }
EW_ABI1(lumen_silu_f32, launch_silu)
EW_ABI1(lumen_copy_f32, launch_copy)
EW_ABI2(lumen_add_f32, launch_add)
EW_ABI2(lumen_mul_f32, launch_mul)
EW_ABI2(lumen_swiglu_f32, launch_swiglu)

extern "C" int lumen_embedding_f32(lumen_ctx *ctx, const float *W, const float *ids_host, int n_ids, int vocab,
                                   int dim, float *out) {
    if (!ctx || !W || (!ids_host && n_ids) || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "embedding: null argument");
    if (n_ids <= 0) return LUMEN_OK;
    std::vector<int> ids(n_ids);
    for (int t = 0; t < n_ids; ++t) {
        const float f = ids_host[t];
        // Rust `as usize`: truncates toward zero, saturates, NaN -> 0 (embedding.rs:50)
        long long idx = (f > 0.0f) ? (f >= 9.0e18f ? (long long)9e18 : (long long)f) : 0;
        if (idx >= vocab)  // embedding.rs:55
            LUMEN_FAIL(LUMEN_ERR_EMBED_OOB, "Embedding index out of bounds: %lld >= %d", idx, vocab);
        ids[t] = (int)idx;
    }
    int *ids_dev = nullptr;
    HIP_TRY(hipMalloc((void **)&ids_dev, sizeof(int) * (size_t)n_ids));
    hipError_t e = hipMemcpyAsync(ids_dev, ids.data(), sizeof(int) * (size_t)n_ids, hipMemcpyHostToDevice, ctx->stream);
    int rc = LUMEN_OK;
    if (e == hipSuccess) rc = launch_embedding(ctx, W, ids_dev, n_ids, dim, vocab, out);
    hipStreamSynchronize(ctx->stream);
    hipFree(ids_dev);
    if (e != hipSuccess) LUMEN_FAIL(LUMEN_ERR_HIP, "embedding: id upload failed: %s", hipGetErrorString(e));
    return rc;
}

extern "C" int lumen_argmax_f32(lumen_ctx *ctx, const float *x, int n, int *index_host_out) {
    if (!ctx || !x || !index_host_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "argmax: null argument");
    if (n <= 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "argmax: empty input");
    LUMEN_TRY(launch_argmax(ctx, x, n, ctx->d_scratch_int, nullptr));
    HIP_TRY(hipMemcpyAsync(index_host_out, ctx->d_scratch_int, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return LUMEN_OK;
}

extern "C" int lumen_rope_create(lumen_ctx *ctx, int dim, int max_seq, float theta, lumen_rope **out) {
    if (!ctx || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "rope_create: null argument");
    if (dim <= 0 || (dim & 1) || max_seq <= 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "rope_create: dim=%d max_seq=%d", dim, max_seq);
    lumen_rope *r = new lumen_rope();
    r->ctx = ctx; r->dim = dim; r->max_seq = max_seq; r->theta = theta;
    rope_tables_host(r->cos_host, r->sin_host, dim, max_seq, theta);
    const size_t bytes = sizeof(float) * (size_t)max_seq * dim;
    if (hipMalloc((void **)&r->cos_dev, bytes) != hipSuccess || hipMalloc((void **)&r->sin_dev, bytes) != hipSuccess) {
        hipFree(r->cos_dev);
        delete r;
        LUMEN_FAIL(LUMEN_ERR_HIP, "rope_create: hipMalloc of %zu bytes failed", bytes);
    }
    int rc = lumen_upload(ctx, r->cos_dev, r->cos_host.data(), bytes);
    if (rc == LUMEN_OK) rc = lumen_upload(ctx, r->sin_dev, r->sin_host.data(), bytes);
    if (rc != LUMEN_OK) { lumen_rope_destroy(r); return rc; }
    *out = r;
    return LUMEN_OK;
}

extern "C" int lumen_rope_destroy(lumen_rope *r) {
    if (!r) return LUMEN_OK;
    hipStreamSynchronize(r->ctx->stream);
    hipFree(r->cos_dev);
    hipFree(r->sin_dev);
    delete r;
    return LUMEN_OK;
}

extern "C" int lumen_rope_tables_download(lumen_rope *r, float *cos_host, float *sin_host) {
    if (!r || !cos_host || !sin_host) LUMEN_FAIL(LUMEN_ERR_INVALID, "rope_tables_download: null argument");
    const size_t bytes = sizeof(float) * (size_t)r->max_seq * r->dim;
    LUMEN_TRY(lumen_download(r->ctx, cos_host, r->cos_dev, bytes));
    return lumen_download(r->ctx, sin_host, r->sin_dev, bytes);
}

extern "C" int lumen_rope_forward_f32(lumen_rope *r, const float *x, float *out, int b, int h, int s, int d, int offset) {
    if (!r || !x || !out) LUMEN_FAIL(LUMEN_ERR_INVALID, "rope_forward: null argument");
    if (d != r->dim) LUMEN_FAIL(LUMEN_ERR_SHAPE, "RoPE dimension mismatch: %d vs %d", d, r->dim);  // encoding.rs:60
    if (offset < 0 || s < 0 || offset + s > r->max_seq)  // encoding.rs:62-68
        LUMEN_FAIL(LUMEN_ERR_ROPE_RANGE, "RoPE index out of range: offset %d + len %d > max %d", offset, s, r->max_seq);
    return launch_rope_bhsd(r->ctx, x, out, r->cos_dev, r->sin_dev, b, h, s, d, offset);
}

extern "C" int lumen_rope_1token_copy_f32(lumen_rope *r, const float *src, float *dst, int d, int pos) {
    if (!r || !src || !dst) LUMEN_FAIL(LUMEN_ERR_INVALID, "rope_1token_copy: null argument");
    if (d != r->dim) LUMEN_FAIL(LUMEN_ERR_SHAPE, "RoPE src len mismatch: %d vs %d", d, r->dim);  // encoding.rs:174-175
    if (pos < 0 || pos >= r->max_seq)  // encoding.rs:176-181
        LUMEN_FAIL(LUMEN_ERR_ROPE_RANGE, "RoPE index out of range: pos %d >= max %d", pos, r->max_seq);
    return launch_rope_bhsd(r->ctx, src, dst, r->cos_dev, r->sin_dev, 1, 1, 1, d, pos);
}

LUMEN_DEFINE_WARM(elementwise)
