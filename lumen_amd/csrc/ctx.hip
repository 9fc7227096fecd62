// Context, device memory, stopwatch and error reporting of liblumen_hip.so.
#include "internal.h"
#include <cstdarg>
#include <cstdio>

#include <cstring>

static thread_local char g_err[512] = "";

void lumen_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char *lumen_last_error(void) { return g_err; }

extern "C" const char *lumen_version(void) { return "lumen-hip 0.1 (gfx950)"; }

extern "C" int lumen_ctx_create(int device, lumen_ctx **out) {
    if (!out) LUMEN_FAIL(LUMEN_ERR_INVALID, "lumen_ctx_create: out is null");
    *out = nullptr;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0)
        LUMEN_FAIL(LUMEN_ERR_NO_DEVICE, "no HIP device visible (%s)", hipGetErrorString(e));
    if (device < 0 || device >= n) LUMEN_FAIL(LUMEN_ERR_INVALID, "device %d out of range [0,%d)", device, n);
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        LUMEN_FAIL(LUMEN_ERR_NO_DEVICE, "device %d is %s; this library is built for gfx950 only", device,
                   prop.gcnArchName);
    lumen_ctx *c = new lumen_ctx();
    c->device = device;
    c->num_cus = prop.multiProcessorCount;
    HIP_TRY(hipStreamCreateWithFlags(&c->own_stream, hipStreamNonBlocking));
    c->stream = c->own_stream;
    HIP_TRY(hipEventCreate(&c->ev0));
    HIP_TRY(hipEventCreate(&c->ev1));
    HIP_TRY(hipMalloc((void **)&c->d_scratch_int, 64 * sizeof(int)));
    HIP_TRY(hipHostMalloc(&c->bounce, LUMEN_BOUNCE_BYTES, hipHostMallocDefault));
    HIP_TRY(hipHostMalloc((void **)&c->err_host, 64, hipHostMallocDefault));
    *c->err_host = 0;
    // load the device code of every translation unit now rather than under the first prompt
    lumen_warm_attention(c->stream);
    lumen_warm_attn_oproj(c->stream);
    lumen_warm_elementwise(c->stream);
    lumen_warm_gemm(c->stream);
    lumen_warm_gemv(c->stream);
    lumen_warm_mlp_chain(c->stream);
    lumen_warm_prefill_attention(c->stream);
    HIP_TRY(hipStreamSynchronize(c->stream));
    {   // the runtime sets up its device-to-host copy path over the first few copies of a process: have them here
        void *tmp = nullptr;
        HIP_TRY(hipMalloc(&tmp, (size_t)256 << 10));
        for (int i = 0; i < 3; ++i) {
            HIP_TRY(hipMemcpyAsync(c->bounce, tmp, (size_t)256 << 10, hipMemcpyDeviceToHost, c->stream));
            HIP_TRY(hipStreamSynchronize(c->stream));
        }
        HIP_TRY(hipFree(tmp));
    }
    const int src = attn_static_scratch_init(c);
    if (src != LUMEN_OK) {
        lumen_ctx_destroy(c);
        return src;
    }
    *out = c;
    return LUMEN_OK;
}

extern "C" int lumen_ctx_destroy(lumen_ctx *ctx) {
    if (!ctx) return LUMEN_OK;
    hipSetDevice(ctx->device);
    hipStreamSynchronize(ctx->stream);
    hipFree(ctx->d_scratch_int);
    if (ctx->bounce) hipHostFree(ctx->bounce);
    if (ctx->err_host) hipHostFree(ctx->err_host);
    if (ctx->gemm_ws) hipFree(ctx->gemm_ws);
    hipEventDestroy(ctx->ev0);
    hipEventDestroy(ctx->ev1);
    hipStreamDestroy(ctx->own_stream);
    delete ctx;
    return LUMEN_OK;
}

extern "C" int lumen_ctx_set_stream(lumen_ctx *ctx, void *hip_stream) {
    if (!ctx) LUMEN_FAIL(LUMEN_ERR_INVALID, "ctx is null");
    ctx->stream = hip_stream ? (hipStream_t)hip_stream : ctx->own_stream;
    return LUMEN_OK;
}

// after a synchronisation: did a bounded wait inside an operator-level launch run out?
static int check_wait_flag(lumen_ctx *ctx) {
    if (!ctx->err_host || !*(volatile int *)ctx->err_host) return LUMEN_OK;
    *(volatile int *)ctx->err_host = 0;
    LUMEN_FAIL(LUMEN_ERR_HIP, "a workgroup gave up waiting for values handed over inside a launch; the results of the "
                              "launches since the last synchronisation are invalid");
}

extern "C" int lumen_ctx_synchronize(lumen_ctx *ctx) {
    if (!ctx) LUMEN_FAIL(LUMEN_ERR_INVALID, "ctx is null");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return check_wait_flag(ctx);
}

extern "C" int lumen_timer_start(lumen_ctx *ctx) {
    if (!ctx) LUMEN_FAIL(LUMEN_ERR_INVALID, "ctx is null");
    HIP_TRY(hipEventRecord(ctx->ev0, ctx->stream));
    return LUMEN_OK;
}

extern "C" int lumen_timer_stop(lumen_ctx *ctx, float *ms_out) {
    if (!ctx || !ms_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "null argument");
    HIP_TRY(hipEventRecord(ctx->ev1, ctx->stream));
    HIP_TRY(hipEventSynchronize(ctx->ev1));
    HIP_TRY(hipEventElapsedTime(ms_out, ctx->ev0, ctx->ev1));
    return LUMEN_OK;
}

extern "C" int lumen_malloc(lumen_ctx *ctx, size_t bytes, void **dev_out) {
    if (!ctx || !dev_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "null argument");
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipMalloc(dev_out, bytes ? bytes : 16));
    return LUMEN_OK;
}

extern "C" int lumen_free(lumen_ctx *ctx, void *dev) {
    if (!ctx) LUMEN_FAIL(LUMEN_ERR_INVALID, "ctx is null");
    if (!dev) return LUMEN_OK;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipFree(dev));
    return LUMEN_OK;
}

extern "C" int lumen_upload(lumen_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    if (!ctx || (bytes && (!dst_dev || !src_host))) LUMEN_FAIL(LUMEN_ERR_INVALID, "null argument");
    if (!bytes) return LUMEN_OK;
    HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return LUMEN_OK;
}

extern "C" int lumen_download(lumen_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    if (!ctx || (bytes && (!dst_host || !src_dev))) LUMEN_FAIL(LUMEN_ERR_INVALID, "null argument");
    if (!bytes) return LUMEN_OK;
    // A row of logits goes through the context's pinned buffer: a copy into pageable memory leaves it to the runtime
    // whether to stage or to pin the caller's pages, and the second such copy of a process took 5 ms for 128 KB.
    if (bytes <= LUMEN_BOUNCE_BYTES && ctx->bounce) {
        HIP_TRY(hipMemcpyAsync(ctx->bounce, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
        HIP_TRY(hipStreamSynchronize(ctx->stream));
        memcpy(dst_host, ctx->bounce, bytes);
        return check_wait_flag(ctx);
    }
    HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return check_wait_flag(ctx);
}

extern "C" int lumen_ctx_num_cus(const lumen_ctx *ctx, int *num_cus_out) {
    if (!ctx || !num_cus_out) LUMEN_FAIL(LUMEN_ERR_INVALID, "null argument");
    *num_cus_out = ctx->num_cus;
    return LUMEN_OK;
}

extern "C" int lumen_copy_d2d(lumen_ctx *ctx, void *dst_dev, const void *src_dev, size_t bytes) {
    if (!ctx || (bytes && (!dst_dev || !src_dev))) LUMEN_FAIL(LUMEN_ERR_INVALID, "null argument");
    if (!bytes) return LUMEN_OK;
    HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return LUMEN_OK;
}

void note_kernel(lumen_ctx *ctx, const char *fmt, ...) {
    if (!ctx || !ctx->note_kernels) return;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ctx->last_kernel, sizeof ctx->last_kernel, fmt, ap);
    va_end(ap);
}
