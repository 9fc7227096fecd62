// Dense C[M,N] = A[M,K] W[N,K]^T for the M > 1 (prompt prefill) branch of
// ops::matmul::matmul, src/ops/matmul.rs:70-92, on the gfx950 matrix cores.
//
// fp32 throughout: v_mfma_f32_32x32x2_f32 takes one f32 of A and one of W per
// lane and accumulates a 32x32 tile in 16 registers per lane, so the result
// carries full fp32 precision (the reference computes in f32 on the CPU).
// bf16-stored weights are widened while they are staged into LDS, which is
// the reference's own load-time upcast (src/loader.rs:58) moved to the device.
//
// Workgroup = 4 wavefronts (2x2), 128x128 output tile, 32-deep K slices staged
// k-major in LDS.  The global loads of slice s+1 are issued into registers
// before the matrix instructions of slice s, so their latency is covered by
// 64 MFMAs per wavefront.  When the tile grid alone cannot fill the chip
// (prompt of a few hundred tokens against a 2048-row weight) the K range is
// split over gridDim.z; each split writes its partial tile to a workspace and
// a second kernel adds the splits in index order and applies the epilogue, so
// the result does not depend on scheduling.
#include "internal.h"

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

#define BM 128
#define BN 128
#define BK 32
#define LDT (BM + 1)
#define STAGE 4  // 16-byte pieces of A and of W per thread per slice: 128 rows x 32 k / 256 threads

__device__ __forceinline__ float silu_g(float g) {
    const float sig = 1.0f / (1.0f + expf(-g));
    return g * sig;
}

// PARTIAL: store the raw tile of this K split to a.part[blockIdx.z][M][N]; the epilogue runs in
// gemm_reduce_kernel.
template <bool BF16, int EPI, bool PARTIAL>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(GemmArgs a) {
    __shared__ float As[BK][LDT];
    __shared__ float Ws[BK][LDT];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int bm = blockIdx.y * BM, bn = blockIdx.x * BN;
    const int M = a.M, N = a.N, K = a.K;
    const float *A = a.A;
    // K range of this split, in whole slices
    const int slices = (K + BK - 1) / BK;
    const int per = (slices + (int)gridDim.z - 1) / (int)gridDim.z;
    const int kb = (int)blockIdx.z * per * BK;
    const int ke = min(K, kb + per * BK);

    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    v4f va[STAGE], vw[STAGE];
    // piece i of this thread: row (tid + 256 i) / 8, k offset 4 * ((tid + 256 i) % 8)
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < STAGE; ++i) {
            const int idx = tid + i * 256;
            const int row = idx >> 3, k4 = (idx & 7) * 4;
            va[i] = (v4f){0.f, 0.f, 0.f, 0.f};
            vw[i] = (v4f){0.f, 0.f, 0.f, 0.f};
            if (k0 + k4 < ke) {  // K % 4 == 0: a piece is inside or outside as a whole
                if (bm + row < M) va[i] = *(const v4f *)(A + (size_t)(bm + row) * K + k0 + k4);
                if (bn + row < N) {
                    if (BF16) {
                        const v2u raw = *(const v2u *)((const uint16_t *)a.W + (size_t)(bn + row) * K + k0 + k4);
                        vw[i].x = __uint_as_float(raw.x << 16);
                        vw[i].y = __uint_as_float(raw.x & 0xffff0000u);
                        vw[i].z = __uint_as_float(raw.y << 16);
                        vw[i].w = __uint_as_float(raw.y & 0xffff0000u);
                    } else {
                        vw[i] = *(const v4f *)((const float *)a.W + (size_t)(bn + row) * K + k0 + k4);
                    }
                }
            }
        }
    };

    if (kb < ke) fetch(kb);
    for (int k0 = kb; k0 < ke; k0 += BK) {
#pragma unroll
        for (int i = 0; i < STAGE; ++i) {
            const int idx = tid + i * 256;
            const int row = idx >> 3, k4 = (idx & 7) * 4;
            As[k4 + 0][row] = va[i].x; As[k4 + 1][row] = va[i].y; As[k4 + 2][row] = va[i].z; As[k4 + 3][row] = va[i].w;
            Ws[k4 + 0][row] = vw[i].x; Ws[k4 + 1][row] = vw[i].y; Ws[k4 + 2][row] = vw[i].z; Ws[k4 + 3][row] = vw[i].w;
        }
        __syncthreads();
        if (k0 + BK < ke) fetch(k0 + BK);  // in flight during the matrix instructions below
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            const int kr = kk + (lane >> 5), c = lane & 31;
            float af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = As[kr][wm * 64 + i * 32 + c];
                bf[i] = Ws[kr][wn * 64 + i * 32 + c];
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // accumulator register r of lane l holds C[row = 8*(r/4) + 4*(l/32) + r%4][col = l%32] of the 32x32 tile
    float *part = PARTIAL ? a.part + (size_t)blockIdx.z * M * N : nullptr;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = bm + wm * 64 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                const int col = bn + wn * 64 + j * 32 + (lane & 31);
                const float v = acc[i][j][r];
                if (PARTIAL) {
                    if (row < M && col < N) part[(size_t)row * N + col] = v;
                } else if (EPI == EPI_SWIGLU) {
                    // columns (2c, 2c+1) = (gate_c, up_c): silu(gate) * up, src/models/llama.rs:60-63
                    const float up = __shfl_xor(v, 1, 64);
                    if (!(col & 1) && row < M && col < N) a.C[(size_t)row * (N >> 1) + (col >> 1)] = silu_g(v) * up;
                } else if (row < M && col < N) {
                    const size_t o = (size_t)row * N + col;
                    a.C[o] = (EPI == EPI_RESIDUAL) ? a.residual[o] + v : v;
                }
            }
}

// Adds the K splits of every output element in split order and applies the epilogue.
template <int EPI>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(GemmArgs a, int splits) {
    const size_t MN = (size_t)a.M * a.N;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    if (EPI == EPI_SWIGLU) {
        for (size_t p = (size_t)blockIdx.x * blockDim.x + threadIdx.x; p < MN / 2; p += stride) {
            float g = 0.f, u = 0.f;
            for (int s = 0; s < splits; ++s) {
                g += a.part[(size_t)s * MN + 2 * p];
                u += a.part[(size_t)s * MN + 2 * p + 1];
            }
            a.C[p] = silu_g(g) * u;  // row-major [M, N/2]: pair p of the flattened [M, N]
        }
    } else {
        for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < MN; o += stride) {
            float v = 0.f;
            for (int s = 0; s < splits; ++s) v += a.part[(size_t)s * MN + o];
            a.C[o] = (EPI == EPI_RESIDUAL) ? a.residual[o] + v : v;
        }
    }
}

// Any K / alignment: one thread per output element.
template <bool BF16>
__global__ __launch_bounds__(256) void gemm_generic_kernel(GemmArgs a) {
    const size_t total = (size_t)a.M * a.N;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += stride) {
        const int m = (int)(o / a.N), n = (int)(o % a.N);
        float acc = 0.f;
        for (int k = 0; k < a.K; ++k) {
            const float w = BF16 ? __uint_as_float((unsigned int)((const uint16_t *)a.W)[(size_t)n * a.K + k] << 16)
                                 : ((const float *)a.W)[(size_t)n * a.K + k];
            acc = fmaf(a.A[(size_t)m * a.K + k], w, acc);
        }
        a.C[o] = acc;
    }
}

template <bool BF16>
static void launch_gemm_epi(const GemmArgs &a, dim3 grid, hipStream_t s) {
    if (grid.z > 1) {
        hipLaunchKernelGGL((gemm_mfma_kernel<BF16, EPI_STORE, true>), grid, dim3(256), 0, s, a);
        return;
    }
    switch (a.epi) {
        case EPI_STORE: hipLaunchKernelGGL((gemm_mfma_kernel<BF16, EPI_STORE, false>), grid, dim3(256), 0, s, a); break;
        case EPI_RESIDUAL: hipLaunchKernelGGL((gemm_mfma_kernel<BF16, EPI_RESIDUAL, false>), grid, dim3(256), 0, s, a); break;
        default: hipLaunchKernelGGL((gemm_mfma_kernel<BF16, EPI_SWIGLU, false>), grid, dim3(256), 0, s, a); break;
    }
}

static void launch_gemm_reduce(const GemmArgs &a, int splits, int blocks, hipStream_t s) {
    switch (a.epi) {
        case EPI_STORE: hipLaunchKernelGGL(gemm_reduce_kernel<EPI_STORE>, dim3(blocks), dim3(256), 0, s, a, splits); break;
        case EPI_RESIDUAL: hipLaunchKernelGGL(gemm_reduce_kernel<EPI_RESIDUAL>, dim3(blocks), dim3(256), 0, s, a, splits); break;
        default: hipLaunchKernelGGL(gemm_reduce_kernel<EPI_SWIGLU>, dim3(blocks), dim3(256), 0, s, a, splits); break;
    }
}

// K splits for a tile grid that does not fill the chip: enough workgroups for two per compute
// unit, at least four 32-deep slices each, partial tiles within the workspace limit.
static int gemm_splits(const lumen_ctx *ctx, const GemmArgs &a) {
    const long tiles = (long)((a.N + BN - 1) / BN) * ((a.M + BM - 1) / BM);
    const long want = 2L * ctx->num_cus;
    if (tiles >= want) return 1;
    long s = (want + tiles - 1) / tiles;
    const long max_by_k = a.K / (4 * BK);
    if (s > max_by_k) s = max_by_k;
    if (s > 16) s = 16;
    while (s > 1 && (size_t)s * a.M * a.N * sizeof(float) > ((size_t)256 << 20)) --s;
    return s < 1 ? 1 : (int)s;
}

int launch_gemm(lumen_ctx *ctx, const GemmArgs &a) {
    if (a.M <= 0 || a.N <= 0) return LUMEN_OK;
    const bool aligned = (((uintptr_t)a.A | (uintptr_t)a.W) & 15) == 0;
    const bool fast = (a.K % 4 == 0) && aligned && a.K > 0;
    if (!fast) {
        if (a.epi != EPI_STORE) LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "fused GEMM needs K %% 4 == 0 and 16-byte alignment (K=%d)", a.K);
        size_t blocks = ((size_t)a.M * a.N + 255) / 256;
        if (blocks > (size_t)ctx->num_cus * 16) blocks = (size_t)ctx->num_cus * 16;
        if (a.w_bf16)
            hipLaunchKernelGGL(gemm_generic_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a);
        else
            hipLaunchKernelGGL(gemm_generic_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, a);
        LUMEN_CHECK_LAUNCH();
        return LUMEN_OK;
    }
    if (a.epi == EPI_SWIGLU && (a.N & 1)) LUMEN_FAIL(LUMEN_ERR_SHAPE, "SwiGLU epilogue needs an even column count, got %d", a.N);
    GemmArgs g = a;
    const int splits = gemm_splits(ctx, a);
    if (splits > 1) {
        const size_t need = (size_t)splits * a.M * a.N * sizeof(float);
        if (ctx->gemm_ws_bytes < need) {
            HIP_TRY(hipStreamSynchronize(ctx->stream));
            if (ctx->gemm_ws) hipFree(ctx->gemm_ws);
            ctx->gemm_ws = nullptr;
            ctx->gemm_ws_bytes = 0;
            HIP_TRY(hipMalloc((void **)&ctx->gemm_ws, need));
            ctx->gemm_ws_bytes = need;
        }
        g.part = ctx->gemm_ws;
    }
    dim3 grid((a.N + BN - 1) / BN, (a.M + BM - 1) / BM, splits);
    if (a.w_bf16) launch_gemm_epi<true>(g, grid, ctx->stream);
    else launch_gemm_epi<false>(g, grid, ctx->stream);
    LUMEN_CHECK_LAUNCH();
    if (splits > 1) {
        size_t blocks = ((size_t)a.M * a.N + 255) / 256;
        if (blocks > (size_t)ctx->num_cus * 8) blocks = (size_t)ctx->num_cus * 8;
        launch_gemm_reduce(g, splits, (int)blocks, ctx->stream);
        LUMEN_CHECK_LAUNCH();
    }
    return LUMEN_OK;
}

static int check_gemm(lumen_ctx *ctx, const void *A, const void *W, const void *C, int M, int N, int K) {
    if (!ctx || !A || !W || !C) LUMEN_FAIL(LUMEN_ERR_INVALID, "gemm: null argument");
    if (M < 0 || N < 0 || K < 0) LUMEN_FAIL(LUMEN_ERR_SHAPE, "gemm: negative dimension");
    return LUMEN_OK;
}

extern "C" int lumen_gemm_f32(lumen_ctx *ctx, const float *A, const float *W, float *C, int M, int N, int K) {
    LUMEN_TRY(check_gemm(ctx, A, W, C, M, N, K));
    GemmArgs a = {};
    a.A = A; a.W = W; a.C = C; a.M = M; a.N = N; a.K = K; a.w_bf16 = 0; a.epi = EPI_STORE;
    return launch_gemm(ctx, a);
}

extern "C" int lumen_gemm_bf16w(lumen_ctx *ctx, const float *A, const uint16_t *W, float *C, int M, int N, int K) {
    LUMEN_TRY(check_gemm(ctx, A, W, C, M, N, K));
    GemmArgs a = {};
    a.A = A; a.W = W; a.C = C; a.M = M; a.N = N; a.K = K; a.w_bf16 = 1; a.epi = EPI_STORE;
    return launch_gemm(ctx, a);
}
