// Dense C[M,N] = A[M,K] W[N,K]^T for the M > 1 (prompt prefill) branch of
// ops::matmul::matmul, src/ops/matmul.rs:70-92, on the gfx950 matrix cores.
//
// fp32 throughout: v_mfma_f32_32x32x2_f32 takes one f32 of A and one of W per
// lane and accumulates a 32x32 tile in 16 registers per lane, so the result
// carries full fp32 precision (the reference computes in f32 on the CPU).
// bf16-stored weights are widened while they are staged into LDS, which is
// the reference's own load-time upcast (src/loader.rs:58) moved to the device.
//
// Workgroup = 4 wavefronts (2x2), 128x128 output tile, 16-deep K slices staged
// k-major in LDS so that the per-instruction operand reads are conflict-free.
#include "internal.h"

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

#define BM 128
#define BN 128
#define BK 16
#define LDT (BM + 4)

__device__ __forceinline__ float silu_g(float g) {
    const float sig = 1.0f / (1.0f + expf(-g));
    return g * sig;
}

template <bool BF16, int EPI>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(GemmArgs a) {
    __shared__ float As[BK][LDT];
    __shared__ float Ws[BK][LDT];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int bm = blockIdx.y * BM, bn = blockIdx.x * BN;
    const int M = a.M, N = a.N, K = a.K;
    const float *A = a.A;

    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
        // stage: 128 rows x 16 k of A and of W, two 4-element pieces per thread each
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int idx = tid + i * 256;
            const int row = idx >> 2, k4 = (idx & 3) * 4;
            v4f va = {0.f, 0.f, 0.f, 0.f}, vw = {0.f, 0.f, 0.f, 0.f};
            if (k0 + k4 < K) {
                if (bm + row < M) va = *(const v4f *)(A + (size_t)(bm + row) * K + k0 + k4);
                if (bn + row < N) {
                    if (BF16) {
                        const v2u raw = *(const v2u *)((const uint16_t *)a.W + (size_t)(bn + row) * K + k0 + k4);
                        vw.x = __uint_as_float(raw.x << 16);
                        vw.y = __uint_as_float(raw.x & 0xffff0000u);
                        vw.z = __uint_as_float(raw.y << 16);
                        vw.w = __uint_as_float(raw.y & 0xffff0000u);
                    } else {
                        vw = *(const v4f *)((const float *)a.W + (size_t)(bn + row) * K + k0 + k4);
                    }
                }
            }
            As[k4 + 0][row] = va.x; As[k4 + 1][row] = va.y; As[k4 + 2][row] = va.z; As[k4 + 3][row] = va.w;
            Ws[k4 + 0][row] = vw.x; Ws[k4 + 1][row] = vw.y; Ws[k4 + 2][row] = vw.z; Ws[k4 + 3][row] = vw.w;
        }
        __syncthreads();
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
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = bm + wm * 64 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                const int col = bn + wn * 64 + j * 32 + (lane & 31);
                const float v = acc[i][j][r];
                if (EPI == EPI_SWIGLU) {
                    // columns (2c, 2c+1) = (gate_c, up_c): silu(gate) * up, src/models/llama.rs:60-63
                    const float up = __shfl_xor(v, 1, 64);
                    if (!(col & 1) && row < M && col < N) a.C[(size_t)row * (N >> 1) + (col >> 1)] = silu_g(v) * up;
                } else if (row < M && col < N) {
                    const size_t o = (size_t)row * N + col;
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
    switch (a.epi) {
        case EPI_STORE: hipLaunchKernelGGL((gemm_mfma_kernel<BF16, EPI_STORE>), grid, dim3(256), 0, s, a); break;
        case EPI_RESIDUAL: hipLaunchKernelGGL((gemm_mfma_kernel<BF16, EPI_RESIDUAL>), grid, dim3(256), 0, s, a); break;
        default: hipLaunchKernelGGL((gemm_mfma_kernel<BF16, EPI_SWIGLU>), grid, dim3(256), 0, s, a); break;
    }
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
    dim3 grid((a.N + BN - 1) / BN, (a.M + BM - 1) / BM);
    if (a.w_bf16) launch_gemm_epi<true>(a, grid, ctx->stream);
    else launch_gemm_epi<false>(a, grid, ctx->stream);
    LUMEN_CHECK_LAUNCH();
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
