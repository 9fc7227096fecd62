// Dense C[M,N] = A[M,K] W[N,K]^T for the M > 1 (prompt prefill) branch of
// ops::matmul::matmul, src/ops/matmul.rs:70-92, on the gfx950 matrix cores.
//
// The reference computes in f32.  The f32 matrix instruction (v_mfma_f32_32x32x2_f32) runs at 1/16
// of the bf16 rate on this chip, so the product is taken on the bf16 matrix cores instead without
// giving up f32 accuracy: an f32 value is the exact sum of three bf16 values (8 + 8 + 8 mantissa
// bits: take the upper 16 bits, subtract, repeat), so x * w is the sum of the products of their
// parts; the six products whose orders add up to at most four carry everything down to 2^-24 of
// the result and are accumulated in f32 by v_mfma_f32_32x32x16_bf16.  A bf16-stored weight (the
// reference widens those at load time, src/loader.rs:58) is a single part: three products.
// Six bf16 instructions of depth 16 against eight f32 instructions of depth 2 per 16 columns of K:
// 2.6x the f32 matrix rate for f32 weights, 5.3x for bf16 weights; measured against an fp64
// product the error is the same as with the f32 instruction (2e-7 .. 2e-6 of the largest element).
//
// Two tile shapes: 128x128 (two or three workgroups per compute unit) for prompts of up to about a
// thousand rows, 256x256 (one workgroup per compute unit, 4x4 register tiles) above; two kernels: a plain
// one (any K that is a multiple of the 16-byte piece; bf16-stored weights at 128x128) and a pipelined one.  When the tile grid alone
// cannot fill the chip (prompt of a few hundred tokens against a 2048-row weight, or 128 large tiles
// on 256 compute units) the K range is split over gridDim.z; each split writes its partial tile to
// a workspace and a second kernel adds the splits in index order and applies the epilogue, so the
// result does not depend on scheduling.
#include "internal.h"
#include "wave_reduce.h"
#include "stage_times.h"

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef unsigned int v2u __attribute__((ext_vector_type(2)));

#define BM 128
#define BN 128
#define BK 32
#define STAGE 4  // 16-byte pieces of A and of W per thread per slice: 128 rows x 32 k / 256 threads

__device__ __forceinline__ float silu_g(float g) {
    const float sig = 1.0f / (1.0f + expf(-g));
    return g * sig;
}

// The 2x2 accumulator tiles of one wavefront to memory.  Accumulator register r of lane l holds
// C[row = 8*(r/4) + 4*(l/32) + r%4][col = l%32] of its 32x32 tile.
template <int EPI, bool PARTIAL>
__device__ __forceinline__ void store_tile(const GemmArgs &a, const v16f (&acc)[2][2], int bm, int bn, int wm, int wn,
                                           int lane) {
    const int M = a.M, N = a.N;
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

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// LDS rows hold the 32 bf16 of a slice (64 bytes, no padding) as four 16-byte chunks; chunk q of row r sits
// at position q ^ ((r >> 1) & 3).  Even rows start at bank 0, odd rows at bank 16, so the 16-byte operand
// reads of 8 neighbouring rows (same chunk index) and the 8-byte staging writes of two neighbouring rows
// each cover all 32 banks exactly once.
#define XROW 32
__device__ __forceinline__ int lds_col(int row, int k) { return ((((k >> 3) ^ (row >> 1)) & 3) << 3) | (k & 7); }

// upper halves of (odd, even) as one dword: two bf16 values, the even one in the low half
__device__ __forceinline__ unsigned pack_hi(float odd, float even) {
    return __builtin_amdgcn_perm(__float_as_uint(odd), __float_as_uint(even), 0x07060302u);
}

// x[0..3] -> three planes of 4 bf16 (2 dwords each): x = p0 + p1 + p2 up to 2^-24 |x|
__device__ __forceinline__ void split3(const v4f x, v2u (&plane)[3]) {
    float r[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int p = 0; p < 3; ++p) {
        plane[p].x = pack_hi(r[1], r[0]);
        plane[p].y = pack_hi(r[3], r[2]);
        if (p < 2) {
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] -= __uint_as_float(__float_as_uint(r[e]) & 0xffff0000u);
        }
    }
}

// Workgroup = 4 wavefronts (2x2), 128x128 output tile, 32-deep slices: the raw values of the next
// slice are in flight from memory during the matrix instructions of the current one, then split
// into their bf16 parts on the way into LDS ([part][row][k], k contiguous: an operand is one
// 16-byte LDS read).  Two workgroups share a compute unit, one computing while the other stages.
template <bool WBF16, int EPI, bool PARTIAL>
__global__ __launch_bounds__(256) void gemm_bf16x3_kernel(GemmArgs a) {
    constexpr int PW = WBF16 ? 1 : 3;       // bf16 parts of a weight
    constexpr int WST = WBF16 ? 2 : STAGE;  // 16-byte pieces of W per thread per slice
    __shared__ __align__(16) uint16_t As[3][BM][XROW];
    __shared__ __align__(16) uint16_t Ws[PW][BN][XROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int bm = blockIdx.y * BM, bn = blockIdx.x * BN;
    const int M = a.M, N = a.N, K = a.K;
    const float *A = a.A;
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

    v4f va[STAGE];
    v4u vw[WST];  // f32 weights: 4 floats; bf16 weights: 8 values
    // A and f32 W: piece i of this thread is row (tid + 256 i) / 8, k offset 4 * ((tid + 256 i) % 8);
    // bf16 W: row (tid + 256 i) / 4, k offset 8 * ((tid + 256 i) % 4)
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < STAGE; ++i) {
            const int idx = tid + i * 256;
            const int row = idx >> 3, k4 = (idx & 7) * 4;
            va[i] = (v4f){0.f, 0.f, 0.f, 0.f};
            if (k0 + k4 < ke && bm + row < M) va[i] = *(const v4f *)(A + (size_t)(bm + row) * K + k0 + k4);
        }
#pragma unroll
        for (int i = 0; i < WST; ++i) {
            const int idx = tid + i * 256;
            const int row = WBF16 ? idx >> 2 : idx >> 3, kk = WBF16 ? (idx & 3) * 8 : (idx & 7) * 4;
            vw[i] = (v4u){0u, 0u, 0u, 0u};
            if (k0 + kk < ke && bn + row < N) {  // K % 8 == 0 (bf16) / K % 4 == 0: a piece is inside or outside as a whole
                if (WBF16) vw[i] = *(const v4u *)((const uint16_t *)a.W + (size_t)(bn + row) * K + k0 + kk);
                else vw[i] = *(const v4u *)((const float *)a.W + (size_t)(bn + row) * K + k0 + kk);
            }
        }
    };

    if (kb < ke) fetch(kb);
    const int c = lane & 31, g8 = (lane >> 5) * 8;
    for (int k0 = kb; k0 < ke; k0 += BK) {
#pragma unroll
        for (int i = 0; i < STAGE; ++i) {
            const int idx = tid + i * 256;
            v2u pl[3];
            split3(va[i], pl);
#pragma unroll
            for (int p = 0; p < 3; ++p) *(v2u *)&As[p][idx >> 3][lds_col(idx >> 3, (idx & 7) * 4)] = pl[p];
        }
#pragma unroll
        for (int i = 0; i < WST; ++i) {
            const int idx = tid + i * 256;
            if (WBF16) {
                *(v4u *)&Ws[0][idx >> 2][lds_col(idx >> 2, (idx & 3) * 8)] = vw[i];
            } else {
                v2u pl[3];
                split3((v4f){__uint_as_float(vw[i].x), __uint_as_float(vw[i].y), __uint_as_float(vw[i].z),
                             __uint_as_float(vw[i].w)}, pl);
#pragma unroll
                for (int p = 0; p < PW; ++p) *(v2u *)&Ws[p][idx >> 3][lds_col(idx >> 3, (idx & 7) * 4)] = pl[p];
            }
        }
        __syncthreads();
        if (k0 + BK < ke) fetch(k0 + BK);  // in flight during the matrix instructions below
#pragma unroll
        for (int ks = 0; ks < BK; ks += 16) {
            // lane (c, g): 8 consecutive k of row c -- the same k for both operands
            bf16x8 af[2][3], wf[2][PW];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int p = 0; p < 3; ++p)
                    af[i][p] = __builtin_bit_cast(bf16x8, *(const v4u *)&As[p][wm * 64 + i * 32 + c][lds_col(c, ks + g8)]);
#pragma unroll
                for (int p = 0; p < PW; ++p)
                    wf[i][p] = __builtin_bit_cast(bf16x8, *(const v4u *)&Ws[p][wn * 64 + i * 32 + c][lds_col(c, ks + g8)]);
            }
            // products by ascending size; the four tiles take turns, so consecutive matrix
            // instructions never wait on each other's accumulator
            constexpr int NPROD = WBF16 ? 3 : 6;
            constexpr int PA_[6] = {2, 0, 1, 1, 0, 0}, PW_[6] = {0, 2, 1, 0, 1, 0};  // f32 weights: a2w0 a0w2 a1w1 a1w0 a0w1 a0w0
#pragma unroll
            for (int q = 0; q < NPROD; ++q) {
                const int xa = WBF16 ? 2 - q : PA_[q], xw = WBF16 ? 0 : PW_[q];
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i][xa], wf[j][xw], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
    }
    store_tile<EPI, PARTIAL>(a, acc, bm, bn, wm, wn, lane);
}

// The pipelined kernel: F x F tiles of 32x32 per wavefront, 2 x 2 wavefronts, 16-deep slices, LDS
// double-buffered.  The split of slice s+1 into the other LDS half stands in the same block as the matrix
// instructions of slice s, one bf16 plane of one 16-byte piece ("plane step") after every F of them, and
// runs in their shadow; slice s+2 travels from memory meanwhile; one barrier per slice.  In LDS the two k halves
// of a slice lie in planes of their own, [k half][row][8 bf16]: 8 neighbouring lanes of an operand read (8 rows, one
// half) take 128 contiguous bytes (with the halves side by side in 32-byte rows a third of the LDS cycles of this
// kernel were bank conflicts).
//   F = 4: 256x256 output tile, all 256 accumulator registers of a wavefront, one workgroup per compute
//          unit.  A 4x4 register tile reads half the LDS bytes per matrix instruction of a 2x2 one, which
//          is what bounds gemm_bf16x3_kernel.  For thousands of prompt rows.
//   F = 2: 128x128, two or three workgroups per compute unit: the tile grid and K splits of
//          gemm_bf16x3_kernel, for shorter prompts with f32 weights.
#define GB_M 256  // the F = 4 tile
#define GB_N 256
#define GB_K 16   // slice depth of the pipelined kernel

template <int EPI, bool PARTIAL, int F>
__device__ __forceinline__ void store_wave_tiles(const GemmArgs &a, const v16f (&acc)[F][F], int bm, int bn, int wm, int wn,
                                               int lane) {
    const int M = a.M, N = a.N;
    float *part = PARTIAL ? a.part + (size_t)blockIdx.z * M * N : nullptr;
#pragma unroll
    for (int i = 0; i < F; ++i)
#pragma unroll
        for (int j = 0; j < F; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = bm + wm * (F * 32) + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                const int col = bn + wn * (F * 32) + j * 32 + (lane & 31);
                const float v = acc[i][j][r];
                if (PARTIAL) {
                    if (row < M && col < N) part[(size_t)row * N + col] = v;
                } else if (EPI == EPI_SWIGLU) {
                    const float up = __shfl_xor(v, 1, 64);
                    if (!(col & 1) && row < M && col < N) a.C[(size_t)row * (N >> 1) + (col >> 1)] = silu_g(v) * up;
                } else if (row < M && col < N) {
                    const size_t o = (size_t)row * N + col;
                    a.C[o] = (EPI == EPI_RESIDUAL) ? a.residual[o] + v : v;
                }
            }
}

template <bool WBF16, int EPI, bool PARTIAL, int F>
__global__ __launch_bounds__(256, (F == 4 ? 1 : 2)) void gemm_bf16x3_tile_kernel(GemmArgs a) {
    constexpr int PW = WBF16 ? 1 : 3;
    constexpr int TM = 64 * F, TN = 64 * F;
    constexpr int AST = F;                    // 16-byte pieces of A per thread per slice: TM rows x 16 k / 256 threads
    constexpr int WST = WBF16 ? F / 2 : F;
    // [half][part][k half g][row][8 bf16]: the 8 k of an operand lane are one 16-byte unit, units of neighbouring rows
    // are neighbours, so the 8 lanes of an LDS pass (8 rows, one g) read 128 contiguous bytes; the two k halves are
    // 64 bytes further apart than a power of two (LPAD rows), so that a staging write of 4 rows x 2 halves x 2 pieces
    // covers all banks once.
    constexpr int LPAD = 4;
    __shared__ __align__(16) uint16_t As[2][3][2][TM + LPAD][8];
    __shared__ __align__(16) uint16_t Ws[2][PW][2][TN + LPAD][8];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int bm = blockIdx.y * TM, bn = blockIdx.x * TN;
    const int M = a.M, N = a.N, K = a.K;
    const float *A = a.A;
    // this workgroup's share of K: whole slices, [kb, ke)
    const int slices = K / GB_K;
    const int per = (slices + (int)gridDim.z - 1) / (int)gridDim.z;
    const int kb = min((int)blockIdx.z * per, slices) * GB_K;
    const int ke = min(K, kb + per * GB_K);

    v16f acc[F][F];
#pragma unroll
    for (int i = 0; i < F; ++i)
#pragma unroll
        for (int j = 0; j < F; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    v4f va[AST];
    v4u vw[WST];
    // A and f32 W: piece i of this thread is row (tid + 256 i) / 4, k offset 4 * ((tid + 256 i) % 4);
    // bf16 W: row (tid + 256 i) / 2, k offset 8 * ((tid + 256 i) % 2).  No branches: K is a multiple of
    // the slice, rows past the end are clamped to the last one (their products are never stored).
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < AST; ++i) {
            const int idx = tid + i * 256;
            const int row = min(bm + (idx >> 2), M - 1), k4 = (idx & 3) * 4;
            va[i] = *(const v4f *)(A + (size_t)row * K + k0 + k4);
        }
#pragma unroll
        for (int i = 0; i < WST; ++i) {
            const int idx = tid + i * 256;
            const int row = min(bn + (WBF16 ? idx >> 1 : idx >> 2), N - 1), kk = WBF16 ? (idx & 1) * 8 : (idx & 3) * 4;
            if (WBF16) vw[i] = *(const v4u *)((const uint16_t *)a.W + (size_t)row * K + k0 + kk);
            else vw[i] = *(const v4u *)((const float *)a.W + (size_t)row * K + k0 + kk);
        }
    };
    // Staging the fetched slice into LDS half b is a sequence of "plane steps": plane 0, 1, 2 of A piece 0,
    // of A piece 1, ..., then (f32 weights) of the W pieces; a bf16 weight piece is copied along with the
    // first steps.  ra is what is left of the piece being split.
    constexpr int NPROD = WBF16 ? 3 : 6;      // products per k: groups of F matrix instructions per column tile
    constexpr int NSTEP = 3 * AST + (WBF16 ? 0 : 3 * WST);
    static_assert(NSTEP == F * NPROD, "one plane step per group of matrix instructions");
    float ra[4];
    auto plane_step = [&](int b, int u) {
        const bool isw = u >= 3 * AST;
        const int pc = (isw ? u - 3 * AST : u) / 3, p = u % 3, idx = tid + pc * 256;
        if (p == 0) {
            if (isw) {
                const v4u w = vw[WBF16 ? 0 : pc];
                ra[0] = __uint_as_float(w.x); ra[1] = __uint_as_float(w.y);
                ra[2] = __uint_as_float(w.z); ra[3] = __uint_as_float(w.w);
            } else {
                ra[0] = va[pc].x; ra[1] = va[pc].y; ra[2] = va[pc].z; ra[3] = va[pc].w;
            }
        }
        if (WBF16 && u < WST) *(v4u *)&Ws[b][0][tid & 1][(tid + u * 256) >> 1][0] = vw[u < WST ? u : 0];
        uint16_t *dst = isw ? &Ws[b][p][(idx & 3) >> 1][idx >> 2][(idx & 1) * 4] : &As[b][p][(idx & 3) >> 1][idx >> 2][(idx & 1) * 4];
        *(v2u *)dst = (v2u){pack_hi(ra[1], ra[0]), pack_hi(ra[3], ra[2])};
        if (p < 2) {
#pragma unroll
            for (int e = 0; e < 4; ++e) ra[e] -= __uint_as_float(__float_as_uint(ra[e]) & 0xffff0000u);
        }
    };
    const int c = lane & 31, gk = lane >> 5;
    // The matrix instructions of the slice in LDS half b.  With with_stage the next slice is split into the
    // other half between them, a plane step after every F matrix instructions, so that the vector ALU works
    // in their shadow.
    auto mma = [&](int b, bool with_stage) {
        constexpr int PA_[6] = {2, 0, 1, 1, 0, 0}, PW_[6] = {0, 2, 1, 0, 1, 0};
        bf16x8 af[F][3];
#pragma unroll
        for (int i = 0; i < F; ++i)
#pragma unroll
            for (int p = 0; p < 3; ++p)
                af[i][p] = __builtin_bit_cast(bf16x8, *(const v4u *)&As[b][p][gk][wm * (F * 32) + i * 32 + c][0]);
#pragma unroll
        for (int j = 0; j < F; ++j) {
            bf16x8 wf[PW];
#pragma unroll
            for (int p = 0; p < PW; ++p)
                wf[p] = __builtin_bit_cast(bf16x8, *(const v4u *)&Ws[b][p][gk][wn * (F * 32) + j * 32 + c][0]);
#pragma unroll
            for (int q = 0; q < NPROD; ++q) {
                const int xa = WBF16 ? 2 - q : PA_[q], xw = WBF16 ? 0 : PW_[q];
#pragma unroll
                for (int i = 0; i < F; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i][xa], wf[xw], acc[i][j], 0, 0, 0);
                if (with_stage) {
                    plane_step(b ^ 1, j * NPROD + q);
                    if (F == 4) {
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one matrix instruction,
                            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);  // three vector ALU instructions in its shadow
                        }
                    } else {
#pragma unroll
                        for (int g = 0; g < 2; ++g) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
                        }
                    }
                    __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);          // the plane's LDS write
                }
            }
        }
    };

    // slice s is multiplied from LDS half s & 1 while slice s+1 is split into the other half (last read
    // before the barrier that ended the previous trip) and slice s+2 travels from memory
    if (kb < ke) {
        fetch(kb);
#pragma unroll
        for (int u = 0; u < NSTEP; ++u) plane_step(0, u);
        if (kb + GB_K < ke) fetch(kb + GB_K);
        __syncthreads();
        int k0 = kb, b = 0;
        for (; k0 + 2 * GB_K < ke; k0 += GB_K, b ^= 1) {
            mma(b, true);
            fetch(k0 + 2 * GB_K);
            __syncthreads();
        }
        if (k0 + GB_K < ke) {
            mma(b, true);
            __syncthreads();
            b ^= 1;
        }
        mma(b, false);
    }
    store_wave_tiles<EPI, PARTIAL, F>(a, acc, bm, bn, wm, wn, lane);
}

// Prompts of two rows (up to four where GEMM_SKINNY_MAX_M is raised): the product is bound by the weights,
// which the tile kernels above cannot stream at anything like the memory's rate (they take 100 us per layer whatever M
// is).  This kernel walks W the way the single-row product does: a wavefront takes units of two whole rows, lanes across
// K with 16-byte loads, in pieces of 4 sweeps x 2 rows = 8 loads per lane, two pieces in flight and the next one
// requested as soon as a register set is free, unit after unit.  Every piece is multiplied with MS rows of A at once:
// plain f32 multiply-adds in the lanes, a wavefront reduction per (row of A, row of W) when a unit is complete -- the
// accumulation order of the single-row product (src/ops/matmul.rs:42-69 applied to each row of A).  The MS rows of A
// lie in LDS for the whole launch, staged once per workgroup (K padded with zeros to whole pieces); more rows of A than
// MS: tiles of MS over gridDim.y (W is then streamed once per tile).
#define SK_WAVES 4  // (8 wavefronts per workgroup leave a round of workgroups uneven over the compute units: 1.48 against 1.44 ms)
#define SK_THREADS (SK_WAVES * 64)
template <int MS, bool BF16, int EPI>
__global__ __launch_bounds__(SK_THREADS) void gemm_skinny_kernel(GemmArgs a, int kpad) {
    constexpr int VEC = BF16 ? 8 : 4;          // elements per 16-byte load
    constexpr int SWEEP = 64 * VEC;            // elements of a row one wavefront covers per load
    constexpr int R = 2, U = 4;
    constexpr int PIECE = SWEEP * U;
    constexpr int ESZ = BF16 ? 2 : 4;
    LUMEN_DYNAMIC_LDS(float, As);  // [MS][kpad]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int M = a.M, N = a.N, K = a.K;
    const int m0 = blockIdx.y * MS;
    const int nunits = (N + R - 1) / R;
    const int gw = blockIdx.x * SK_WAVES + wave, nw = gridDim.x * SK_WAVES;
    const char *Wb = (const char *)a.W;
    const size_t row_bytes = (size_t)K * ESZ;

    // every load is issued unconditionally: positions past the end of a row are clamped to its last 16 bytes (they meet
    // the zero padding of A), a row past N to row N-1 (not stored)
    auto load_piece = [&](int u, int k0, v4u (&raw)[R][U]) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const char *rp = Wb + (size_t)min(u * R + r, N - 1) * row_bytes;
#pragma unroll
            for (int uu = 0; uu < U; ++uu) {
                const int kk = min(k0 + uu * SWEEP + lane * VEC, K - VEC);
                raw[r][uu] = __builtin_nontemporal_load((const v4u *)(rp + (size_t)kk * ESZ));
            }
        }
    };
    const int np = kpad / PIECE;
    int lu = gw, lk = 0;  // unit / element offset of the next piece to load
    auto advance_load = [&]() __attribute__((always_inline)) {
        lk += PIECE;
        if (lk >= kpad) {
            lk = 0;
            lu += nw;
        }
    };
    const int my_units = (nunits > gw) ? (nunits - gw + nw - 1) / nw : 0;
    const int T = my_units * np;
    // the first weights are on their way before A is staged: they do not depend on it
    v4u rawA[R][U], rawB[R][U];
    load_piece(min(lu, nunits - 1), lk, rawA);
    advance_load();
    if (T > 1) {
        load_piece(lu, lk, rawB);
        advance_load();
    }
    for (int i = tid * 4; i < MS * kpad; i += SK_THREADS * 4) {
        const int m = i / kpad, k = i - m * kpad;
        v4f v = {0.f, 0.f, 0.f, 0.f};
        if (m0 + m < M && k < K) v = *(const v4f *)(a.A + (size_t)(m0 + m) * K + k);  // K % 4 == 0
        *(v4f *)&As[i] = v;
    }
    __syncthreads();

    float acc[R][MS];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int m = 0; m < MS; ++m) acc[r][m] = 0.f;
    int u = gw, k0 = 0;  // unit / element offset of the piece being multiplied
    auto consume = [&](const v4u (&raw)[R][U]) __attribute__((always_inline)) {
#pragma unroll
        for (int uu = 0; uu < U; ++uu) {
            const int kl = k0 + uu * SWEEP + lane * VEC;
#pragma unroll
            for (int m = 0; m < MS; ++m) {
                const v4f x0 = *(const v4f *)&As[m * kpad + kl];
                v4f x1 = x0;
                if (BF16) x1 = *(const v4f *)&As[m * kpad + kl + 4];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const v4u w = raw[r][uu];
                    float s = acc[r][m];
                    if (BF16) {  // eight bf16 values, widened by a shift (src/loader.rs:58)
                        s = fmaf(__uint_as_float(w.x << 16), x0.x, s);
                        s = fmaf(__uint_as_float(w.x & 0xffff0000u), x0.y, s);
                        s = fmaf(__uint_as_float(w.y << 16), x0.z, s);
                        s = fmaf(__uint_as_float(w.y & 0xffff0000u), x0.w, s);
                        s = fmaf(__uint_as_float(w.z << 16), x1.x, s);
                        s = fmaf(__uint_as_float(w.z & 0xffff0000u), x1.y, s);
                        s = fmaf(__uint_as_float(w.w << 16), x1.z, s);
                        s = fmaf(__uint_as_float(w.w & 0xffff0000u), x1.w, s);
                    } else {
                        s = fmaf(__uint_as_float(w.x), x0.x, s);
                        s = fmaf(__uint_as_float(w.y), x0.y, s);
                        s = fmaf(__uint_as_float(w.z), x0.z, s);
                        s = fmaf(__uint_as_float(w.w), x0.w, s);
                    }
                    acc[r][m] = s;
                }
            }
        }
        k0 += PIECE;
        if (k0 >= kpad) {  // unit complete
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int m = 0; m < MS; ++m) acc[r][m] = wave_sum(acc[r][m]);
            if (lane == 0) {
                const int row = u * R;
#pragma unroll
                for (int m = 0; m < MS; ++m) {
                    if (m0 + m >= M) continue;
                    const size_t mrow = (size_t)(m0 + m);
                    if (EPI == EPI_SWIGLU) {
                        // rows (2u, 2u + 1) hold (gate_u, up_u): silu(gate) * up, src/models/llama.rs:60-63
                        if (row + 1 < N) a.C[mrow * (N >> 1) + u] = silu_g(acc[0][m]) * acc[1][m];
                    } else {
#pragma unroll
                        for (int r = 0; r < R; ++r)
                            if (row + r < N) {
                                const size_t o = mrow * N + row + r;
                                a.C[o] = (EPI == EPI_RESIDUAL) ? a.residual[o] + acc[r][m] : acc[r][m];
                            }
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int m = 0; m < MS; ++m) acc[r][m] = 0.f;
            k0 = 0;
            u += nw;
        }
    };
    for (int t = 0; t < T; t += 2) {
        consume(rawA);
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
}

// Prompts of three to 32 rows (a chat turn's new tokens, the tail of a chunked prompt): the product is bound by the
// weights, and the tile kernels above take the same ~100 us per layer for 5 rows as for 128.  This kernel streams W once
// and multiplies on the matrix cores without sharing anything between wavefronts: a wavefront owns 16 rows of W (a column
// tile of C; N / 16 tiles spread evenly over the compute units where N / 32 would not) over a range of K and all
// MT <= 2 row tiles of 16 rows of A.  It fetches 16 x 32 blocks of W (8 or 16 blocks ahead: 16 KB per wavefront in flight,
// what the single-row product keeps in flight) and 16 x 32 blocks of A (those come from L2) with coalesced 16-byte loads,
// turns them into operand order through a wavefront-private LDS buffer (no barriers) and multiplies with the f32
// matrix instruction (v_mfma_f32_16x16x4_f32: a sixteenth of the bf16 rate, but no splitting into bf16 parts on the
// vector ALU, which is what bounded a bf16-part form of this kernel -- 31 us for the 92 MB gate|up matrix against 25; every
// further row tile costs 20 us per layer in f32 matrix instructions, so beyond 32 rows the tile kernels are as fast).  The four wavefronts of a
// workgroup take consecutive K ranges of ONE column tile and add their accumulators through LDS in wavefront order; ranges
// are split further over gridDim.z like the tile kernels' (partial tiles of M x 16).
#define GS_LD 36  // floats per LDS row of a staged 16 x 32 block: rows start 4 banks apart, 8 rows cover all banks (blocks of
                  // 128 and 256 k -- longer visits to a row of W -- measured no faster: 23.6 and 35 against 24.7 us)
#define GS_DA 2   // blocks of A in flight
typedef float v4acc __attribute__((ext_vector_type(4)));
// BF16: W holds bf16 bits; widened by a shift on the way into the operand registers like src/loader.rs:58 widens them at
// load time, so the products are those of f32 weights with the same values.
template <int MT, bool BF16, int EPI, bool PARTIAL>
__global__ __launch_bounds__(256) void gemm_stream_kernel(GemmArgs a) {
    constexpr int DW = BF16 ? 16 : 8;  // blocks of W in flight per wavefront (16 KB)
    constexpr int WP = BF16 ? 1 : 2;   // 16-byte pieces of a W block per lane
    __shared__ __align__(16) float stage_w[4][16 * GS_LD];
    __shared__ __align__(16) float stage_a[4][MT][16 * GS_LD];
    STAGE_T(0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int bn = blockIdx.x * 16;
    const int M = a.M, N = a.N, K = a.K;
    const float *A = a.A;
    // blocks of 32 k: this workgroup's share [z per_wg, (z + 1) per_wg), this wavefront's quarter of it
    const int nblk = (K + 31) / 32;
    const int per_wg = (nblk + (int)gridDim.z - 1) / (int)gridDim.z;
    const int per_wave = (per_wg + 3) / 4;
    const int wg0 = (int)blockIdx.z * per_wg;
    const int d0 = min(wg0 + wave * per_wave, nblk);
    const int d1 = min(min(d0 + per_wave, wg0 + per_wg), nblk);

    v4acc acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = v4acc{0.f, 0.f, 0.f, 0.f};

    // Piece i (0, 1) of this lane in a 16 x 32 block of f32 values: row 8 i + lane / 8, k offset 4 * (lane % 8) -- the 8
    // lanes of a row read 128 contiguous bytes; a block of bf16 weights is one piece per lane: row lane / 4, k offset
    // 8 * (lane % 4).  K is a multiple of the piece: a piece is inside or outside as a whole.  Rows past the end are
    // clamped (their products are never stored).
    const int arow = lane >> 3, ak = (lane & 7) * 4;
    const int wrow = BF16 ? lane >> 2 : arow, wk = BF16 ? (lane & 3) * 8 : ak;
    const char *wp[WP];
    const float *ap[MT][2];
#pragma unroll
    for (int i = 0; i < WP; ++i)
        wp[i] = (const char *)a.W + ((size_t)min(bn + wrow + 8 * i, N - 1) * K + wk) * (BF16 ? 2 : 4);
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int i = 0; i < 2; ++i) ap[t][i] = A + (size_t)min(t * 16 + arow + 8 * i, M - 1) * K + ak;
    v4u vw[DW][WP];
    v4f va[GS_DA][MT][2];
    auto fetch_w = [&](int slot, int d) {
        const bool in = d * 32 + wk < K;
#pragma unroll
        for (int i = 0; i < WP; ++i) {
            vw[slot][i] = v4u{0u, 0u, 0u, 0u};
            if (in) vw[slot][i] = __builtin_nontemporal_load((const v4u *)(wp[i] + (size_t)d * (BF16 ? 64 : 128)));
        }
    };
    auto fetch_a = [&](int slot, int d) {
        const bool in = d * 32 + ak < K;
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                va[slot][t][i] = v4f{0.f, 0.f, 0.f, 0.f};
                if (in) va[slot][t][i] = *(const v4f *)(ap[t][i] + d * 32);
            }
    };
    float *sw = stage_w[wave];
    auto block = [&](int ws, int as) {
        if (BF16) {  // rows of 36 bf16 (72 bytes): 8-byte accesses
            uint16_t *h = (uint16_t *)sw + wrow * GS_LD + wk;
            *(v2u *)h = v2u{vw[ws][0].x, vw[ws][0].y};
            *(v2u *)(h + 4) = v2u{vw[ws][0].z, vw[ws][0].w};
        } else {
#pragma unroll
            for (int i = 0; i < WP; ++i) *(v4u *)(sw + (wrow + 8 * i) * GS_LD + wk) = vw[ws][i];
        }
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 2; ++i) *(v4f *)(stage_a[wave][t] + (arow + 8 * i) * GS_LD + ak) = va[as][t][i];
        // The buffers are this wavefront's own and its LDS instructions execute in order: the reads below see the
        // writes above without a workgroup barrier (the wave barrier emits no instruction; it keeps the compiler
        // from moving LDS accesses across it).
        __builtin_amdgcn_wave_barrier();
        // lane (c, g) takes the k = 16 j + 4 g + e of row c for both operands: instruction (j, e) multiplies four k
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            v4f wf;
            if (BF16) {
                const v2u r = *(const v2u *)((const uint16_t *)sw + c * GS_LD + j * 16 + g * 4);
                wf = v4f{__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                         __uint_as_float(r.y & 0xffff0000u)};
            } else {
                wf = *(const v4f *)(sw + c * GS_LD + j * 16 + g * 4);
            }
            v4f af[MT];
#pragma unroll
            for (int t = 0; t < MT; ++t) af[t] = *(const v4f *)(stage_a[wave][t] + c * GS_LD + j * 16 + g * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[t][e], wf[e], acc[t], 0, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();  // (the next block's writes come after these reads)
    };
    // block d0 + j of W sits in slot j % DW, of A in slot j % GS_DA (a trip of the loop below is a whole number of turns
    // of both rings); a slot is requested anew as soon as its block is used
    static_assert(DW % GS_DA == 0, "the A ring must divide a trip of the loop");
#pragma unroll
    for (int j = 0; j < DW; ++j)
        if (d0 + j < d1) fetch_w(j, d0 + j);
#pragma unroll
    for (int j = 0; j < GS_DA; ++j)
        if (d0 + j < d1) fetch_a(j, d0 + j);
    STAGE_T(1);
    for (int d = d0; d < d1; d += DW) {
#pragma unroll
        for (int j = 0; j < DW; ++j)
            if (d + j < d1) {
                block(j, j % GS_DA);
                if (d + j + DW < d1) fetch_w(j, d + j + DW);
                if (d + j + GS_DA < d1) fetch_a(j % GS_DA, d + j + GS_DA);
                if (d + j == d0) STAGE_T(2);
                if (d + j == d0 + 7) STAGE_T(3);
            }
    }
    STAGE_T(4);
    // the four K ranges of the workgroup, added in wavefront order
    __syncthreads();
    STAGE_T(5);
    float *red = &stage_w[0][0];  // [3][MT][4][64] floats
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[(((wave - 1) * MT + t) * 4 + r) * 64 + lane] = acc[t][r];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][r] += red[((w * MT + t) * 4 + r) * 64 + lane];
    float *part = PARTIAL ? a.part + (size_t)blockIdx.z * M * N : nullptr;
    const int col = bn + c;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            // accumulator register r of lane (c, g): row 4 g + r of its 16 x 16 tile, column c
            const int row = t * 16 + g * 4 + r;
            const float v = acc[t][r];
            if (PARTIAL) {
                if (row < M && col < N) part[(size_t)row * N + col] = v;
            } else if (EPI == EPI_SWIGLU) {
                const float up = __shfl_xor(v, 1, 64);
                if (!(col & 1) && row < M && col < N) a.C[(size_t)row * (N >> 1) + (col >> 1)] = silu_g(v) * up;
            } else if (row < M && col < N) {
                const size_t o = (size_t)row * N + col;
                a.C[o] = (EPI == EPI_RESIDUAL) ? a.residual[o] + v : v;
            }
        }
    STAGE_T_STORES_DONE(6);
}

#define GEMM_MAX_SPLITS 16
// Adds the K splits of every output element in split order and applies the epilogue.
template <int EPI>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(GemmArgs a, int splits) {
    const size_t MN = (size_t)a.M * a.N;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    if ((MN & 3) == 0 && splits <= GEMM_MAX_SPLITS && ((((uintptr_t)a.C | (uintptr_t)a.residual | (uintptr_t)a.part) & 15) == 0)) {
        // four elements per thread; the partials of all splits are requested before the first is added (one
        // trip to memory instead of one per split), then added in split order as in the scalar loop below
        typedef float v4 __attribute__((ext_vector_type(4)));
        for (size_t q = (size_t)blockIdx.x * blockDim.x + threadIdx.x; q < MN / 4; q += stride) {
            v4 pv[GEMM_MAX_SPLITS];
#pragma unroll
            for (int s = 0; s < GEMM_MAX_SPLITS; ++s)
                if (s < splits) pv[s] = *(const v4 *)(a.part + (size_t)s * MN + 4 * q);
            v4 r4 = {0.f, 0.f, 0.f, 0.f};
            if (EPI == EPI_RESIDUAL) r4 = *(const v4 *)(a.residual + 4 * q);
            v4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < GEMM_MAX_SPLITS; ++s)
                if (s < splits) v += pv[s];
            if (EPI == EPI_SWIGLU) {
                // row-major [M, N/2]: pairs 2q, 2q + 1 of the flattened [M, N]
                a.C[2 * q] = silu_g(v.x) * v.y;
                a.C[2 * q + 1] = silu_g(v.z) * v.w;
            } else if (EPI == EPI_RESIDUAL) {
                *(v4 *)(a.C + 4 * q) = r4 + v;
            } else {
                *(v4 *)(a.C + 4 * q) = v;
            }
        }
        return;
    }
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

// The same for whole rows, with the RMSNorm of the finished row on top: one workgroup per row of C (N <= 4096, a
// multiple of 4); a thread keeps its pieces of the row in registers between the sum of squares and the scaling.
// Splits are added in index order, the sum of squares in the order of rmsnorm_vec_kernel: same bits as the two
// launches it replaces.
#define GEMM_ROW_VPT 4
__global__ __launch_bounds__(256) void gemm_reduce_norm_kernel(GemmArgs a, int splits) {
    typedef float v4 __attribute__((ext_vector_type(4)));
    __shared__ float red[4];
    const int row = blockIdx.x, tid = threadIdx.x, N = a.N;
    const size_t MN = (size_t)a.M * N, base = (size_t)row * N;
    v4 v[GEMM_ROW_VPT], g[GEMM_ROW_VPT];
#pragma unroll
    for (int i = 0; i < GEMM_ROW_VPT; ++i) {
        const int k = (tid + i * 256) * 4;
        v[i] = v4{0.f, 0.f, 0.f, 0.f};
        g[i] = v[i];
        if (k < N) {
            v4 pv[GEMM_MAX_SPLITS];
#pragma unroll
            for (int s = 0; s < GEMM_MAX_SPLITS; ++s)
                if (s < splits) pv[s] = *(const v4 *)(a.part + (size_t)s * MN + base + k);
            const v4 r4 = *(const v4 *)(a.residual + base + k);
            g[i] = *(const v4 *)(a.norm_w + k);
            v4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < GEMM_MAX_SPLITS; ++s)
                if (s < splits) acc += pv[s];
            v[i] = r4 + acc;
            *(v4 *)(a.C + base + k) = v[i];
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < GEMM_ROW_VPT; ++i) {
        ss = fmaf(v[i].x, v[i].x, ss);
        ss = fmaf(v[i].y, v[i].y, ss);
        ss = fmaf(v[i].z, v[i].z, ss);
        ss = fmaf(v[i].w, v[i].w, ss);
    }
    ss = wave_sum(ss);
    if ((tid & 63) == 0) red[tid >> 6] = ss;
    __syncthreads();
    const float tot = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv = 1.0f / sqrtf(tot / (float)N + a.norm_eps);
#pragma unroll
    for (int i = 0; i < GEMM_ROW_VPT; ++i) {
        const int k = (tid + i * 256) * 4;
        if (k < N) {
            v4 r;
            r.x = v[i].x * inv * g[i].x;
            r.y = v[i].y * inv * g[i].y;
            r.z = v[i].z * inv * g[i].z;
            r.w = v[i].w * inv * g[i].w;
            *(v4 *)(a.norm_out + base + k) = r;
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
        hipLaunchKernelGGL((gemm_bf16x3_kernel<BF16, EPI_STORE, true>), grid, dim3(256), 0, s, a);
        return;
    }
    switch (a.epi) {
        case EPI_STORE: hipLaunchKernelGGL((gemm_bf16x3_kernel<BF16, EPI_STORE, false>), grid, dim3(256), 0, s, a); break;
        case EPI_RESIDUAL: hipLaunchKernelGGL((gemm_bf16x3_kernel<BF16, EPI_RESIDUAL, false>), grid, dim3(256), 0, s, a); break;
        default: hipLaunchKernelGGL((gemm_bf16x3_kernel<BF16, EPI_SWIGLU, false>), grid, dim3(256), 0, s, a); break;
    }
}

template <bool BF16, int F>
static void launch_gemm_tile(const GemmArgs &a, dim3 grid, hipStream_t s) {
    if (grid.z > 1) {
        hipLaunchKernelGGL((gemm_bf16x3_tile_kernel<BF16, EPI_STORE, true, F>), grid, dim3(256), 0, s, a);
        return;
    }
    switch (a.epi) {
        case EPI_STORE: hipLaunchKernelGGL((gemm_bf16x3_tile_kernel<BF16, EPI_STORE, false, F>), grid, dim3(256), 0, s, a); break;
        case EPI_RESIDUAL: hipLaunchKernelGGL((gemm_bf16x3_tile_kernel<BF16, EPI_RESIDUAL, false, F>), grid, dim3(256), 0, s, a); break;
        default: hipLaunchKernelGGL((gemm_bf16x3_tile_kernel<BF16, EPI_SWIGLU, false, F>), grid, dim3(256), 0, s, a); break;
    }
}

static void launch_gemm_reduce(const GemmArgs &a, int splits, int blocks, hipStream_t s) {
    switch (a.epi) {
        case EPI_STORE: hipLaunchKernelGGL(gemm_reduce_kernel<EPI_STORE>, dim3(blocks), dim3(256), 0, s, a, splits); break;
        case EPI_RESIDUAL: hipLaunchKernelGGL(gemm_reduce_kernel<EPI_RESIDUAL>, dim3(blocks), dim3(256), 0, s, a, splits); break;
        default: hipLaunchKernelGGL(gemm_reduce_kernel<EPI_SWIGLU>, dim3(blocks), dim3(256), 0, s, a, splits); break;
    }
}

// K splits for a 128x128 tile grid that does not fill the chip.  A compute unit works its workgroups off
// one after the other as far as the matrix pipes are concerned, so what counts is the largest number of
// workgroups any compute unit gets times the length of one: ceil(tiles * s / CUs) * (slices / s + a
// fixed cost per workgroup for its first loads and its partial tile).  88 tiles of 128 slices: s = 6
// makes 528 workgroups -- three for 16 of the compute units -- where s = 5 makes 440, two at most.
// At least 128 of K per split, 16 splits at most, partial tiles within the workspace limit.
static int gemm_splits(const lumen_ctx *ctx, const GemmArgs &a) {
    const long tiles = (long)((a.N + BN - 1) / BN) * ((a.M + BM - 1) / BM);
    const long cus = ctx->num_cus;
    if (tiles * 4 >= 2 * cus * 3) return 1;  // three quarters of two per compute unit: a split would cost more in partial tiles than it gains
    const long slices = (a.K + GB_K - 1) / GB_K;
    const long fixed = 6;  // per workgroup, in slices
    long best = 1, best_cost = 0;
    for (long s = 1; s <= 16; ++s) {
        if (s > 1 && (a.K / s < 4 * BK || (size_t)s * a.M * a.N * sizeof(float) > ((size_t)256 << 20))) break;
        const long per_cu = (tiles * s + cus - 1) / cus;
        // a workgroup alone on its compute unit has nobody to overlap its barriers and first loads with
        const long cost = per_cu * ((slices + s - 1) / s + fixed) * (per_cu == 1 ? 4 : 3);
        if (s == 1 || cost < best_cost) {  // ties: the fewer partial tiles
            best = s;
            best_cost = cost;
        }
    }
    return (int)best;
}

// K splits (1 to 4) for the 256x256 kernel, or 0 where the 128x128 kernel is to run.  The large tile
// pays from about a thousand rows of A on, when its workgroups -- one per compute unit at a time --
// come in nearly whole rounds: the smallest split that fills 90 % of its last round, else the best
// of them if that fills 80 %.  A split keeps at least 512 of K and the partial tiles within the
// workspace limit.
static int gemm_big_splits(const lumen_ctx *ctx, const GemmArgs &a) {
    if (a.M < 1024 || a.K % GB_K != 0) return 0;
    const long tiles = (long)((a.N + GB_N - 1) / GB_N) * ((a.M + GB_M - 1) / GB_M);
    const long cus = ctx->num_cus;
    int best = 0;
    double best_fill = 0.0;
    for (int s = 1; s <= 4; ++s) {
        if (s > 1 && (a.K / s < 512 || (size_t)s * a.M * a.N * sizeof(float) > ((size_t)256 << 20))) break;
        const long w = tiles * s, rounds = (w + cus - 1) / cus;
        const double fill = (double)w / (double)(rounds * cus);
        if (fill > best_fill) {
            best_fill = fill;
            best = s;
        }
        if (fill >= 0.9) break;
    }
    if (best_fill < 0.8) return 0;
    // A split writes and re-reads s partial copies of C.  Where the 128x128 grid fills the chip two and a
    // half times over on its own (1024 x 11264: 704 tiles) that costs more than the large tile gains
    // (336 against 270 us there).
    const long tiles128 = (long)((a.N + BN - 1) / BN) * ((a.M + BM - 1) / BM);
    if (best > 1 && tiles128 * 2 >= cus * 5) return 0;
    return best;
}

// Two rows of A: the vector-ALU kernel above (TinyLlama shape: prompt pass of 2 tokens 1.43 ms against 1.57 with the
// matrix-core kernel below; with three and four rows it is the other way round, 1.75 / 1.83 against 1.57 ms, and on the
// Llama-2-7B shape with bf16 weights 8.1 / 8.3 against 5.7 ms)
#ifndef GEMM_SKINNY_MAX_M
#define GEMM_SKINNY_MAX_M 2
#endif
// The weight-streaming matrix-core kernel takes three to 32 rows of A, with bf16-stored weights three to 16: a bf16
// weight is half the bytes for the same f32 matrix instructions, and the second row tile then costs more than the tile
// kernels do (Llama-2-7B shape, prompt pass of 32 tokens: 7.7 against 6.0 ms; of 5-16 tokens 5.7 against 5.9).
#define GEMM_STREAM_MAX_M 32
static int gemm_stream_max_rows(int w_bf16) { return w_bf16 ? 16 : GEMM_STREAM_MAX_M; }
static bool gemm_stream_applies(const GemmArgs &a) {
    const bool aligned = (((uintptr_t)a.A | (uintptr_t)a.W) & 15) == 0;
    return aligned && a.K > 0 && a.K % (a.w_bf16 ? 8 : 4) == 0 && a.M > GEMM_SKINNY_MAX_M && a.M <= gemm_stream_max_rows(a.w_bf16) &&
           !(a.epi == EPI_SWIGLU && (a.N & 1));
}
// Workgroups along K per column tile of 16: about three workgroups per compute unit over the chip, at least four
// blocks of K per wavefront, 16 splits at most (the split sum takes that many).
static int gemm_stream_splits(const lumen_ctx *ctx, const GemmArgs &a) {
    const long tiles = (a.N + 15) / 16, nblk = (a.K + 31) / 32;
    long s = (3L * ctx->num_cus + tiles / 2) / tiles;
    while (s > 1 && nblk / (4 * s) < 4) --s;
    if (s > GEMM_MAX_SPLITS) s = GEMM_MAX_SPLITS;
    while (s > 1 && (size_t)s * a.M * a.N * sizeof(float) > ((size_t)256 << 20)) --s;
    return s < 1 ? 1 : (int)s;
}
int gemm_reserve_workspace(lumen_ctx *ctx, size_t need) {
    if (ctx->gemm_ws_bytes >= need) return LUMEN_OK;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    if (ctx->gemm_ws) hipFree(ctx->gemm_ws);
    ctx->gemm_ws = nullptr;
    ctx->gemm_ws_bytes = 0;
    HIP_TRY(hipMalloc((void **)&ctx->gemm_ws, need));
    ctx->gemm_ws_bytes = need;
    return LUMEN_OK;
}

// bytes of partial tiles launch_gemm would want for this product (0: no K split)
size_t gemm_workspace_bytes(const lumen_ctx *ctx, int M, int N, int K, int w_bf16) {
    GemmArgs a = {};
    a.M = M; a.N = N; a.K = K; a.w_bf16 = w_bf16;
    if (M <= 0 || N <= 0 || K <= 0 || K % (w_bf16 ? 8 : 4)) return 0;
    if (M > GEMM_SKINNY_MAX_M && M <= gemm_stream_max_rows(w_bf16)) {  // (alignment is the caller's: assume the streaming kernel)
        const int st = gemm_stream_splits(ctx, a);
        return st > 1 ? (size_t)st * M * N * sizeof(float) : 0;
    }
    int splits = gemm_big_splits(ctx, a);
    if (splits <= 0) splits = gemm_splits(ctx, a);
    return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

template <int MS, bool BF16>
static int launch_gemm_skinny(lumen_ctx *ctx, const GemmArgs &a, int kpad) {
    const size_t lds = (size_t)MS * kpad * sizeof(float);
    // one round of workgroups: as many as fit the compute units' LDS side by side, 16 wavefronts at most
    int per_cu = (int)((size_t)(160 * 1024) / (lds + 512));
    if (per_cu > 16 / SK_WAVES) per_cu = 16 / SK_WAVES;
    if (per_cu < 1) per_cu = 1;
    const int nunits = (a.N + 1) / 2;
    int blocks = (nunits + SK_WAVES - 1) / SK_WAVES;
    const int cap = ctx->num_cus * per_cu;
    if (blocks > cap) {  // every wavefront the same number of units
        const int per_wave = (nunits + cap * SK_WAVES - 1) / (cap * SK_WAVES);
        blocks = (nunits + SK_WAVES * per_wave - 1) / (SK_WAVES * per_wave);
    }
    dim3 grid(blocks, (a.M + MS - 1) / MS);
#define SK_LAUNCH(E)                                                                                                  \
    do {                                                                                                              \
        if (lds > 64 * 1024)                                                                                          \
            HIP_TRY(hipFuncSetAttribute((const void *)gemm_skinny_kernel<MS, BF16, E>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
        hipLaunchKernelGGL((gemm_skinny_kernel<MS, BF16, E>), grid, dim3(SK_THREADS), lds, ctx->stream, a, kpad);      \
    } while (0)
    switch (a.epi) {
        case EPI_STORE: SK_LAUNCH(EPI_STORE); break;
        case EPI_RESIDUAL: SK_LAUNCH(EPI_RESIDUAL); break;
        case EPI_SWIGLU: SK_LAUNCH(EPI_SWIGLU); break;
        default: LUMEN_FAIL(LUMEN_ERR_INVALID, "few-row product: epilogue %d", a.epi);
    }
#undef SK_LAUNCH
    LUMEN_CHECK_LAUNCH();
    return LUMEN_OK;
}

// rows of A per tile of the few-row kernel for this product, 0: the tile kernels take it
static int gemm_skinny_rows(const GemmArgs &a, int *kpad_out) {
    const bool aligned = (((uintptr_t)a.A | (uintptr_t)a.W) & 15) == 0;
    const bool fast = (a.K % (a.w_bf16 ? 8 : 4) == 0) && aligned && a.K > 0;  // rows of 16-byte pieces
    if (!fast || a.M <= 0 || a.M > GEMM_SKINNY_MAX_M || (a.epi == EPI_SWIGLU && (a.N & 1))) return 0;
    if (a.epi != EPI_STORE && a.epi != EPI_RESIDUAL && a.epi != EPI_SWIGLU) return 0;  // (the three epilogues it has)
    const int piece = 64 * (a.w_bf16 ? 8 : 4) * 4;
    const int kpad = (a.K + piece - 1) / piece * piece;
    int ms = a.M <= 2 ? 2 : 4;
    if ((size_t)ms * kpad * sizeof(float) > 150 * 1024) ms = 2;
    if ((size_t)ms * kpad * sizeof(float) > 150 * 1024) return 0;
    if (kpad_out) *kpad_out = kpad;
    return ms;
}


template <int MT, bool BF16>
static void launch_gemm_stream(const GemmArgs &g, int splits, hipStream_t s) {
    dim3 grid((g.N + 15) / 16, 1, splits);
    if (splits > 1) hipLaunchKernelGGL((gemm_stream_kernel<MT, BF16, EPI_STORE, true>), grid, dim3(256), 0, s, g);
    else if (g.epi == EPI_STORE) hipLaunchKernelGGL((gemm_stream_kernel<MT, BF16, EPI_STORE, false>), grid, dim3(256), 0, s, g);
    else if (g.epi == EPI_RESIDUAL) hipLaunchKernelGGL((gemm_stream_kernel<MT, BF16, EPI_RESIDUAL, false>), grid, dim3(256), 0, s, g);
    else hipLaunchKernelGGL((gemm_stream_kernel<MT, BF16, EPI_SWIGLU, false>), grid, dim3(256), 0, s, g);
}

int launch_gemm(lumen_ctx *ctx, const GemmArgs &a) {
    if (a.M <= 0 || a.N <= 0) return LUMEN_OK;
    if (a.epi != EPI_STORE && a.epi != EPI_RESIDUAL && a.epi != EPI_SWIGLU)  // (the switches below read SwiGLU into "else")
        LUMEN_FAIL(LUMEN_ERR_INVALID, "GEMM: epilogue %d (store, residual or SwiGLU)", a.epi);
    const bool aligned = (((uintptr_t)a.A | (uintptr_t)a.W) & 15) == 0;
    const bool fast = (a.K % (a.w_bf16 ? 8 : 4) == 0) && aligned && a.K > 0;  // rows of 16-byte pieces
    int kpad = 0;
    const int ms = gemm_skinny_rows(a, &kpad);
    if (ms) {
        // two rows of A: the weights are streamed the way the single-row product streams them, once per MS rows
        // of A (4, or 2 where 4 rows of K padded to whole pieces do not fit LDS)
        {
            if (a.splits_used) *a.splits_used = 1;
            int rc;
            if (a.w_bf16) rc = ms == 4 ? launch_gemm_skinny<4, true>(ctx, a, kpad) : launch_gemm_skinny<2, true>(ctx, a, kpad);
            else rc = ms == 4 ? launch_gemm_skinny<4, false>(ctx, a, kpad) : launch_gemm_skinny<2, false>(ctx, a, kpad);
            LUMEN_TRY(rc);
            if (a.norm_w && a.norm_out && a.epi == EPI_RESIDUAL)
                LUMEN_TRY(launch_rmsnorm(ctx, a.C, a.norm_w, a.norm_out, a.M, a.N, a.norm_eps));
            return LUMEN_OK;
        }
    }
    if (!fast) {
        if (a.epi != EPI_STORE) LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "fused GEMM needs rows of whole 16-byte pieces and 16-byte alignment (K=%d)", a.K);
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
    const bool stream = gemm_stream_applies(a);
    int splits = stream ? 0 : gemm_big_splits(ctx, a);
    const bool big = splits > 0;
    if (stream) splits = gemm_stream_splits(ctx, a);
    else if (!big) splits = gemm_splits(ctx, a);
    if (splits > 1) {
        LUMEN_TRY(gemm_reserve_workspace(ctx, (size_t)splits * a.M * a.N * sizeof(float)));
        g.part = ctx->gemm_ws;
    }
    dim3 grid((a.N + BN - 1) / BN, (a.M + BM - 1) / BM, splits);
    if (stream) {
        if (a.w_bf16) {
            launch_gemm_stream<1, true>(g, splits, ctx->stream);
        } else {
            if (a.M <= 16) launch_gemm_stream<1, false>(g, splits, ctx->stream);
            else launch_gemm_stream<2, false>(g, splits, ctx->stream);
        }
        stage_times_report(ctx, "weight-streaming prompt product", (a.N + 15) / 16 * splits,
                           "start, [1] requests out, [2] first block done, [3] eighth block done, [4] blocks done, [5] after the "
                           "barrier, [6] stores acknowledged");
    } else if (big) {
        dim3 bgrid((a.N + GB_N - 1) / GB_N, (a.M + GB_M - 1) / GB_M, splits);
        if (a.w_bf16) launch_gemm_tile<true, 4>(g, bgrid, ctx->stream);
        else launch_gemm_tile<false, 4>(g, bgrid, ctx->stream);
    } else if (!a.w_bf16 && a.K % GB_K == 0) {
        // same 128x128 tiles and K splits as gemm_bf16x3_kernel, pipelined like the large tile: 5-13 % faster
        // with f32 weights (bf16-stored weights, half the matrix instructions per slice, run 3 % slower on it)
        launch_gemm_tile<false, 2>(g, grid, ctx->stream);
    } else if (a.w_bf16) {
        launch_gemm_epi<true>(g, grid, ctx->stream);
    } else {
        launch_gemm_epi<false>(g, grid, ctx->stream);
    }
    LUMEN_CHECK_LAUNCH();
    if (a.splits_used) *a.splits_used = 1;
    if (a.keep_splits && a.splits_used && a.epi == EPI_STORE && splits > 1) {
        *a.splits_used = splits;  // the consumer adds the partial products
        return LUMEN_OK;
    }
    const bool want_norm = a.norm_w && a.norm_out && a.epi == EPI_RESIDUAL;
    bool norm_done = false;
    if (splits > 1) {
        if (want_norm && splits <= GEMM_MAX_SPLITS && a.N % 4 == 0 && a.N <= 256 * 4 * GEMM_ROW_VPT &&
            ((((uintptr_t)a.C | (uintptr_t)a.residual | (uintptr_t)g.part | (uintptr_t)a.norm_w | (uintptr_t)a.norm_out) & 15) == 0)) {
            hipLaunchKernelGGL(gemm_reduce_norm_kernel, dim3(a.M), dim3(256), 0, ctx->stream, g, splits);
            norm_done = true;
        } else {
            size_t blocks = ((size_t)a.M * a.N + 255) / 256;
            if (blocks > (size_t)ctx->num_cus * 8) blocks = (size_t)ctx->num_cus * 8;
            launch_gemm_reduce(g, splits, (int)blocks, ctx->stream);
        }
        LUMEN_CHECK_LAUNCH();
    }
    if (want_norm && !norm_done) LUMEN_TRY(launch_rmsnorm(ctx, a.C, a.norm_w, a.norm_out, a.M, a.N, a.norm_eps));
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

LUMEN_DEFINE_WARM(gemm)
