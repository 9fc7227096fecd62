// Host side of the persistent decode kernel: shape checks, LDS sizing and the
// cooperative launch (the device code lives in decode_persistent_device.h).
#include "internal.h"
#include "decode_persistent_device.h"

// ---------------------------------------------------------------------- host
size_t pk_lds_bytes(const PkArgs &a, int nrep) {
    const int vec = a.w_bf16 ? 8 : 4, sweep = 64 * vec;
    int kmax = a.H > a.I ? a.H : a.I;
    if (a.qd > kmax) kmax = a.qd;
    const size_t xs = (size_t)((kmax + sweep - 1) / sweep * sweep) * sizeof(float);
    const size_t att = ((size_t)2 * nrep * a.D + 3 * a.D + (size_t)PK_WAVES * nrep * a.D + 2 * PK_WAVES * nrep + 4) * sizeof(float);
    size_t need = (xs > att ? xs : att) + PK_LDS_HEADER * sizeof(float);
    // more than half of the CU's 160 KiB so that exactly one workgroup lives on each compute unit
    const size_t floor_bytes = 84 * 1024;
    return need > floor_bytes ? need : floor_bytes;
}

bool pk_supported(const PkArgs &a) {
    const int nrep = a.hkv > 0 ? a.hq / a.hkv : 0;
    if (!(a.D == 64 || a.D == 128)) return false;
    if (!(nrep == 1 || nrep == 2 || nrep == 4 || nrep == 8)) return false;
    const int vec = a.w_bf16 ? 8 : 4;
    if (a.H % vec || a.I % vec || a.qd % vec || (a.qd + 2 * a.kvd) % 2 || a.H % 2 || a.V % 1) return false;
    if (pk_lds_bytes(a, nrep) > 150 * 1024) return false;
    return true;
}

template <int D, int NREP, bool BF16>
static int launch_pk_t(lumen_ctx *ctx, PkArgs &a, int nblocks, size_t lds) {
    auto kern = decode_persistent_kernel<D, NREP, BF16>;
    static size_t configured_lds = 0;
    if (configured_lds != lds) {
        HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        int per_cu = 0;
        HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, PK_THREADS, lds));
        if (per_cu < 1) LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "persistent decode kernel does not fit a compute unit");
        configured_lds = lds;
    }
    void *params[] = {&a};
    HIP_TRY(hipLaunchCooperativeKernel((const void *)kern, dim3(nblocks), dim3(PK_THREADS), params, (unsigned)lds,
                                       ctx->stream));
    return LUMEN_OK;
}

template <int D, bool BF16>
static int launch_pk_d(lumen_ctx *ctx, PkArgs &a, int nrep, int nblocks, size_t lds) {
    switch (nrep) {
        case 1: return launch_pk_t<D, 1, BF16>(ctx, a, nblocks, lds);
        case 2: return launch_pk_t<D, 2, BF16>(ctx, a, nblocks, lds);
        case 4: return launch_pk_t<D, 4, BF16>(ctx, a, nblocks, lds);
        default: return launch_pk_t<D, 8, BF16>(ctx, a, nblocks, lds);
    }
}

int launch_decode_persistent(lumen_ctx *ctx, PkArgs &a) {
    if (!pk_supported(a)) LUMEN_FAIL(LUMEN_ERR_UNSUPPORTED, "shape outside the persistent decode kernel");
    const int nrep = a.hq / a.hkv;
    const int nblocks = ctx->num_cus;
    const size_t lds = pk_lds_bytes(a, nrep);
    a.timeout_ticks = 200000000ull;  // 2 s of the 100 MHz wall clock per barrier
    HIP_TRY(hipMemsetAsync(a.bar, 0, sizeof(unsigned), ctx->stream));
    HIP_TRY(hipMemsetAsync(a.err, 0, sizeof(int), ctx->stream));
    if (a.D == 64) return a.w_bf16 ? launch_pk_d<64, true>(ctx, a, nrep, nblocks, lds) : launch_pk_d<64, false>(ctx, a, nrep, nblocks, lds);
    return a.w_bf16 ? launch_pk_d<128, true>(ctx, a, nrep, nblocks, lds) : launch_pk_d<128, false>(ctx, a, nrep, nblocks, lds);
}
