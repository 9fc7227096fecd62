// Where the time of a kernel goes: a build option (-DLUMEN_STAGE_TIMES) that makes thread 0 of every workgroup
// write the 100 MHz wall clock at up to eight points of a kernel into a device array; after launches inside a window
// chosen with LUMEN_STAGE_TIMES_WINDOW="first,count" (launch numbers of the process, default 4000,8) the host waits
// for the launch and prints, per point, the minimum / median / maximum over the workgroups in microseconds relative
// to the first workgroup's start.  The waits make the printed launches start on an idle chip: the first ~1 us of
// skew between XCDs seen then is absent in back-to-back launches.  Product builds compile all of it away.
#pragma once
#include <hip/hip_runtime.h>

#ifdef LUMEN_STAGE_TIMES
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>
#define STAGE_MAX_WG 4096
__device__ unsigned long long lumen_stage_clock[STAGE_MAX_WG * 8];
#define STAGE_WG_INDEX ((blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x)
#define STAGE_T(i)                                                                                      \
    do {                                                                                                \
        if (threadIdx.x == 0 && STAGE_WG_INDEX < STAGE_MAX_WG) lumen_stage_clock[STAGE_WG_INDEX * 8 + (i)] = wall_clock64(); \
    } while (0)
#define STAGE_T_STORES_DONE(i)              \
    do {                                    \
        __builtin_amdgcn_s_waitcnt(0);      \
        STAGE_T(i);                         \
    } while (0)
// seg_ends: optional ascending workgroup indices that end the roles of a chained launch (each role is reported on its own)
static inline void stage_times_report(lumen_ctx *ctx, const char *what, int n_wg, const char *legend,
                                      const int *seg_ends = nullptr, int nseg = 0) {
    static int first = -1, count = 0, calls = 0;
    if (first < 0) {
        first = 4000;
        count = 8;
        if (const char *e = getenv("LUMEN_STAGE_TIMES_WINDOW")) sscanf(e, "%d,%d", &first, &count);
    }
    const int call = calls++;
    if (call < first || call >= first + count) return;
    hipStreamSynchronize(ctx->stream);
    static unsigned long long h[STAGE_MAX_WG * 8];
    hipMemcpyFromSymbol(h, HIP_SYMBOL(lumen_stage_clock), sizeof(h));
    const int nb = n_wg < STAGE_MAX_WG ? n_wg : STAGE_MAX_WG;
    unsigned long long t0 = ~0ull;
    for (int b = 0; b < nb; ++b) t0 = h[b * 8] < t0 ? h[b * 8] : t0;
    fprintf(stderr, "[stage times] launch %d: %s, %d workgroups\n", call, what, n_wg);
    const int one_end[1] = {nb};
    if (!seg_ends || nseg <= 0) { seg_ends = one_end; nseg = 1; }
    int b0 = 0;
    for (int sgi = 0; sgi < nseg; ++sgi) {
        const int b1 = seg_ends[sgi] < nb ? seg_ends[sgi] : nb;
        fprintf(stderr, "    workgroups %d..%d:", b0, b1 - 1);
        for (int i = 0; i < 8; ++i) {
            std::vector<double> v;
            for (int b = b0; b < b1; ++b)
                if (h[b * 8 + i] >= t0 && h[b * 8 + i] - t0 < 100000000ull) v.push_back((double)(h[b * 8 + i] - t0) * 0.01);
            if (v.empty()) continue;
            std::sort(v.begin(), v.end());
            fprintf(stderr, " [%d] %.2f/%.2f/%.2f", i, v[0], v[v.size() / 2], v.back());
        }
        fprintf(stderr, "\n");
        b0 = b1;
    }
    fprintf(stderr, "    us min/median/max over workgroups: %s\n", legend);
    static unsigned long long zero[STAGE_MAX_WG * 8];
    hipMemcpyToSymbol(HIP_SYMBOL(lumen_stage_clock), zero, sizeof(zero));
}
#else
#define STAGE_T(i) do { } while (0)
#define STAGE_T_STORES_DONE(i) do { } while (0)
struct lumen_ctx;
static inline void stage_times_report(lumen_ctx *, const char *, int, const char *, const int * = nullptr, int = 0) {}
#endif
