// Host-side stand-ins for the few HIP device facilities the kernels use, so that the device
// code in lumen_amd/csrc/*_device.h can run on the CPU, one OS thread per GPU thread, under
// AddressSanitizer / gdb.  A workgroup barrier is a pthread barrier over the workgroup's
// threads; a wavefront shuffle is an exchange through a per-wavefront slot array bracketed by
// a per-wavefront barrier, which gives the lock-step semantics the kernels rely on.
#pragma once
#define LUMEN_CPU_EMU 1
#include <pthread.h>
#include <sched.h>
#include <stdint.h>

#include <chrono>
#include <cmath>
#include <cstring>
#include <vector>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define __HIP_MEMORY_SCOPE_AGENT 0

struct dim3 {
    unsigned x = 1, y = 1, z = 1;
};

struct EmuBlock {
    pthread_barrier_t bar;
    std::vector<pthread_barrier_t> wave_bar;
    std::vector<uint32_t> slots;  // [waves][64]
    std::vector<float> lds;
};

extern thread_local dim3 threadIdx, blockIdx;
extern dim3 gridDim, blockDim;
extern thread_local EmuBlock *emu_block;

static inline void __syncthreads() { pthread_barrier_wait(&emu_block->bar); }
static inline void __builtin_amdgcn_s_barrier() { pthread_barrier_wait(&emu_block->bar); }

template <typename T>
static inline T __shfl_xor(T v, int off, int width = 64) {
    (void)width;
    static_assert(sizeof(T) == 4, "32-bit shuffles only");
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    uint32_t *s = emu_block->slots.data() + wave * 64;
    memcpy(&s[lane], &v, 4);
    pthread_barrier_wait(&emu_block->wave_bar[wave]);
    T r;
    memcpy(&r, &s[lane ^ off], 4);
    pthread_barrier_wait(&emu_block->wave_bar[wave]);
    return r;
}

static inline float __uint_as_float(unsigned u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline int __float_as_int(float f) {
    int i;
    memcpy(&i, &f, 4);
    return i;
}
static inline float __int_as_float(int i) {
    float f;
    memcpy(&f, &i, 4);
    return f;
}
static inline float emu_exp2f(float x) { return exp2f(x); }
#define __builtin_amdgcn_exp2f(x) emu_exp2f(x)
// DPP row_ror:n (control 0x121..0x12f): lane i of each 16-lane row receives the value of lane (i - n) mod 16
static inline int emu_update_dpp(int old, int src, int ctrl) {
    (void)old;
    const int lane = threadIdx.x & 63;
    int v = src;
    if (ctrl >= 0x121 && ctrl <= 0x12f) {
        const int n = ctrl - 0x120, row = lane & ~15, i = lane & 15;
        const int from = row + ((i - n) & 15);
        const int wave = threadIdx.x >> 6;
        uint32_t *s = emu_block->slots.data() + wave * 64;
        memcpy(&s[lane], &src, 4);
        pthread_barrier_wait(&emu_block->wave_bar[wave]);
        memcpy(&v, &s[from], 4);
        pthread_barrier_wait(&emu_block->wave_bar[wave]);
    }
    return v;
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) emu_update_dpp((old), (src), (ctrl))
static inline int min(int a, int b) { return a < b ? a : b; }
static inline int max(int a, int b) { return a > b ? a : b; }

template <typename T>
static inline T emu_atomic_load(const T *p) {
    static_assert(sizeof(T) == 4, "32-bit atomics only");
    uint32_t u = __atomic_load_n((const uint32_t *)p, __ATOMIC_SEQ_CST);
    T v;
    memcpy(&v, &u, 4);
    return v;
}
template <typename T, typename V>
static inline void emu_atomic_store(T *p, V val) {
    static_assert(sizeof(T) == 4, "32-bit atomics only");
    const T v = (T)val;
    uint32_t u;
    memcpy(&u, &v, 4);
    __atomic_store_n((uint32_t *)p, u, __ATOMIC_SEQ_CST);
}
#define __hip_atomic_load(p, order, scope) emu_atomic_load(p)
#define __hip_atomic_store(p, v, order, scope) emu_atomic_store((p), (v))
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add((p), (v), __ATOMIC_SEQ_CST)
static inline int atomicAdd(int *p, int v) { return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
static inline void __threadfence() { __atomic_thread_fence(__ATOMIC_SEQ_CST); }
#define __builtin_amdgcn_fence(order, scope) __atomic_thread_fence(__ATOMIC_SEQ_CST)
static inline void __builtin_amdgcn_s_sleep(int) { sched_yield(); }
static inline unsigned long long wall_clock64() {  // 100 MHz like the device's constant clock
    using namespace std::chrono;
    return (unsigned long long)duration_cast<nanoseconds>(steady_clock::now().time_since_epoch()).count() / 10ull;
}
// workgroup-shared dynamic memory of the running thread's workgroup
#define PK_DYNAMIC_LDS(name) float *name = emu_block->lds.data()
