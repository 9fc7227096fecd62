// CPU stand-in for <hip/hip_runtime.h>: the device code and the launchers of lumen_amd/csrc compile with a host
// compiler against this header and run on the CPU -- the GPU threads of a workgroup as user-space fibers switched at
// every barrier, wavefront exchange and polling pause, the workgroups of a launch one after the other in index order (producers inside a chained launch have lower indices than their
// consumers, so every wait finds its value) -- under AddressSanitizer / UndefinedBehaviorSanitizer, where every
// load and store of a kernel is bounds-checked: device memory is host heap memory, static LDS arrays are static
// arrays, the dynamic LDS array of a launch is a heap block of exactly the size the launch asked for.
//
// Wavefront-wide operations (DPP rotations, lane reads, shuffles) exchange values through a slot array of the
// wavefront once every live lane has arrived: every lane must reach the call, as on the GPU.
// The matrix-core instructions are not emulated: a kernel that issues one stops the program.
#pragma once
#define LUMEN_CPU_EMU 1
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <cmath>
#include <functional>

// ------------------------------------------------------------------ qualifiers
#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)
#define __align__(n) __attribute__((aligned(n)))
#define __shared__ static
#define amdgpu_waves_per_eu(...) __unused__  // (an occupancy request of the GPU compiler: nothing to do here)
#define __HIP_MEMORY_SCOPE_AGENT 4
#define HIP_SYMBOL(x) (&(x))

struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};
extern dim3 threadIdx, blockIdx, gridDim, blockDim;  // (of the fiber that is running)

// ------------------------------------------------------------------ engine (emu_runtime.cpp)
namespace emu {
void launch(dim3 grid, dim3 block, size_t lds_bytes, std::function<void()> body);
void workgroup_barrier();
uint32_t wave_exchange(uint32_t mine, int from_lane);  // every lane gives a value and names the lane it reads
void *dynamic_lds();
void yield();
[[noreturn]] void not_emulated(const char *what);
}  // namespace emu

#define LUMEN_DYNAMIC_LDS(type, name) type *name = (type *)emu::dynamic_lds()
#define hipLaunchKernelGGL(kernel, grid, block, lds, stream, ...) \
    emu::launch((grid), (block), (lds), [=]() { (kernel)(__VA_ARGS__); })

// ------------------------------------------------------------------ device builtins
static inline void __syncthreads() { emu::workgroup_barrier(); }
template <typename T>
static inline T emu_bits_to(uint32_t u) {
    static_assert(sizeof(T) == 4, "32-bit values only");
    T v;
    memcpy(&v, &u, 4);
    return v;
}
template <typename T>
static inline uint32_t emu_bits_of(T v) {
    static_assert(sizeof(T) == 4, "32-bit values only");
    uint32_t u;
    memcpy(&u, &v, 4);
    return u;
}
template <typename T>
static inline T __shfl_xor(T v, int off, int width = 64) {
    (void)width;
    return emu_bits_to<T>(emu::wave_exchange(emu_bits_of(v), (int)((threadIdx.x & 63) ^ (unsigned)off)));
}
// DPP row_ror:n (control 0x121 .. 0x12f): lane i of a row of 16 lanes receives the value of lane (i - n) mod 16
static inline int emu_update_dpp(int src, int ctrl) {
    if (ctrl < 0x121 || ctrl > 0x12f) emu::not_emulated("DPP control other than row_ror");
    const int lane = (int)(threadIdx.x & 63), n = ctrl - 0x120;
    return (int)emu::wave_exchange((uint32_t)src, (lane & ~15) | ((lane - n) & 15));
}
#define __builtin_amdgcn_update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl) emu_update_dpp((src), (ctrl))
static inline int emu_readlane(int v, int lane) { return (int)emu::wave_exchange((uint32_t)v, lane); }
#define __builtin_amdgcn_readlane(v, lane) emu_readlane((v), (lane))

static inline float __uint_as_float(unsigned u) { return emu_bits_to<float>(u); }
static inline unsigned __float_as_uint(float f) { return emu_bits_of(f); }
static inline int __float_as_int(float f) { return (int)emu_bits_of(f); }
static inline float __int_as_float(int i) { return emu_bits_to<float>((uint32_t)i); }
#define __builtin_amdgcn_exp2f(x) exp2f(x)
#define __builtin_amdgcn_s_waitcnt(x) ((void)0)
#define __builtin_amdgcn_sched_group_barrier(a, b, c) ((void)0)
void emu_sleep();
#define __builtin_amdgcn_s_sleep(n) emu_sleep()
unsigned long long wall_clock64();  // 100 MHz like the device's constant clock
static inline unsigned emu_perm(unsigned hi, unsigned lo, unsigned sel) {  // v_perm_b32
    const uint64_t src = ((uint64_t)hi << 32) | lo;
    unsigned out = 0;
    for (int i = 0; i < 4; ++i) {
        const unsigned s = (sel >> (8 * i)) & 0xff;
        unsigned byte = 0;
        if (s <= 7) byte = (unsigned)(src >> (8 * s)) & 0xff;
        else if (s == 0x0c) byte = 0;
        else emu::not_emulated("v_perm_b32 selector");
        out |= byte << (8 * i);
    }
    return out;
}
#define __builtin_amdgcn_perm(hi, lo, sel) emu_perm((hi), (lo), (sel))
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) (emu::not_emulated("v_mfma_f32_32x32x16_bf16"), (c))
// v_mfma_f32_16x16x4_f32: D[i][j] = C[i][j] + sum over k < 4 of A[i][k] B[k][j]; lane l gives A[l % 16][l / 16] and
// B[l / 16][l % 16] and holds D[4 (l / 16) + r][l % 16] in element r.  (The order of the four products inside the
// instruction is the hardware's; results are compared to a tolerance.)
template <typename V>
static inline V emu_mfma_16x16x4f32(float a, float b, V c) {
    const int lane = (int)(threadIdx.x & 63), j = lane & 15, g = lane >> 4;
    float bk[4];
    for (int k = 0; k < 4; ++k) bk[k] = emu_bits_to<float>(emu::wave_exchange(emu_bits_of(b), k * 16 + j));
    for (int r = 0; r < 4; ++r)
        for (int k = 0; k < 4; ++k) {
            const float aik = emu_bits_to<float>(emu::wave_exchange(emu_bits_of(a), k * 16 + 4 * g + r));
            c[r] = fmaf(aik, bk[k], c[r]);
        }
    return c;
}
#define __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, x, y, z) emu_mfma_16x16x4f32((a), (b), (c))
// On the GPU the lanes of a wavefront run in lockstep and the wave barrier only orders the compiler; here the lanes are
// fibers of their own and have to meet.
#define __builtin_amdgcn_wave_barrier() ((void)emu::wave_exchange(0u, 0))

using std::max;
using std::min;
static inline int min(int a, unsigned b) { return a < (int)b ? a : (int)b; }

// agent-scope atomics on 4- and 8-byte objects
template <typename T>
static inline T emu_atomic_load(const T *p) {
    T v;
    __atomic_load(p, &v, __ATOMIC_SEQ_CST);
    return v;
}
template <typename T, typename V>
static inline void emu_atomic_store(T *p, V val) {
    T v = (T)val;
    __atomic_store(p, &v, __ATOMIC_SEQ_CST);
}
#define __hip_atomic_load(p, order, scope) emu_atomic_load(p)
#define __hip_atomic_store(p, v, order, scope) emu_atomic_store((p), (v))
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add((p), (v), __ATOMIC_SEQ_CST)

// ------------------------------------------------------------------ host API (the part the library uses)
typedef int hipError_t;
enum { hipSuccess = 0, hipErrorLaunchFailure = 719, hipErrorInvalidValue = 1 };
typedef struct emu_stream *hipStream_t;
typedef struct emu_event *hipEvent_t;
typedef struct emu_graph *hipGraph_t;
typedef struct emu_graph *hipGraphExec_t;
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum { hipStreamNonBlocking = 1, hipHostMallocDefault = 0, hipStreamCaptureModeThreadLocal = 1,
       hipFuncAttributeMaxDynamicSharedMemorySize = 8 };
struct hipDeviceProp_t {
    char gcnArchName[64];
    int multiProcessorCount;
};
const char *hipGetErrorString(hipError_t e);
hipError_t hipGetLastError();
hipError_t hipGetDeviceCount(int *n);
hipError_t hipSetDevice(int d);
hipError_t hipGetDeviceProperties(hipDeviceProp_t *p, int d);
hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned flags);
hipError_t hipStreamDestroy(hipStream_t s);
hipError_t hipStreamSynchronize(hipStream_t s);
hipError_t hipEventCreate(hipEvent_t *e);
hipError_t hipEventDestroy(hipEvent_t e);
hipError_t hipEventRecord(hipEvent_t e, hipStream_t s);
hipError_t hipEventSynchronize(hipEvent_t e);
hipError_t hipEventElapsedTime(float *ms, hipEvent_t a, hipEvent_t b);
hipError_t hipMalloc(void **p, size_t bytes);
hipError_t hipFree(void *p);
hipError_t hipHostMalloc(void **p, size_t bytes, unsigned flags);
hipError_t hipHostFree(void *p);
hipError_t hipMemcpy(void *dst, const void *src, size_t bytes, hipMemcpyKind kind);
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind kind, hipStream_t s);
hipError_t hipMemcpy2DAsync(void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t height,
                            hipMemcpyKind kind, hipStream_t s);
hipError_t hipMemset(void *p, int v, size_t bytes);
hipError_t hipMemsetAsync(void *p, int v, size_t bytes, hipStream_t s);
hipError_t hipStreamBeginCapture(hipStream_t s, int mode);
hipError_t hipStreamEndCapture(hipStream_t s, hipGraph_t *g);
hipError_t hipGraphInstantiate(hipGraphExec_t *e, hipGraph_t g, void *, void *, unsigned long long);
hipError_t hipGraphLaunch(hipGraphExec_t e, hipStream_t s);
hipError_t hipGraphUpload(hipGraphExec_t e, hipStream_t s);
hipError_t hipGraphDestroy(hipGraph_t g);
hipError_t hipGraphExecDestroy(hipGraphExec_t e);
template <typename T>
static inline hipError_t hipGetSymbolAddress(void **p, T *symbol) {
    *p = (void *)symbol;
    return hipSuccess;
}
template <typename F>
static inline hipError_t hipFuncSetAttribute(F, int, int) { return hipSuccess; }
template <typename T>
static inline hipError_t hipMemcpyFromSymbol(void *dst, T *symbol, size_t bytes) { memcpy(dst, symbol, bytes); return hipSuccess; }
template <typename T>
static inline hipError_t hipMemcpyToSymbol(T *symbol, const void *src, size_t bytes) { memcpy(symbol, src, bytes); return hipSuccess; }
template <typename T>
static inline hipError_t hipMalloc(T **p, size_t bytes) { return hipMalloc((void **)p, bytes); }
