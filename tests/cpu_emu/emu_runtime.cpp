// Engine behind tests/cpu_emu/shim/hip/hip_runtime.h: runs a launch's workgroups one after the other, the threads of
// a workgroup as user-space fibers, and stands in for the few host calls of the HIP runtime the library makes.
#include <hip/hip_runtime.h>
#include <pthread.h>
#include <stdio.h>
#include <sys/mman.h>

#include <chrono>
#include <vector>

#if defined(__has_feature)
#if __has_feature(address_sanitizer)
#define EMU_ASAN 1
#endif
#endif
#ifdef EMU_ASAN
#include <sanitizer/common_interface_defs.h>
#endif

dim3 threadIdx, blockIdx, gridDim, blockDim;

// The GPU threads of a workgroup are fibers of ONE OS thread, switched in user space at every point where a GPU
// thread waits for others: a workgroup barrier, a wavefront-wide exchange, a pause inside a polling loop.  A fiber
// runs until it blocks; the next runnable one (in thread order) goes on.  A thread that has returned from the kernel
// no longer counts at a barrier, as on the GPU; if nobody can run, the launch is stuck (a barrier that not every
// live thread reaches) and the program stops with the state of the workgroup.
extern "C" void emu_switch(void **save_sp, void *load_sp);
asm(R"(
.text
.globl emu_switch
.type emu_switch,@function
emu_switch:
    pushq %rbp
    pushq %rbx
    pushq %r12
    pushq %r13
    pushq %r14
    pushq %r15
    movq %rsp, (%rdi)
    movq %rsi, %rsp
    popq %r15
    popq %r14
    popq %r13
    popq %r12
    popq %rbx
    popq %rbp
    ret
.size emu_switch, .-emu_switch
)");

namespace {
constexpr size_t STACK_BYTES = (size_t)1 << 20;
constexpr int MAX_THREADS = 1024;
enum Wait { RUNNABLE = 0, AT_BLOCK_BARRIER, AT_WAVE_EXCHANGE, DONE };
struct Fiber {
    void *sp = nullptr;
    char *stack = nullptr;
    void *fake_stack = nullptr;
    int wait = DONE;
    unsigned long gen = 0;  // generation of the barrier / exchange it waits for
    int parity = 0;
    dim3 tid;
};
struct Wave {
    int lanes = 0, live = 0, arrived = 0;
    unsigned long gen = 0;
    uint32_t slot[2][64];
};
struct Launch {
    dim3 grid, block;
    size_t lds_bytes = 0;
    std::function<void()> body;
};
struct Engine {
    std::vector<Fiber> fibers;
    std::vector<Wave> waves;
    int n = 0, cur = -1, live = 0, barrier_arrived = 0;
    unsigned long barrier_gen = 0;
    void *main_sp = nullptr;
    void *main_fake = nullptr;
    const void *main_stack_bottom = nullptr;
    size_t main_stack_size = 0;
    void *lds = nullptr;
    const Launch *launch = nullptr;
};
Engine E;
bool g_capturing = false;
struct emu_graph_impl { std::vector<Launch> nodes; };
unsigned long g_launches = 0;
void capture_node(Launch &&L);

void annotate_leave(void **fake_save, const void *to_bottom, size_t to_size) {
#ifdef EMU_ASAN
    __sanitizer_start_switch_fiber(fake_save, to_bottom, to_size);
#else
    (void)fake_save; (void)to_bottom; (void)to_size;
#endif
}
void annotate_arrive(void *fake_saved) {
#ifdef EMU_ASAN
    __sanitizer_finish_switch_fiber(fake_saved, nullptr, nullptr);
#else
    (void)fake_saved;
#endif
}

bool runnable(const Fiber &f) {
    switch (f.wait) {
        case RUNNABLE: return true;
        case AT_BLOCK_BARRIER: return E.barrier_gen != f.gen;
        case AT_WAVE_EXCHANGE: return E.waves[f.tid.x >> 6].gen != f.gen;
        default: return false;
    }
}

[[noreturn]] void stuck() {
    int at_bar = 0, at_wave = 0, done = 0;
    for (int i = 0; i < E.n; ++i) {
        at_bar += E.fibers[(size_t)i].wait == AT_BLOCK_BARRIER;
        at_wave += E.fibers[(size_t)i].wait == AT_WAVE_EXCHANGE;
        done += E.fibers[(size_t)i].wait == DONE;
    }
    fprintf(stderr, "cpu emulation: workgroup (%u,%u,%u) is stuck: %d thread(s) at a workgroup barrier, %d at a wavefront "
                    "exchange, %d returned, of %d\n", blockIdx.x, blockIdx.y, blockIdx.z, at_bar, at_wave, done, E.n);
    abort();
}

// from inside fiber `cur` (or from the main context, cur == -1): run the next runnable fiber; returns when this
// context is resumed
void switch_to_next() {
    const int from = E.cur;
    for (int k = 1; k <= E.n; ++k) {
        const int i = (from + k + E.n) % E.n;
        Fiber &f = E.fibers[(size_t)i];
        if (!runnable(f)) continue;
        if (i == from) return;  // only this one can run
        f.wait = RUNNABLE;
        E.cur = i;
        threadIdx = f.tid;
        if (from >= 0) {
            Fiber &me = E.fibers[(size_t)from];
            annotate_leave(me.wait == DONE ? nullptr : &me.fake_stack, f.stack, STACK_BYTES);
            emu_switch(&me.sp, f.sp);
            annotate_arrive(me.fake_stack);
        } else {
            annotate_leave(&E.main_fake, f.stack, STACK_BYTES);
            emu_switch(&E.main_sp, f.sp);
            annotate_arrive(E.main_fake);
        }
        return;
    }
    if (E.live == 0 && from >= 0) {  // the last thread of the workgroup has returned: back to the launcher
        Fiber &me = E.fibers[(size_t)from];
        E.cur = -1;
        annotate_leave(nullptr, E.main_stack_bottom, E.main_stack_size);
        emu_switch(&me.sp, E.main_sp);
    }
    if (E.live == 0) return;
    stuck();
}

void block_barrier_release_if_complete() {
    if (E.live > 0 && E.barrier_arrived == E.live) {
        E.barrier_arrived = 0;
        ++E.barrier_gen;
    }
}
void wave_release_if_complete(Wave &w) {
    if (w.live > 0 && w.arrived == w.live) {
        w.arrived = 0;
        ++w.gen;
    }
}

extern "C" void emu_fiber_main() {
    annotate_arrive(nullptr);
    E.launch->body();
    Fiber &me = E.fibers[(size_t)E.cur];
    me.wait = DONE;
    --E.live;
    Wave &w = E.waves[me.tid.x >> 6];
    --w.live;
    block_barrier_release_if_complete();  // those still waiting no longer wait for this thread
    wave_release_if_complete(w);
    switch_to_next();
    abort();  // a finished fiber is never resumed
}

void prepare_fiber(Fiber &f, unsigned t) {
    if (!f.stack) {
        f.stack = (char *)mmap(nullptr, STACK_BYTES, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
        if (f.stack == MAP_FAILED) emu::not_emulated("mmap of a fiber stack");
    }
    // a frame emu_switch can return through: six callee-saved registers, then the entry point as the return
    // address, placed so that the entry point sees the stack as after a call (16-byte aligned + 8)
    uintptr_t top = ((uintptr_t)f.stack + STACK_BYTES) & ~(uintptr_t)15;
    void **sp = (void **)(top - 8);
    *--sp = (void *)emu_fiber_main;
    for (int i = 0; i < 6; ++i) *--sp = nullptr;
    f.sp = sp;
    f.fake_stack = nullptr;
    f.wait = RUNNABLE;
    f.gen = 0;
    f.parity = 0;
    f.tid = dim3(t, 0, 0);
}

void run(const Launch &L) {
    const int n = (int)(L.block.x * L.block.y * L.block.z);
    if (n <= 0 || n > MAX_THREADS || L.block.y != 1 || L.block.z != 1) emu::not_emulated("workgroup shape");
    ++g_launches;
    if (!E.main_stack_bottom) {
        pthread_attr_t attr;
        pthread_getattr_np(pthread_self(), &attr);
        void *addr = nullptr;
        pthread_attr_getstack(&attr, &addr, &E.main_stack_size);
        pthread_attr_destroy(&attr);
        E.main_stack_bottom = addr;
    }
    gridDim = L.grid;
    blockDim = L.block;
    E.launch = &L;
    E.n = n;
    if ((int)E.fibers.size() < n) E.fibers.resize((size_t)n);
    const int nw = (n + 63) / 64;
    // exactly the bytes the launch asked for, so that an access past them is an access past a heap block
    E.lds = L.lds_bytes ? malloc(L.lds_bytes) : nullptr;
    for (unsigned bz = 0; bz < L.grid.z; ++bz)
        for (unsigned by = 0; by < L.grid.y; ++by)
            for (unsigned bx = 0; bx < L.grid.x; ++bx) {  // one workgroup at a time: statics stand for LDS
                blockIdx = dim3(bx, by, bz);
                E.waves.assign((size_t)nw, Wave());
                for (int w = 0; w < nw; ++w) E.waves[(size_t)w].lanes = E.waves[(size_t)w].live = std::min(64, n - w * 64);
                for (int t = 0; t < n; ++t) prepare_fiber(E.fibers[(size_t)t], (unsigned)t);
                E.live = n;
                E.barrier_arrived = 0;
                E.cur = -1;
                switch_to_next();  // returns when every thread of the workgroup has returned
                if (E.live != 0) stuck();
            }
    free(E.lds);
    E.lds = nullptr;
    E.launch = nullptr;
}
}  // namespace

namespace emu {
void launch(dim3 grid, dim3 block, size_t lds_bytes, std::function<void()> body) {
    Launch L;
    L.grid = grid;
    L.block = block;
    L.lds_bytes = lds_bytes;
    L.body = std::move(body);
    if (g_capturing) capture_node(std::move(L));
    else run(L);
}
void workgroup_barrier() {
    Fiber &me = E.fibers[(size_t)E.cur];
    me.gen = E.barrier_gen;
    me.wait = AT_BLOCK_BARRIER;
    ++E.barrier_arrived;
    block_barrier_release_if_complete();
    if (runnable(me)) me.wait = RUNNABLE;  // the last one to arrive goes straight on
    else switch_to_next();
}
uint32_t wave_exchange(uint32_t mine, int from_lane) {
    Fiber &me = E.fibers[(size_t)E.cur];
    Wave &w = E.waves[me.tid.x >> 6];
    const int lane = (int)(me.tid.x & 63), par = me.parity;
    me.parity ^= 1;
    w.slot[par][lane] = mine;
    me.gen = w.gen;
    me.wait = AT_WAVE_EXCHANGE;
    ++w.arrived;
    wave_release_if_complete(w);
    if (runnable(me)) me.wait = RUNNABLE;
    else switch_to_next();
    // (a lane that has returned from the kernel gives nothing: its reader keeps its own value)
    return (from_lane >= 0 && from_lane < w.lanes) ? w.slot[par][from_lane] : mine;
}
void *dynamic_lds() { return E.lds; }
void yield() {
    if (E.cur >= 0) switch_to_next();
}
void not_emulated(const char *what) {
    fprintf(stderr, "cpu emulation: %s is not emulated\n", what);
    abort();
}
unsigned long launches() { return g_launches; }
}  // namespace emu

void emu_sleep() { emu::yield(); }
unsigned long long wall_clock64() {
    using namespace std::chrono;
    return (unsigned long long)duration_cast<nanoseconds>(steady_clock::now().time_since_epoch()).count() / 10ull;
}

// ---------------------------------------------------------------------- host API
struct emu_stream { int unused; };
struct emu_event { std::chrono::steady_clock::time_point t; };
struct emu_graph { emu_graph_impl impl; };

const char *hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "error (cpu emulation)"; }
hipError_t hipGetLastError() { return hipSuccess; }
hipError_t hipGetDeviceCount(int *n) { *n = 1; return hipSuccess; }
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipGetDeviceProperties(hipDeviceProp_t *p, int) {
    memset(p, 0, sizeof(*p));
    strcpy(p->gcnArchName, "gfx950:cpu-emulation");
    p->multiProcessorCount = 256;  // the launchers size their grids for the real chip
    return hipSuccess;
}
hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) { *s = new emu_stream(); return hipSuccess; }
hipError_t hipStreamDestroy(hipStream_t s) { delete s; return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t *e) { *e = new emu_event(); return hipSuccess; }
hipError_t hipEventDestroy(hipEvent_t e) { delete e; return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t e, hipStream_t) { e->t = std::chrono::steady_clock::now(); return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t a, hipEvent_t b) {
    *ms = std::chrono::duration<float, std::milli>(b->t - a->t).count();
    return hipSuccess;
}
hipError_t hipMalloc(void **p, size_t bytes) {
    // exactly `bytes`: the first byte behind a device allocation is out of bounds here
    *p = nullptr;
    return posix_memalign(p, 256, bytes ? bytes : 1) == 0 ? hipSuccess : hipErrorInvalidValue;
}
hipError_t hipFree(void *p) { free(p); return hipSuccess; }
hipError_t hipHostMalloc(void **p, size_t bytes, unsigned) { *p = malloc(bytes ? bytes : 1); return *p ? hipSuccess : hipErrorInvalidValue; }
hipError_t hipHostFree(void *p) { free(p); return hipSuccess; }
hipError_t hipMemcpy(void *dst, const void *src, size_t bytes, hipMemcpyKind) { memmove(dst, src, bytes); return hipSuccess; }
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind k, hipStream_t) {
    if (g_capturing) emu::not_emulated("a copy inside a captured graph");
    return hipMemcpy(dst, src, bytes, k);
}
hipError_t hipMemcpy2DAsync(void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t height,
                            hipMemcpyKind, hipStream_t) {
    for (size_t r = 0; r < height; ++r) memmove((char *)dst + r * dpitch, (const char *)src + r * spitch, width);
    return hipSuccess;
}
hipError_t hipMemset(void *p, int v, size_t bytes) { memset(p, v, bytes); return hipSuccess; }
hipError_t hipMemsetAsync(void *p, int v, size_t bytes, hipStream_t) {
    if (g_capturing) emu::not_emulated("a memset inside a captured graph");
    memset(p, v, bytes);
    return hipSuccess;
}
static emu_graph *g_capture = nullptr;
namespace {
void capture_node(Launch &&L) { g_capture->impl.nodes.push_back(std::move(L)); }
}  // namespace
hipError_t hipStreamBeginCapture(hipStream_t, int) {
    g_capture = new emu_graph();
    g_capturing = true;
    return hipSuccess;
}
hipError_t hipStreamEndCapture(hipStream_t, hipGraph_t *g) {
    g_capturing = false;
    *g = g_capture;
    g_capture = nullptr;
    return hipSuccess;
}
hipError_t hipGraphInstantiate(hipGraphExec_t *e, hipGraph_t g, void *, void *, unsigned long long) {
    emu_graph *c = new emu_graph();
    c->impl.nodes = g->impl.nodes;
    *e = c;
    return hipSuccess;
}
hipError_t hipGraphLaunch(hipGraphExec_t e, hipStream_t) {
    for (const Launch &L : e->impl.nodes) run(L);
    return hipSuccess;
}
hipError_t hipGraphUpload(hipGraphExec_t, hipStream_t) { return hipSuccess; }
hipError_t hipGraphDestroy(hipGraph_t g) { delete g; return hipSuccess; }
hipError_t hipGraphExecDestroy(hipGraphExec_t e) { delete e; return hipSuccess; }
