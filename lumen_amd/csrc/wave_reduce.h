// Reductions over the 64 lanes of a wavefront that leave the same value in every lane.  Four DPP
// rotate-and-combine steps give each row of 16 lanes its result, the four row results are read through
// scalar registers.  (__shfl_xor compiles to ds_bpermute: six dependent trips through the LDS crossbar.)
// Every lane of the wavefront must be active at the call.
#pragma once
#include <hip/hip_runtime.h>


__device__ __forceinline__ float wave_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false));  // row_ror:8
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false));  // row_ror:4
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false));  // row_ror:2
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false));  // row_ror:1
    const int b = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xf, 0xf, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124, 0xf, 0xf, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x122, 0xf, 0xf, false)));
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x121, 0xf, 0xf, false)));
    const int b = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(b, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(b, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(b, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(b, 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// Arrival at a cross-workgroup hand-over: the workgroup has stored its partial results, passed a workgroup
// barrier, and one thread now counts it in; the workgroup that sees the full count reads all partials.
//
// What orders the partial stores before the later loads is the hardware, not the language's memory model:
//  * every partial is written with an agent-scope atomic store and read with an agent-scope atomic load.  On
//    gfx950 these are `global_store ... sc1` / `global_load ... sc1`: the store writes through the XCD's L2 to
//    the memory side shared by all XCDs, the load misses the compute unit's L1 and the XCD's non-coherent L2
//    lines, so neither a cache write-back nor an invalidate is needed for them to meet;
//  * the workgroup barrier in front of the arrival makes every wavefront wait for the acknowledgement of its own
//    stores (s_waitcnt vmcnt(0)) before thread 0 issues the read-modify-write, itself an agent-scope atomic that
//    executes at the memory side, and the barrier behind it holds the readers back until thread 0 has the count.
// With LUMEN_HANDOVER_ORDER = __ATOMIC_ACQ_REL the read-modify-write is a formal acquire-release at agent scope
// (cumulative with the barriers on both sides); the compiler then adds an L2 write-back in front of it and an
// invalidate behind it for every arriving workgroup, which the write-through stores do not need: measured, the
// lm_head product with the arg-max tail goes from 44 to 89 us (1000 workgroups) and the 16-slice merge of decode
// attention from 10.4 to 14.5 us.  The default is therefore the relaxed read-modify-write; both builds give the
// same bits, and tests/test_gpu_model.py repeats a sliced decode twenty times to hold the default to that.
#ifndef LUMEN_HANDOVER_ORDER
#define LUMEN_HANDOVER_ORDER __ATOMIC_RELAXED
#endif
// In front of the barrier that precedes handover_arrive: this wavefront's partial stores are acknowledged (written
// through to the memory side) before it enters the barrier.  The compiler emits this wait in front of s_barrier
// anyway; stating it here keeps the hand-over independent of that.
__device__ __forceinline__ void handover_stores_done() { __builtin_amdgcn_s_waitcnt(0); }
__device__ __forceinline__ int handover_arrive(int *counter) {
    return __hip_atomic_fetch_add(counter, 1, LUMEN_HANDOVER_ORDER, __HIP_MEMORY_SCOPE_AGENT);
}
