// Global memory -> LDS without passing through registers (gfx950: 16 bytes per lane).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qproj {

// One instruction moves 64 x 16 bytes: lane l's 16 bytes at `g` (any address per lane) land at l + 16*l,
// with `l` the same LDS address in every lane.  Completion is counted by vmcnt like any vector load; the
// compiler does not order LDS reads against these writes, the callers wait (s_waitcnt vmcnt) themselves.
__device__ __forceinline__ void global_to_lds16(const void *g, void *l) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)g,
                                     (__attribute__((address_space(3))) void *)l, 16, 0, 0);
}

// a wave-uniform pointer pinned to scalar registers: what is added to it afterwards stays a 32-bit lane
// offset (scalar base + vector offset addressing) instead of becoming a 64-bit pointer per lane
template <typename T>
__device__ __forceinline__ const T *scalar_pointer(const T *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return reinterpret_cast<const T *>(((uint64_t)hi << 32) | lo);
}

// The same, typed as a pointer into global memory: a pointer rebuilt from integers has lost its address space,
// and loads through it would be flat loads, which count against the LDS wait counter as well as the vector
// memory one (a wait for an LDS read would then also wait for them).
template <typename T>
using global_ptr = const T __attribute__((address_space(1))) *;

template <typename T>
__device__ __forceinline__ global_ptr<T> scalar_global(const T *p) {
    return (global_ptr<T>)scalar_pointer(p);
}

// 16 / 8 / 4 bytes at byte offset `off` from a global base
template <typename V, typename T>
__device__ __forceinline__ V load_global(global_ptr<T> base, uint32_t off) {
#if defined(__HIP_DEVICE_COMPILE__)
    return *(global_ptr<V>)((global_ptr<uint8_t>)base + off);
#else
    return V{};   // device-only; the host pass just has to parse it
#endif
}

}  // namespace qproj
