// fm_ring.h — primitives of the weight ring in LDS that the streaming kernels share.
//
// LDS-direct loads (global_load_lds_dword / _dwordx4): every lane supplies a global
// address, the wave's 64 x 4 or 64 x 16 bytes land back to back in LDS at the
// address in M0.  They need no destination registers, so several slices per wave
// can be in flight while the multiply keeps the registers.  They complete in issue
// order and count in vmcnt: a slice is known to have landed once at most
// (loads per slice) x (younger slices) vector-memory operations are outstanding.
// The compiler does not see the dependence between such a load and a later LDS
// read, and it makes every LDS access that it does see wait for all of them — so
// the consumers wait and read with explicit instructions.
#pragma once

#include "fm_common.h"

#if defined(__HIPCC__)

typedef const __attribute__((address_space(1))) void *fm_gptr;
typedef __attribute__((address_space(3))) void *fm_lptr;

// A pointer every lane of the wave agrees on, moved to scalar registers.
__device__ __forceinline__ const uint8_t *fm_uniform(const uint8_t *p) {
    uintptr_t v = (uintptr_t)p;
    uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const uint8_t *)(((uintptr_t)hi << 32) | lo);
}

// wait until at most N vector-memory operations are outstanding (all of them: drain)
template <int N>
__device__ __forceinline__ void fm_dma_wait(bool drain) {
    if (drain) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// LDS byte address of a pointer into __shared__ memory
__device__ __forceinline__ uint32_t fm_lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(fm_lptr)p;
}

#endif
