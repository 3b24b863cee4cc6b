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

#include "fm_index.h"
#include "fm_unpack.h"

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


// One ring slot = one slice (a wave step's rows of one matrix): 64 lanes' worth of
// codes laid out as the rows lie in memory, 256 B of scales, 256 B of biases, and a
// 16-byte trailer for the tag (which unit the slice belongs to).
template <int BITS>
struct FmSlot {
    static constexpr int NQ = FmLaneBytes<BITS>::value / 16;
    static constexpr int WBYTES = FM_WAVE * FmLaneBytes<BITS>::value;
    static constexpr int TAG = WBYTES + 512;
    static constexpr int BYTES = WBYTES + 512 + 16;
    static constexpr int LOADS = NQ + 2;            // LDS-direct loads per slice
};

// Lane map of a wave step: LPR lanes share a row (lane = 4*chunk + row-in-quad), the
// step covers 64/LPR consecutive rows.  woff / soff: this lane's 48/64 code bytes and
// its scale/bias word inside a slot whose rows are row_bytes / sb_row_bytes apart.
template <int BITS, int LPR>
__device__ __forceinline__ void fm_unit_lane_offsets(int lane, int row_bytes, int sb_row_bytes,
                                                     uint32_t &woff, uint32_t &soff,
                                                     int &row_in_step, int &ch) {
    const FmUnitLane u = fm_unit_lane(lane, LPR, FmLaneBytes<BITS>::value, row_bytes, sb_row_bytes);
    woff = u.woff, soff = u.soff, row_in_step = u.row_in_step, ch = u.ch;
}

// Cache policy of a weight load (the builtin's last argument).  FM_AUX_ONCE = the non-temporal
// bit, for bytes a launch reads exactly once (the experts of a decode step, a vocabulary
// projection): the line is not kept in the caches, and the stream runs 4-12 % faster — the
// dense probe 7.0 instead of 6.25 TB/s, the decode step 85.9 instead of 89.7 us.  FM_AUX_KEEP
// where later units of the launch read the same bytes again (positions of a chunk that share
// experts, the grouped products: with the bit set a 512-position chunk takes 202 instead of
// 163 us).  An immediate of the instruction, hence a template argument.
#define FM_AUX_KEEP 0
#define FM_AUX_ONCE 2

template <int BITS, int I, int AUX>
__device__ __forceinline__ void fm_dma_codes(uint32_t slot, fm_gptr w) {
    if constexpr (I < FmSlot<BITS>::NQ) {
        // the instruction offset moves the global and the LDS address alike; it holds
        // -4096..4095, so from the fifth load on both addresses move by 4096 instead
        constexpr int BASE = (I / 4) * 4096, IMM = (I % 4) * 1024;
        __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)((const uint8_t *)w + BASE),
                                         (fm_lptr)(uintptr_t)(slot + BASE), 16, IMM, AUX);
        fm_dma_codes<BITS, I + 1, AUX>(slot, w);
    }
}

// w, s, b: first byte of the unit's rows in the weight, scale and bias regions
template <int BITS, int AUX = FM_AUX_KEEP>
__device__ __forceinline__ void fm_dma_issue(uint32_t slot, const uint8_t *w, const uint8_t *s,
                                             const uint8_t *b, int lane) {
    fm_dma_codes<BITS, 0, AUX>(slot, (fm_gptr)(uintptr_t)(w + lane * 16));
    __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(s + lane * 4),
                                     (fm_lptr)(uintptr_t)(slot + FmSlot<BITS>::WBYTES), 4, 0, AUX);
    __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(b + lane * 4),
                                     (fm_lptr)(uintptr_t)(slot + FmSlot<BITS>::WBYTES + 256), 4, 0, AUX);
}
// (once: uniform over the wave)
template <int BITS>
__device__ __forceinline__ void fm_dma_issue_as(bool once, uint32_t slot, const uint8_t *w, const uint8_t *s,
                                                const uint8_t *b, int lane) {
    if (once) fm_dma_issue<BITS, FM_AUX_ONCE>(slot, w, s, b, lane);
    else fm_dma_issue<BITS, FM_AUX_KEEP>(slot, w, s, b, lane);
}

// this lane's codes and scale/bias words out of a landed slot
// (returns the slot's tag)
template <int BITS>
__device__ __forceinline__ uint32_t fm_dma_read(uint32_t slot, uint32_t woff, uint32_t soff,
                                                FmRowSlice<BITS> &t) {
    const uint32_t aw = slot + woff, as = slot + FmSlot<BITS>::WBYTES + soff;
    const uint32_t at = slot + FmSlot<BITS>::TAG;
    uint32_t tag;
    if constexpr (BITS == 3) {
        asm volatile("ds_read_b128 %0, %6\n\tds_read_b128 %1, %6 offset:16\n\t"
                     "ds_read_b128 %2, %6 offset:32\n\tds_read_b32 %3, %7\n\t"
                     "ds_read_b32 %4, %7 offset:256\n\tds_read_b32 %5, %8\n\t"
                     "s_waitcnt lgkmcnt(0)"
                     : "=&v"(t.q[0]), "=&v"(t.q[1]), "=&v"(t.q[2]), "=&v"(t.s), "=&v"(t.b),
                       "=&v"(tag)
                     : "v"(aw), "v"(as), "v"(at)
                     : "memory");
    } else if constexpr (BITS == 8) {
        asm volatile("ds_read_b128 %0, %11\n\tds_read_b128 %1, %11 offset:16\n\t"
                     "ds_read_b128 %2, %11 offset:32\n\tds_read_b128 %3, %11 offset:48\n\t"
                     "ds_read_b128 %4, %11 offset:64\n\tds_read_b128 %5, %11 offset:80\n\t"
                     "ds_read_b128 %6, %11 offset:96\n\tds_read_b128 %7, %11 offset:112\n\t"
                     "ds_read_b32 %8, %12\n\tds_read_b32 %9, %12 offset:256\n\t"
                     "ds_read_b32 %10, %13\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(t.q[0]), "=&v"(t.q[1]), "=&v"(t.q[2]), "=&v"(t.q[3]), "=&v"(t.q[4]),
                       "=&v"(t.q[5]), "=&v"(t.q[6]), "=&v"(t.q[7]), "=&v"(t.s), "=&v"(t.b), "=&v"(tag)
                     : "v"(aw), "v"(as), "v"(at)
                     : "memory");
    } else {
        asm volatile("ds_read_b128 %0, %7\n\tds_read_b128 %1, %7 offset:16\n\t"
                     "ds_read_b128 %2, %7 offset:32\n\tds_read_b128 %3, %7 offset:48\n\t"
                     "ds_read_b32 %4, %8\n\tds_read_b32 %5, %8 offset:256\n\t"
                     "ds_read_b32 %6, %9\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(t.q[0]), "=&v"(t.q[1]), "=&v"(t.q[2]), "=&v"(t.q[3]), "=&v"(t.s),
                       "=&v"(t.b), "=&v"(tag)
                     : "v"(aw), "v"(as), "v"(at)
                     : "memory");
    }
    return __builtin_amdgcn_readfirstlane(tag);
}

// Units of a segment are handed out one at a time from a counter in LDS: the
// hardware favours the older of two waves that share a SIMD, so with a fixed
// share per wave the favoured half finishes early and the CU runs the rest of
// the kernel half empty.  With a shared counter every wave of the workgroup
// ends within one unit of the others.
// (Written as an instruction: the compiler would make an LDS atomic wait for
// every outstanding LDS-direct load, which empties the ring.)
__device__ __forceinline__ uint32_t fm_claim_unit(unsigned int *next, int lane) {
    uint32_t v = 0;
    if (lane == 0) {
        const uint32_t addr = (uint32_t)(uintptr_t)(fm_lptr)next, one = 1u;
        asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(v)
                     : "v"(addr), "v"(one)
                     : "memory");
    }
    return __builtin_amdgcn_readfirstlane(v);
}

// tag of the slice in a slot (which unit it belongs to), kept in the slot's
// trailer so that the consumer needs no queue in registers
__device__ __forceinline__ void fm_slot_tag(uint32_t slot_tag_addr, uint32_t tag) {
    asm volatile("ds_write_b32 %0, %1" ::"v"(slot_tag_addr), "v"(tag) : "memory");
}
__device__ __forceinline__ uint32_t fm_slot_peek(uint32_t slot_tag_addr) {
    uint32_t tag;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(tag)
                 : "v"(slot_tag_addr)
                 : "memory");
    return __builtin_amdgcn_readfirstlane(tag);
}


// The intermediate vectors (act, expert_out) are written by one phase and read
// by the next, possibly inside one launch and from a CU behind another L2.
// They are stored and loaded as device-scope relaxed atomics: such accesses are
// performed at the level all CUs share, so a consumer that starts after the
// producer's stores have completed sees them without any cache maintenance.
__device__ __forceinline__ void fm_st_shared(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float fm_ld_shared(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// LDS words with explicit instructions (the compiler would order a visible LDS access behind
// every LDS-direct load in flight)
__device__ __forceinline__ void fm_lds_w32(uint32_t addr, uint32_t v) {
    asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ uint32_t fm_lds_r32(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
    return v;
}
// workgroup barrier that waits for this wave's LDS operations only (the compiler's own puts a
// wait for every LDS-direct load in front)
__device__ __forceinline__ void fm_wg_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Host side: raise a kernel's dynamic LDS limit above the 64 KB default, once per
// kernel and device (the attribute belongs to a device's copy of the kernel, and the
// runtime call costs more host time than a launch).
struct FmLdsAttr {
    bool set[64] = {};
};
inline bool fm_dyn_lds_ready(FmLdsAttr &a, const void *fn, size_t bytes) {
    int d = 0;
    (void)hipGetDevice(&d);
    const bool known = d >= 0 && d < 64;
    if (known && a.set[d]) return true;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess)
        return false;
    if (known) a.set[d] = true;
    return true;
}

#endif
