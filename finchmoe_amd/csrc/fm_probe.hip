// fm_probe.hip — the streaming ceiling of the memory system, measured the way the expert
// kernels read: one workgroup of twelve waves per CU, every wave a ring of two 4 KB slots in LDS
// filled with LDS-direct 16-byte loads, no arithmetic; three orders in which the waves walk
// the buffer (with two waves per SIMD the rate depended on the order by up to 5 %; with three
// it hardly does).
// What this kernel reaches is what a bandwidth-bound kernel of that structure can reach at
// best; the decode kernels are priced against the published peak and compared with this.
// No counterpart in the reference (a measurement aid, like its --timing accumulators,
// finchmoe/infer.m:281-298).
#include "fm_index.h"
#include "fm_ring.h"

namespace {

constexpr int PROBE_WAVES = FM_PROBE_WAVES;
constexpr int PROBE_RING = FM_PROBE_RING;
constexpr int PROBE_SLOT = 4096;       // 4 loads of 64 lanes x 16 bytes

extern __shared__ __attribute__((aligned(16))) uint8_t fm_probe_lds[];

// PATTERN: which 4 KB slots a wave reads, in order
//   0  dense: slot i of the buffer goes to wave i % (all waves of the grid) — at any moment the
//      chip reads one contiguous window
//   1  every workgroup a contiguous share, its waves interleaved over it (the order of
//      the expert decode kernels)
//   2  every wave a contiguous share
//   3, 4, 5  groups of 4 / 8 / 8 workgroups share a contiguous region whose slots go to the
//      group's waves in turn (5: the eight workgroups of a group sit on one XCD)
//   6  as 1 with neighbouring shares on one XCD;  7  groups of 4 workgroups of one XCD
// AUX: the loads' cache policy — FM_AUX_ONCE as the decode kernels read weights (fm_ring.h), or
// FM_AUX_KEEP, ordinary caching (patterns 8..15 = 0..7 with it).
template <int PATTERN, int AUX>
__global__ __launch_bounds__(PROBE_WAVES * 64) void fm_stream_probe_k(const uint8_t *buf, size_t n_slots,
                                                                      unsigned int *sink) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t ring0 = fm_lds_addr(fm_probe_lds) + (uint32_t)wave * (PROBE_RING * PROBE_SLOT);
    const FmProbeWalk pw = fm_probe_walk(PATTERN, n_slots, blockIdx.x, gridDim.x, wave, PROBE_WAVES);
    size_t next = pw.next;
    const size_t end = pw.end, step = pw.step;
    uint32_t issued = 0, consumed = 0;
    int wpos = 0, c = 0;
    auto issue = [&]() __attribute__((always_inline)) {
        if (next >= end) return;
        const uint8_t *src = fm_uniform(buf + next * PROBE_SLOT) + lane * 16;
        const uint32_t slot = ring0 + (uint32_t)wpos * PROBE_SLOT;
#pragma unroll
        for (int j = 0; j < 4; j++)
            __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(src + 1024 * j),
                                             (fm_lptr)(uintptr_t)(slot + 1024 * j), 16, 0, AUX);
        next += step;
        wpos = wpos + 1 == PROBE_RING ? 0 : wpos + 1;
        issued++;
    };
#pragma unroll
    for (int k = 0; k < PROBE_RING; k++) issue();
    uint32_t acc = 0;
    while (consumed < issued) {
        if (issued - consumed == (uint32_t)PROBE_RING) fm_dma_wait<4 * (PROBE_RING - 1)>(false);
        else fm_dma_wait<0>(true);
        // one dword of the landed slot per lane, so that the data is really consumed
        uint32_t v;
        const uint32_t addr = ring0 + (uint32_t)c * PROBE_SLOT + 4 * lane;
        asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
        acc ^= v;
        consumed++;
        c = c + 1 == PROBE_RING ? 0 : c + 1;
        issue();
    }
    if (acc == 0x9E3779B9u && sink) *sink = acc;     // practically never: keeps `acc` alive
}

}  // namespace

// reads nbytes (rounded down to whole 4 KB slots) of d_buf once, in the given pattern
// (0..7 with the non-temporal hint, 8..15 the same walks with ordinary caching)
extern "C" int fm_launch_stream_probe(const void *d_buf, size_t nbytes, int pattern, unsigned int *d_sink,
                                      int n_cu, hipStream_t st) {
    const size_t n_slots = nbytes / PROBE_SLOT;
    if (!d_buf || n_slots == 0 || ((uintptr_t)d_buf & 15) || pattern < 0 || pattern > 15) return FM_ERR_ARG;
    const size_t sh = (size_t)PROBE_WAVES * PROBE_RING * PROBE_SLOT;
    static FmLdsAttr attr[16];
    typedef void (*probe_fn)(const uint8_t *, size_t, unsigned int *);
#define FM_PROBE_FNS(AUX)                                                                                  \
    fm_stream_probe_k<0, AUX>, fm_stream_probe_k<1, AUX>, fm_stream_probe_k<2, AUX>, fm_stream_probe_k<3, AUX>, \
        fm_stream_probe_k<4, AUX>, fm_stream_probe_k<5, AUX>, fm_stream_probe_k<6, AUX>, fm_stream_probe_k<7, AUX>
    static const probe_fn fns[16] = {FM_PROBE_FNS(FM_AUX_ONCE), FM_PROBE_FNS(FM_AUX_KEEP)};
#undef FM_PROBE_FNS
    if (!fm_dyn_lds_ready(attr[pattern], (const void *)fns[pattern], sh)) return FM_ERR_HIP;
    const dim3 grid(n_cu), block(PROBE_WAVES * 64);
    const uint8_t *b = (const uint8_t *)d_buf;
    hipLaunchKernelGGL(fns[pattern], grid, block, sh, st, b, n_slots, d_sink);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}
