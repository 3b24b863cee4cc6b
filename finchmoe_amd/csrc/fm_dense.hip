// fm_dense.hip — dense affine-quantized GEMV: n tensors sharing one input
// vector, optionally over M positions.  Replaces dequant_matvec_4bit_v3 /
// _8bit / _3bit driven through BatchMatvecSpec (finchmoe/infer.m:3401-3411,
// 3528-3652; finchmoe/shaders.metal:374-463) and the M-position clone
// dequant_matvec_4bit_prefill (shaders.metal:2460-2529), whose grid is
// position x row tile exactly as here.
//
// Same lane mapping as the expert kernels: a lane owns 128 columns, LPR =
// in_dim/128 lanes share a row, a wave step covers 64/LPR rows that are
// contiguous in memory.
//
// Kernels: fm_dense_gemv (one workgroup per row tile, vector-ALU unpack: small launches),
// fm_dense_stream (one workgroup per CU, weight ring in LDS, matrix cores: launches with a wave
// step for every wave of the chip; up to two raw-BF16 tensors of a few rows can ride along at
// its end), fm_dense_gemv_mixed (tensors of different code widths in one launch, optionally with
// the token's routing done by the workgroup that finishes last), fm_dense_bf16 (unquantized
// BF16 tensors, cpu_dequant_matvec with scales == NULL, finchmoe/infer.m:1689-1701).
#include "fm_mfma.h"
#include "fm_ring.h"
#include "fm_route.h"

#include <type_traits>

#define FM_MAX_BATCH 8

struct FmDenseArgs {
    FmDenseSpec spec[FM_MAX_BATCH];
    int n;
    int in_dim;
    int rows_per_item;
    const float *x;      // [M][in_dim]
    size_t out_stride;   // elements between positions in every out (= out_dim of that tensor if 0)
    int unit_first[FM_MAX_BATCH + 1];   // streaming kernel: first wave step of every tensor
    // fm_dense_gemv_mixed only: the token's routing over tensor 0's outputs, run by the
    // workgroup that finishes last (route_ticket: a device word that is 0 between launches)
    int route_on;
    RouteArgs route;
    unsigned int *route_ticket;
    // fm_dense_stream only: raw-BF16 tensors of a few rows that ride along (one row per wave,
    // after the wave's share of the stream): rider r's rows are [rider_first[r], rider_first[r+1])
    int n_riders;
    FmDenseSpec rider[2];
    int rider_first[3];
};

namespace {

// the tensor a workgroup of the launch belongs to
__device__ __forceinline__ int fm_dense_which(const FmDenseArgs &a) {
    int t = 0;
#pragma unroll
    for (int i = 1; i < FM_MAX_BATCH; i++)
        if (i < a.n && (int)blockIdx.x >= a.spec[i].first_item) t = i;
    return t;
}

template <int BITS, int LPR, bool FP16>
__device__ __forceinline__ void fm_dense_gemv_rows(const FmDenseArgs &a, int t) {
    constexpr int RPS = FM_WAVE / LPR;
    constexpr int BPL = FmLaneBytes<BITS>::value;
    const FmDenseSpec sp = a.spec[t];
    const int chunk = blockIdx.x - sp.first_item;
    const int m = blockIdx.y;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane % LPR, r = lane / LPR;
    const FmGemvWave gw = fm_gemv_wave(chunk, wave, a.rows_per_item, LPR, sp.out_dim);
    const int row0 = gw.row0, steps = gw.steps;
    if (steps == 0) return;                  // (the wave comes back to its caller)
    const int row_bytes = a.in_dim * BITS / 8;
    const int sb_row_bytes = (a.in_dim / 64) * 2;
    const int last_row = sp.out_dim - 1;
    // rows past the end (only when out_dim is not a multiple of 64/LPR) re-read
    // the last row and are not stored
    auto rowc = [&](int row) { return fm_gemv_row_clamp(row, sp.out_dim); };
    int row = row0 + r;
    FmRowSlice<BITS> cur, next;
    {
        size_t ro = (size_t)rowc(row);
        fm_load_slice<BITS>(cur, sp.W + ro * row_bytes + (size_t)c * BPL,
                            sp.S + ro * sb_row_bytes + (size_t)c * 4,
                            sp.B + ro * sb_row_bytes + (size_t)c * 4);
    }
    float xs[FM_CPL], xsum0, xsum1;
    fm_load_x<BITS>(a.x + (size_t)m * a.in_dim + c * FM_CPL, xs, xsum0, xsum1);
    float *out = sp.out + (size_t)m * sp.out_dim;
    for (int it = 0; it < steps; it++) {
        if (it + 1 < steps) {
            size_t ro = (size_t)rowc(row + RPS);
            fm_load_slice<BITS>(next, sp.W + ro * row_bytes + (size_t)c * BPL,
                                sp.S + ro * sb_row_bytes + (size_t)c * 4,
                                sp.B + ro * sb_row_bytes + (size_t)c * 4);
        }
        float v = fm_group_sum<LPR>(fm_lane_dot<BITS, FP16>(cur, xs, xsum0, xsum1));
        if (c == 0 && row <= last_row) {
            // read later in this launch by another workgroup (the routing): stored at device scope
            if (a.route_on) __hip_atomic_store(out + row, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else out[row] = v;
        }
        row += RPS;
        cur = next;
    }
}

template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(256) void fm_dense_gemv(FmDenseArgs a) {
    fm_dense_gemv_rows<BITS, LPR, FP16>(a, fm_dense_which(a));
}

// Tensors of different code widths in one launch (the routing batch of a layer: the 8-bit
// router and the 4-bit shared-expert projections read the same x, finchmoe/infer.m:9285-9300;
// two launches cost twice the start-up latency, which is most of a launch this small).  Every
// workgroup runs the rows of one tensor with that tensor's arithmetic, exactly as the launch
// of one width does.
template <int LPR, bool FP16>
__global__ __launch_bounds__(256) void fm_dense_gemv_mixed(FmDenseArgs a) {
    const int t = fm_dense_which(a);
    switch (a.spec[t].bits) {
        case 3: fm_dense_gemv_rows<3, LPR, FP16>(a, t); break;
        case 8: fm_dense_gemv_rows<8, LPR, FP16>(a, t); break;
        default: fm_dense_gemv_rows<4, LPR, FP16>(a, t); break;
    }
    if (!a.route_on) return;
    // The routing (softmax, top-K, weights: fm_route.h) needs every logit: each workgroup takes
    // a ticket once its rows are in memory, and the one that draws the last runs it — the
    // pattern of the layer tail's norm (fm_tail.hip).
    __shared__ float route_p[FM_ROUTE_MAX];
    __shared__ unsigned int ticket;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this wave's rows are in memory
    __syncthreads();
    if (threadIdx.x == 0)
        ticket = __hip_atomic_fetch_add(a.route_ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (ticket != gridDim.x - 1 || threadIdx.x >= 64) return;
    __atomic_signal_fence(__ATOMIC_ACQUIRE);             // the loads below stay behind the ticket
    fm_route_wave<true>(a.route, route_p);
    if (threadIdx.x == 0)
        __hip_atomic_store(a.route_ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// one row of raw BF16 weights times x, by one wave (every lane receives the sum)
template <bool VEC>
__device__ __forceinline__ float fm_bf16_row(const uint16_t *w, const float *x, int in_dim, int lane) {
    float acc = 0.0f;
    if constexpr (VEC) {
        for (int c = lane * 8; c < in_dim; c += 64 * 8) {
            const uint4 q = *reinterpret_cast<const uint4 *>(w + c);
            const float4 x0 = *reinterpret_cast<const float4 *>(x + c);
            const float4 x1 = *reinterpret_cast<const float4 *>(x + c + 4);
            acc = fmaf(fm_bf16_lo(q.x), x0.x, acc);
            acc = fmaf(fm_bf16_hi(q.x), x0.y, acc);
            acc = fmaf(fm_bf16_lo(q.y), x0.z, acc);
            acc = fmaf(fm_bf16_hi(q.y), x0.w, acc);
            acc = fmaf(fm_bf16_lo(q.z), x1.x, acc);
            acc = fmaf(fm_bf16_hi(q.z), x1.y, acc);
            acc = fmaf(fm_bf16_lo(q.w), x1.z, acc);
            acc = fmaf(fm_bf16_hi(q.w), x1.w, acc);
        }
    } else {
        for (int c = lane; c < in_dim; c += 64)
            acc = fmaf(__uint_as_float((uint32_t)w[c] << 16), x[c], acc);
    }
    return fm_group_sum<64>(acc);
}

// ----------------------------------------------------------------------
// Streaming form (3-, 4- and 8-bit, in_dim up to 2048, or 4096 at 4 bits): the
// structure of the expert kernels (fm_decode.hip) without segments.  All wave
// steps ("units", 64/LPR rows) of all tensors of the launch form one sequence;
// workgroup g (12 waves, or 8 for the two forms that need the registers; one per CU) takes
// [U*g/G, U*(g+1)/G), its waves claim
// units from an LDS counter, copy their bytes into a per-wave ring in LDS with
// LDS-direct loads (two units in flight per wave, no destination registers)
// and multiply on the matrix cores against the activation registers, which the
// workgroup builds once.  in_dim = 4096 is two slabs of 2048 columns: a unit is
// two slices, each against its own activation registers, summed in slab order.
// 8-bit (the vocabulary projection, finchmoe/infer.m:5728-5760): same ring, two
// 8 KB units in flight per wave, multiply on the vector ALU.
// ----------------------------------------------------------------------
template <int BITS, int NS>
struct FmDenseRing {
    static constexpr int RING = FM_DENSE_RING, NW = FM_DENSE_NW(BITS, NS);
    static constexpr int BYTES = NW * RING * FmSlot<BITS>::BYTES;
};

template <int BITS, int LPR, int NS>
constexpr size_t fm_dense_stream_lds() {
    return FmDenseRing<BITS, NS>::BYTES + (BITS == 8 ? 0 : NS * sizeof(FmActLds<LPR>));
}

extern __shared__ __attribute__((aligned(16))) uint8_t fm_dense_lds[];

template <int BITS, int LPR, int NS, bool FP16>
__global__ __launch_bounds__(FM_DENSE_NW(BITS, NS) * 64) void fm_dense_stream(FmDenseArgs a, int total_units) {
#if defined(__HIP_DEVICE_COMPILE__)
    using SL = FmSlot<BITS>;
    constexpr int RPS = FM_WAVE / LPR, RING = FmDenseRing<BITS, NS>::RING;
    constexpr int SLAB_COLS = FM_CPL * LPR;
    constexpr int SLAB_ROW_BYTES = LPR * FmLaneBytes<BITS>::value, SLAB_SB = 4 * LPR;
    static_assert(NS == 1 || (SLAB_ROW_BYTES == 1024 && RPS == SL::NQ), "one load per row and slab");
    __shared__ unsigned int next_unit;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int m = blockIdx.y;
    const uint32_t ring0 = fm_lds_addr(fm_dense_lds) + (uint32_t)wave * (RING * SL::BYTES);
    FmActLds<LPR> *img = reinterpret_cast<FmActLds<LPR> *>(fm_dense_lds + FmDenseRing<BITS, NS>::BYTES);
    const int row_bytes = NS * SLAB_ROW_BYTES, sb_row_bytes = NS * SLAB_SB;
    const FmRange wg = fm_share(total_units, blockIdx.x, gridDim.x);
    const long wg0 = wg.lo;
    const uint32_t n_units = (uint32_t)(wg.hi - wg.lo);
    // The launch is a chain of memory round trips; the activations' is started first so
    // that it runs beside the counter set-up and the first weight loads instead of after them.
    typedef typename std::conditional<BITS == 8, FmBuildSlot<4>, FmBuildSlot<BITS>>::type BuildSlot;
    BuildSlot bslot;
    FmActX<LPR> xr[NS];
    if constexpr (BITS != 8) {
        bslot.init();
#pragma unroll
        for (int k = 0; k < NS; k++)
            if (threadIdx.x < 256)
                fm_act_load<BITS, LPR, false>(a.x + (size_t)m * a.in_dim + k * SLAB_COLS, bslot, xr[k]);
    }
    if (threadIdx.x == 0) next_unit = 0u;
    __syncthreads();                 // the counter is set
    uint32_t woff, soff;
    int ris, ch;
    fm_unit_lane_offsets<BITS, LPR>(lane, SLAB_ROW_BYTES, SLAB_SB, woff, soff, ris, ch);

    // unit u of the launch -> tensor and first row (no indexing of the argument arrays
    // with a run-time value: that would move them to private memory)
    struct Where {
        const uint8_t *W, *S, *B;
        float *out;
        int row0, out_dim;
    };
    auto locate = [&](long u) __attribute__((always_inline)) {
        Where w{a.spec[0].W, a.spec[0].S, a.spec[0].B, a.spec[0].out, 0, a.spec[0].out_dim};
        const int t = fm_dense_unit_tensor(a.unit_first, a.n, u);
        int first = 0;
#pragma unroll
        for (int i = 1; i < FM_MAX_BATCH; i++)
            if (i == t) {
                w.W = a.spec[i].W, w.S = a.spec[i].S, w.B = a.spec[i].B, w.out = a.spec[i].out;
                w.out_dim = a.spec[i].out_dim;
                first = a.unit_first[i];
            }
        w.row0 = (int)(u - first) * RPS;
        return w;
    };

    // ---- loader
    int kn = 0, wpos = 0;
    uint32_t issued = 0, consumed = 0, tag_n = 0;
    const uint8_t *wp = nullptr, *sp = nullptr, *bp = nullptr;
    bool dry = false;
    // one position: every weight byte is read once (fm_ring.h, FM_AUX_ONCE); with more positions
    // (gridDim.y) each of them reads the tensors again
    const bool once = gridDim.y == 1;
    auto issue = [&]() __attribute__((always_inline)) {
        if (dry) return;
        if (kn == 0) {
            const uint32_t ul = fm_claim_unit(&next_unit, lane);
            if (ul >= n_units) {
                dry = true;
                return;
            }
            const Where w = locate(wg0 + ul);
            wp = fm_uniform(w.W + (size_t)w.row0 * row_bytes);
            sp = fm_uniform(w.S + (size_t)w.row0 * sb_row_bytes);
            bp = fm_uniform(w.B + (size_t)w.row0 * sb_row_bytes);
            tag_n = ul;
        }
        const uint32_t slot = ring0 + (uint32_t)wpos * SL::BYTES;
        fm_slot_tag(slot + SL::TAG, tag_n);
        if constexpr (NS == 1) {
            fm_dma_issue_as<BITS>(once, slot, wp, sp, bp, lane);
        } else {
            // slab kn of the unit's rows: one 1 KB run per row, 64 B of scales / biases per row
            const uint32_t so = fm_dense_slab_sboff(kn, lane, sb_row_bytes, SLAB_SB);
#define FM_DENSE_SLAB_LOADS(AUX)                                                                        \
    do {                                                                                                \
        _Pragma("unroll") for (int i = 0; i < RPS; i++) __builtin_amdgcn_global_load_lds(               \
            (fm_gptr)(uintptr_t)(wp + fm_dense_slab_woff(i, kn, lane, row_bytes, SLAB_ROW_BYTES)),      \
            (fm_lptr)(uintptr_t)(slot + 1024 * i), 16, 0, AUX);                                         \
        __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(sp + so),                                 \
                                         (fm_lptr)(uintptr_t)(slot + SL::WBYTES), 4, 0, AUX);           \
        __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(bp + so),                                 \
                                         (fm_lptr)(uintptr_t)(slot + SL::WBYTES + 256), 4, 0, AUX);     \
    } while (0)
            if (once) FM_DENSE_SLAB_LOADS(FM_AUX_ONCE);
            else FM_DENSE_SLAB_LOADS(FM_AUX_KEEP);
#undef FM_DENSE_SLAB_LOADS
        }
        kn = kn + 1 == NS ? 0 : kn + 1;
        wpos = wpos + 1 == RING ? 0 : wpos + 1;
        issued++;
    };
#pragma unroll
    for (int k = 0; k < RING; k++) issue();      // the weights do not wait for the activations

    if constexpr (BITS == 8) {
        // A byte does not fit a bf16 mantissa, and at one byte per code the vector ALU has
        // time for convert + multiply-add: the plain dot product against the lane's 128
        // activations, fed from the ring.
        static_assert(BITS != 8 || NS == 1, "one slab");
        float xs[FM_CPL], xsum0, xsum1;
        fm_load_x<8>(a.x + (size_t)m * a.in_dim + ch * FM_CPL, xs, xsum0, xsum1);
        int c8 = 0;
        while (consumed < issued) {
            FmRowSlice<BITS> t;
            if (issued - consumed == (uint32_t)RING) fm_dma_wait<SL::LOADS *(RING - 1)>(false);
            else fm_dma_wait<0>(true);
            const uint32_t tag = fm_dma_read<BITS>(ring0 + (uint32_t)c8 * SL::BYTES, woff, soff, t);
            consumed++;
            c8 = c8 + 1 == RING ? 0 : c8 + 1;
            issue();
            const float v = fm_chunk_sum<LPR>(fm_lane_dot<BITS, FP16>(t, xs, xsum0, xsum1));
            const Where w = locate(wg0 + tag);
            if (ch == 0) w.out[(size_t)m * w.out_dim + w.row0 + ris] = v;
        }
    } else {
    // the activation registers of every slab, built once (the activations were requested
    // at the kernel's start)
#pragma unroll
    for (int k = 0; k < NS; k++)
        if (threadIdx.x < 256) fm_act_build<BITS, LPR>(xr[k], bslot, img[k]);
    __syncthreads();
    FmActRegs ar[NS];
#pragma unroll
    for (int k = 0; k < NS; k++) fm_read_act_lds<LPR>(img[k], lane, ar[k]);

    int c = 0;
    while (consumed < issued) {
        float v = 0.0f;
        uint32_t tag = 0;
#pragma unroll
        for (int k = 0; k < NS; k++) {
            FmRowSlice<BITS> t;
            if (issued - consumed == (uint32_t)RING) fm_dma_wait<SL::LOADS *(RING - 1)>(false);
            else fm_dma_wait<0>(true);
            tag = fm_dma_read<BITS>(ring0 + (uint32_t)c * SL::BYTES, woff, soff, t);
            consumed++;
            c = c + 1 == RING ? 0 : c + 1;
            issue();
            v += fm_chunk_sum<LPR>(fm_lane_dot_mfma<BITS, FP16>(t, ar[k]));
        }
        const Where w = locate(wg0 + tag);
        if (ch == 0) w.out[(size_t)m * w.out_dim + w.row0 + ris] = v;
    }
    }
    // riders: wave gw of the launch takes row gw of the raw-BF16 tensors (the in_proj_b /
    // in_proj_a rows next to in_proj_qkv / in_proj_z: finchmoe/infer.m:8118-8122), so that the
    // set is one launch
    if (a.n_riders > 0) {
        int row = 0;
        const int r = fm_dense_rider_of(a.rider_first, a.n_riders, (int)blockIdx.x * FM_DENSE_NW(BITS, NS) + wave, &row);
        if (r >= 0) {
            const FmDenseSpec sp = r ? a.rider[1] : a.rider[0];
            const uint16_t *w = reinterpret_cast<const uint16_t *>(sp.W) + (size_t)row * a.in_dim;
            const float *x = a.x + (size_t)m * a.in_dim;
            const bool vec = a.in_dim % 8 == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0;
            const float acc = vec ? fm_bf16_row<true>(w, x, a.in_dim, lane) : fm_bf16_row<false>(w, x, a.in_dim, lane);
            if (lane == 0) sp.out[(size_t)m * sp.out_dim + row] = acc;
        }
    }
#else
    (void)a;
    (void)total_units;
#endif
}

// launches the streaming kernel when the shapes allow it; FM_ERR_UNSUPPORTED otherwise
template <int BITS, bool FP16>
int launch_dense_stream_t(FmDenseArgs &a, int M, int n_cu, hipStream_t st) {
    if (BITS == 8 && ((uintptr_t)a.x & 15)) return FM_ERR_UNSUPPORTED;
    int out_dims[FM_MAX_BATCH];
    for (int i = 0; i < a.n; i++) out_dims[i] = a.spec[i].out_dim;
    // (decided by the tensor shapes alone, so that M positions and one position take the same
    // kernel and stay bitwise equal; worth it only when every wave of the chip gets a unit: below
    // that the launch is a chain of latencies either way, and the plain kernel's chain is shorter —
    // 2048 rows of 4096 columns take 6.0 us there and 12.4 us here)
    const FmDensePlan plan = fm_dense_stream_plan(out_dims, a.n, a.in_dim, BITS, n_cu);
    if (!plan.ok) return FM_ERR_UNSUPPORTED;
    for (int i = 0; i <= FM_MAX_BATCH; i++) a.unit_first[i] = plan.unit_first[i];
    const int ns = plan.ns, lpr = plan.lpr, units = plan.units;
    const long wgs = plan.wgs;
    if (a.n_riders > 0 && a.rider_first[a.n_riders] > plan.nw * wgs) a.n_riders = 0;   // one row per wave
    dim3 grid((unsigned)wgs, M);
#define FM_DS(L, NS_)                                                                          \
    do {                                                                                       \
        auto kfn = fm_dense_stream<BITS, L, NS_, FP16>;                                        \
        const size_t sh = fm_dense_stream_lds<BITS, L, NS_>();                                 \
        static FmLdsAttr attr;                                                                 \
        if (!fm_dyn_lds_ready(attr, (const void *)kfn, sh)) return FM_ERR_HIP;                 \
        hipLaunchKernelGGL(kfn, grid, dim3(FM_DENSE_NW(BITS, NS_) * 64), sh, st, a, units);    \
    } while (0)
    if (ns == 2) {
        if constexpr (BITS == 4) FM_DS(16, 2);
    } else {
        switch (lpr) {
            case 4: FM_DS(4, 1); break;
            case 8: FM_DS(8, 1); break;
            default: FM_DS(16, 1); break;
        }
    }
#undef FM_DS
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

template <int BITS, bool FP16>
int launch_dense_t(const FmDenseArgs &a, int total_items, int M, hipStream_t st) {
    dim3 grid(total_items, M), b(256);
#define FM_D(L) hipLaunchKernelGGL((fm_dense_gemv<BITS, L, FP16>), grid, b, 0, st, a)
    switch (a.in_dim / FM_CPL) {
        case 1: FM_D(1); break;
        case 2: FM_D(2); break;
        case 4: FM_D(4); break;
        case 8: FM_D(8); break;
        case 16: FM_D(16); break;
        case 32: FM_D(32); break;
        case 64: FM_D(64); break;
        default: return FM_ERR_UNSUPPORTED;
    }
#undef FM_D
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

// ----------------------------------------------------------------------
// Raw BF16 weights [out_dim][in_dim] (cpu_dequant_matvec with scales == NULL,
// finchmoe/infer.m:1689-1701): the tensors the reference's quantizer leaves
// unquantized (mlp.gate, shared_expert_gate, in_proj_a, in_proj_b:
// finchmoe/quantize_non_experts.py:103-107).  One wave per row: a lane takes
// eight weights per 128-bit load (bf16 -> fp32 is a shift), fp32 accumulate, sum
// over the wave.  VEC: rows are 16-byte aligned and in_dim is a multiple of 8.
// ----------------------------------------------------------------------
template <bool VEC>
__global__ __launch_bounds__(256) void fm_dense_bf16(FmDenseArgs a, int total_rows) {
    const int lane = threadIdx.x & 63;
    const int gr = blockIdx.x * 4 + (threadIdx.x >> 6);   // row of the launch (wave-uniform)
    if (gr >= total_rows) return;
    int t = 0;
#pragma unroll
    for (int i = 1; i < FM_MAX_BATCH; i++)
        if (i < a.n && gr >= a.unit_first[i]) t = i;
    const FmDenseSpec sp = a.spec[t];
    const int row = gr - a.unit_first[t];
    const int m = blockIdx.y;
    const float acc = fm_bf16_row<VEC>(reinterpret_cast<const uint16_t *>(sp.W) + (size_t)row * a.in_dim,
                                       a.x + (size_t)m * a.in_dim, a.in_dim, lane);
    if (lane == 0) sp.out[(size_t)m * sp.out_dim + row] = acc;
}

// ----------------------------------------------------------------------
// 1- and 2-bit affine tensors (cpu_dequant_matvec's generic branch, finchmoe/infer.m:1734-1760:
// 32 / 16 codes per little-endian u32, LSB first; the legacy widths of the reference's tensor
// boundary, in none of its benchmark configurations).  One wave per row: a lane takes whole
// words (a word never straddles a group of 64), per word s * sum(q x) + b * sum(x) in fp32, sum
// over the wave.
// ----------------------------------------------------------------------
template <int BITS, bool FP16>
__global__ __launch_bounds__(256) void fm_dense_lowbit(FmDenseArgs a, int total_rows) {
    constexpr int VPU = 32 / BITS;
    const int lane = threadIdx.x & 63;
    const int gr = blockIdx.x * 4 + (threadIdx.x >> 6);   // row of the launch (wave-uniform)
    if (gr >= total_rows) return;
    int t = 0;
#pragma unroll
    for (int i = 1; i < FM_MAX_BATCH; i++)
        if (i < a.n && gr >= a.unit_first[i]) t = i;
    const FmDenseSpec sp = a.spec[t];
    const int row = gr - a.unit_first[t];
    const int m = blockIdx.y;
    const int words = a.in_dim / VPU, ng = a.in_dim / 64;
    const uint32_t *w = reinterpret_cast<const uint32_t *>(sp.W) + (size_t)row * words;
    const uint16_t *S = reinterpret_cast<const uint16_t *>(sp.S) + (size_t)row * ng;
    const uint16_t *B = reinterpret_cast<const uint16_t *>(sp.B) + (size_t)row * ng;
    const float *x = a.x + (size_t)m * a.in_dim;
    float acc = 0.0f;
    for (int wi = lane; wi < words; wi += 64) {
        const uint32_t q = w[wi];
        const int col0 = wi * VPU, g = col0 >> 6;
        const float sc = FP16 ? fm_fp16_bits(S[g]) : fm_bf16_lo(S[g]);
        const float bs = FP16 ? fm_fp16_bits(B[g]) : fm_bf16_lo(B[g]);
        float dq = 0.0f, dx = 0.0f;
#pragma unroll
        for (int j = 0; j < VPU; j++) {
            const float xv = x[col0 + j];
            dq = fmaf((float)((q >> (j * BITS)) & ((1u << BITS) - 1u)), xv, dq);
            dx += xv;
        }
        acc = fmaf(sc, dq, fmaf(bs, dx, acc));
    }
    acc = fm_group_sum<64>(acc);
    if (lane == 0) sp.out[(size_t)m * sp.out_dim + row] = acc;
}

}  // namespace

// n 1- or 2-bit affine tensors [out_dim][in_dim] (in_dim a multiple of 64) sharing x[M][in_dim]
extern "C" int fm_launch_dense_lowbit(const FmDenseSpec *specs, int n, int in_dim, int bits, int scale_fp16,
                                      const float *d_x, int M, hipStream_t st) {
    if (n < 1 || n > FM_MAX_BATCH || M < 1 || in_dim < 64 || in_dim % 64 || (bits != 1 && bits != 2))
        return FM_ERR_ARG;
    FmDenseArgs a;
    a.n = n;
    a.in_dim = in_dim;
    a.rows_per_item = 0;
    a.x = d_x;
    a.out_stride = 0;
    a.route_on = 0;
    a.n_riders = 0;
    int rows = 0;
    for (int i = 0; i < n; i++) {
        a.spec[i] = specs[i];
        a.unit_first[i] = rows;
        rows += specs[i].out_dim;
    }
    for (int i = n; i < FM_MAX_BATCH; i++) a.spec[i] = a.spec[0];
    for (int i = n; i <= FM_MAX_BATCH; i++) a.unit_first[i] = rows;
    const dim3 grid((rows + 3) / 4, M);
    if (bits == 1) {
        if (scale_fp16) hipLaunchKernelGGL((fm_dense_lowbit<1, true>), grid, dim3(256), 0, st, a, rows);
        else hipLaunchKernelGGL((fm_dense_lowbit<1, false>), grid, dim3(256), 0, st, a, rows);
    } else {
        if (scale_fp16) hipLaunchKernelGGL((fm_dense_lowbit<2, true>), grid, dim3(256), 0, st, a, rows);
        else hipLaunchKernelGGL((fm_dense_lowbit<2, false>), grid, dim3(256), 0, st, a, rows);
    }
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

// n raw-BF16 tensors [out_dim][in_dim] sharing x[M][in_dim]; specs[i].S / .B are unused.
extern "C" int fm_launch_dense_bf16(const FmDenseSpec *specs, int n, int in_dim, const float *d_x,
                                    int M, hipStream_t st) {
    if (n < 1 || n > FM_MAX_BATCH || M < 1 || in_dim < 1) return FM_ERR_ARG;
    FmDenseArgs a;
    a.n = n;
    a.in_dim = in_dim;
    a.rows_per_item = 0;
    a.x = d_x;
    a.out_stride = 0;
    a.route_on = 0;
    a.n_riders = 0;
    int rows = 0;
    bool vec = in_dim % 8 == 0 && ((uintptr_t)d_x & 15) == 0;
    for (int i = 0; i < n; i++) {
        a.spec[i] = specs[i];
        a.unit_first[i] = rows;
        rows += specs[i].out_dim;
        vec = vec && ((uintptr_t)specs[i].W & 15) == 0;
    }
    for (int i = n; i < FM_MAX_BATCH; i++) a.spec[i] = a.spec[0];
    for (int i = n; i <= FM_MAX_BATCH; i++) a.unit_first[i] = rows;
    const dim3 grid((rows + 3) / 4, M);
    if (vec) hipLaunchKernelGGL(fm_dense_bf16<true>, grid, dim3(256), 0, st, a, rows);
    else hipLaunchKernelGGL(fm_dense_bf16<false>, grid, dim3(256), 0, st, a, rows);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

// Tensors of different widths (specs[i].bits in {3, 4, 8}), one position, plain kernel.
// route (optional): the routing over specs[0]'s outputs in the same launch; ticket: a device word
// that is zero between launches.
extern "C" int fm_launch_dense_mixed(FmDenseSpec *specs, int n, int in_dim, int scale_fp16,
                                     const float *d_x, int n_cu, const RouteArgs *route,
                                     unsigned int *ticket, hipStream_t st) {
    if (n < 1 || n > FM_MAX_BATCH) return FM_ERR_ARG;
    const int lpr = in_dim / FM_CPL;
    if (lpr < 1 || lpr > 64 || (lpr & (lpr - 1)) || in_dim % FM_CPL) return FM_ERR_UNSUPPORTED;
    long total_rows = 0;
    for (int i = 0; i < n; i++) {
        if (specs[i].bits != 3 && specs[i].bits != 4 && specs[i].bits != 8) return FM_ERR_UNSUPPORTED;
        total_rows += specs[i].out_dim;
    }
    const int rpi = fm_gemv_rows_per_item(total_rows, 1, lpr, n_cu);     // as fm_launch_dense
    FmDenseArgs a;
    a.n = n;
    a.in_dim = in_dim;
    a.rows_per_item = rpi;
    a.x = d_x;
    a.out_stride = 0;
    a.route_on = 0;
    a.n_riders = 0;
    int items = 0;
    for (int i = 0; i < n; i++) {
        specs[i].first_item = items;
        items += (specs[i].out_dim + rpi - 1) / rpi;
        a.spec[i] = specs[i];
    }
    for (int i = n; i < FM_MAX_BATCH; i++) a.spec[i] = a.spec[0];
    a.route_on = 0;
    a.n_riders = 0;
    if (route) {
        if (!ticket || route->n < 1 || route->n > FM_ROUTE_MAX || route->K < 1 || route->K > FM_MAX_K ||
            route->K > route->n || route->n != specs[0].out_dim)
            return FM_ERR_UNSUPPORTED;
        a.route_on = 1;
        a.route = *route;
        a.route_ticket = ticket;
    }
    const dim3 grid(items), b(256);
#define FM_DM(L)                                                                           \
    do {                                                                                   \
        if (scale_fp16) hipLaunchKernelGGL((fm_dense_gemv_mixed<L, true>), grid, b, 0, st, a);  \
        else hipLaunchKernelGGL((fm_dense_gemv_mixed<L, false>), grid, b, 0, st, a);       \
    } while (0)
    switch (lpr) {
        case 1: FM_DM(1); break;
        case 2: FM_DM(2); break;
        case 4: FM_DM(4); break;
        case 8: FM_DM(8); break;
        case 16: FM_DM(16); break;
        case 32: FM_DM(32); break;
        case 64: FM_DM(64); break;
        default: return FM_ERR_UNSUPPORTED;
    }
#undef FM_DM
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

// specs[i].first_item is filled here.  in_dim must be 128 * 2^j, j <= 6.
// riders (optional, at most two): raw-BF16 tensors of a few rows computed in the same launch when
// the streaming kernel takes it; *riders_done says whether they were.
extern "C" int fm_launch_dense(FmDenseSpec *specs, int n, int in_dim, int bits, int scale_fp16,
                               const float *d_x, int M, int n_cu, hipStream_t st,
                               const FmDenseSpec *riders, int n_riders, int *riders_done) {
    if (riders_done) *riders_done = 0;
    if (n < 1 || n > FM_MAX_BATCH || M < 1) return FM_ERR_ARG;
    const int lpr = in_dim / FM_CPL;
    if (lpr < 1 || lpr > 64 || (lpr & (lpr - 1)) || in_dim % FM_CPL) return FM_ERR_UNSUPPORTED;
    long total_rows = 0;
    for (int i = 0; i < n; i++) total_rows += specs[i].out_dim;
    // Rows per workgroup: the register budget keeps two workgroups per CU resident, and a
    // launch that needs a second round of workgroups pays its start-up latencies twice —
    // so grow the tile until the launch fits in one round (or the tile is 8 steps deep).
    const int rpi = fm_gemv_rows_per_item(total_rows, M, lpr, n_cu);
    FmDenseArgs a;
    a.n = n;
    a.in_dim = in_dim;
    a.rows_per_item = rpi;
    a.x = d_x;
    a.out_stride = 0;
    a.route_on = 0;
    a.n_riders = 0;
    int items = 0;
    for (int i = 0; i < n; i++) {
        specs[i].first_item = items;
        items += (specs[i].out_dim + rpi - 1) / rpi;
        a.spec[i] = specs[i];
    }
    for (int i = n; i < FM_MAX_BATCH; i++) a.spec[i] = a.spec[0];
    const bool no_stream = (fm_kernel_forms & FM_FORM_PLAIN_DENSE) != 0;
    if (!no_stream && (bits == 3 || bits == 4 || bits == 8)) {
        if (riders && n_riders >= 1 && n_riders <= 2 && riders_done) {
            a.n_riders = n_riders;
            a.rider_first[0] = 0;
            for (int i = 0; i < n_riders; i++) {
                a.rider[i] = riders[i];
                a.rider_first[i + 1] = a.rider_first[i] + riders[i].out_dim;
            }
            for (int i = n_riders; i < 2; i++) {
                a.rider[i] = a.rider[0];
                a.rider_first[i + 1] = a.rider_first[n_riders];
            }
        }
        int rc = FM_ERR_UNSUPPORTED;
        if (bits == 3) rc = scale_fp16 ? launch_dense_stream_t<3, true>(a, M, n_cu, st)
                                       : launch_dense_stream_t<3, false>(a, M, n_cu, st);
        else if (bits == 8) rc = scale_fp16 ? launch_dense_stream_t<8, true>(a, M, n_cu, st)
                                            : launch_dense_stream_t<8, false>(a, M, n_cu, st);
        else rc = scale_fp16 ? launch_dense_stream_t<4, true>(a, M, n_cu, st)
                             : launch_dense_stream_t<4, false>(a, M, n_cu, st);
        if (rc != FM_ERR_UNSUPPORTED) {
            if (riders_done && rc == FM_OK) *riders_done = a.n_riders > 0;
            return rc;
        }
        a.n_riders = 0;
    }
    switch (bits) {
        case 3: return scale_fp16 ? launch_dense_t<3, true>(a, items, M, st)
                                  : launch_dense_t<3, false>(a, items, M, st);
        case 4: return scale_fp16 ? launch_dense_t<4, true>(a, items, M, st)
                                  : launch_dense_t<4, false>(a, items, M, st);
        case 8: return scale_fp16 ? launch_dense_t<8, true>(a, items, M, st)
                                  : launch_dense_t<8, false>(a, items, M, st);
        default: return FM_ERR_UNSUPPORTED;
    }
}
