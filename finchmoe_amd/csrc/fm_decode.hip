// fm_decode.hip — routed-expert decode for affine-packed experts:
//   kernel 1  gate GEMV + up GEMV + SwiGLU for every (layer, slot) pair
//   kernel 2  down GEMV per pair -> per-expert output vectors
//   kernel 3  router-weighted sum of the K vectors of a layer, in slot order
// Replaces the four dispatches per expert of gpu_encode_experts_batched
// (finchmoe/infer.m:4337-4378: dequant_matvec_3bit x3 + swiglu_fused) and the
// weighted sum of moe_combine_residual (finchmoe/shaders.metal:2213-2228).
//
// Work decomposition.  A pair p = (layer l, slot k) selects expert idx[l][k].
// A 256-thread workgroup (4 waves) takes `rows_per_item` consecutive output
// rows of one pair.  Inside a wave, LPR = in_dim/128 adjacent lanes share a
// row (each owns 128 columns, see fm_unpack.h), so one wave step covers
// 64/LPR rows, read as one contiguous run of memory:
//   gate/up (in 2048): 16 lanes x 48 B = one 768-byte row, 4 rows per step
//   down    (in 512):   4 lanes x 48 B = one 192-byte row, 16 rows per step
// The scales (and biases) of those rows are contiguous too — [rows][groups]
// 16-bit, two groups per lane = one dword per lane.
//
// What the file holds, in order: the three plain kernels above (fm_gate_up_swiglu, fm_down,
// fm_combine: any shape, registers only); the streaming forms of the first two
// (fm_gate_up_swiglu_lds, fm_down_lds: weight ring in LDS filled by LDS-direct loads, inner
// product on the matrix cores); fm_moe_fused, the three phases as one persistent launch with
// dependency counters per vector (the form that keeps the per-expert vectors and the finite
// guard); fm_moe_fused_rows, the launch that sums a row block's experts in LDS and writes only
// the layer's output (the default when nobody asks for the per-expert vectors); the launchers.
// All of them add the K experts of a row in slot order with the same arithmetic, so their
// results are equal bit for bit.
#include "fm_index.h"
#include "fm_mfma.h"
#include "fm_ring.h"
#include "fm_route.h"

#include <type_traits>

namespace {

// Waves per workgroup of the streaming kernels: one workgroup per CU, three waves per SIMD (the
// kernels need up to 160 vector registers, so three is the most), each with a ring of two
// slices.  Measured on the 40-layer step with the non-temporal loads: 8 waves with rings of 4 /
// 3 / 2 slices 86.3 / 86.3 / 84.7 us — the ring's depth buys nothing, the memory pipeline takes
// fewer requests than the rings hold — and 12 waves with rings of 2, the same LDS, 82.5 us: a
// third wave per SIMD covers part of what the multiply of the other two leaves uncovered.
constexpr int FM_NW = 12;

struct DecodeArgs {
    const uint8_t *const *layer_ptrs;   // [n_layers] device pointers to layer blobs
    FmExpertGeom g;
    int layer0;
    int layer_stride;   // 1: pair group l is layer layer0+l; 0: all groups use layer0 (positions of a chunk)
    int K;
    const float *x;          // [nl][hidden]
    const int32_t *idx;      // [nl][K]
    const float *w;          // [nl][K]
    float *act;              // [nl][K][inter]   scratch
    float *expert_out;       // [nl][K][hidden]
    float *out;              // [nl][hidden]
    int rows_per_item;
    int items_per_pair;
    int flags;
};


// ---------------------------------------------------------------- kernel 1
template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(256) void fm_gate_up_swiglu(DecodeArgs a) {
    constexpr int RPS = FM_WAVE / LPR;   // rows per wave step
    constexpr int BPL = FmLaneBytes<BITS>::value;
    const int item = blockIdx.x;
    const int pair = item / a.items_per_pair;
    const int chunk = item - pair * a.items_per_pair;
    const int l = pair / a.K;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane % LPR, r = lane / LPR;
    const int rows_per_wave = a.rows_per_item >> 2;
    const int row0 = chunk * a.rows_per_item + wave * rows_per_wave;
    float *act = a.act + (size_t)pair * a.g.inter;

    const int e = a.idx[pair];
    if ((unsigned)e >= (unsigned)a.g.n_experts) {   // treated as weight 0
        for (int i = lane; i < rows_per_wave; i += FM_WAVE) act[row0 + i] = 0.0f;
        return;
    }
    const uint8_t *blob = a.layer_ptrs[a.layer0 + l * a.layer_stride] + (size_t)e * a.g.expert_size;
    const int row_bytes = a.g.hidden * BITS / 8;
    const int sb_row_bytes = (a.g.hidden / 64) * 2;

    // issue the first weight loads before the activation loads
    size_t woff = (size_t)(row0 + r) * row_bytes + (size_t)c * BPL;
    size_t soff = (size_t)(row0 + r) * sb_row_bytes + (size_t)c * 4;
    const size_t wstep = (size_t)RPS * row_bytes, sstep = (size_t)RPS * sb_row_bytes;
    FmRowSlice<BITS> gcur, ucur, gnext, unext;
    fm_load_slice<BITS>(gcur, blob + a.g.gate_w + woff, blob + a.g.gate_s + soff,
                        blob + a.g.gate_b + soff);
    fm_load_slice<BITS>(ucur, blob + a.g.up_w + woff, blob + a.g.up_s + soff,
                        blob + a.g.up_b + soff);

    float xs[FM_CPL], xsum0, xsum1;
    fm_load_x<BITS>(a.x + (size_t)l * a.g.hidden + c * FM_CPL, xs, xsum0, xsum1);

    const int steps = rows_per_wave / RPS;
    for (int it = 0; it < steps; it++) {
        if (it + 1 < steps) {
            woff += wstep;
            soff += sstep;
            fm_load_slice<BITS>(gnext, blob + a.g.gate_w + woff, blob + a.g.gate_s + soff,
                                blob + a.g.gate_b + soff);
            fm_load_slice<BITS>(unext, blob + a.g.up_w + woff, blob + a.g.up_s + soff,
                                blob + a.g.up_b + soff);
        }
        float gv = fm_group_sum<LPR>(fm_lane_dot<BITS, FP16>(gcur, xs, xsum0, xsum1));
        float uv = fm_group_sum<LPR>(fm_lane_dot<BITS, FP16>(ucur, xs, xsum0, xsum1));
        if (c == 0) act[row0 + it * RPS + r] = fm_silu_mul(gv, uv);
        gcur = gnext;
        ucur = unext;
    }
}

// ---------------------------------------------------------------- kernel 3
// out[l][j] = sum_k w[l][k] * expert_out[l][k][j], k in slot order
// (finchmoe/shaders.metal:2213-2228).  GUARD adds the CPU path's finite check
// and renormalisation (finchmoe/infer.m:10190-10204); it needs the whole
// vector of each expert, so one workgroup covers a layer.
template <bool GUARD>
__device__ __forceinline__ void fm_combine_rows(const DecodeArgs &a, int l, int j0, int j1,
                                                float *red) {
    const int H = a.g.hidden, K = a.K;
    const float *eo = a.expert_out + (size_t)l * K * H;
    float wk[FM_MAX_K];
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < FM_MAX_K; k++) {
        float w = 0.0f;
        if (k < K) {
            w = a.w[l * K + k];
            if ((unsigned)a.idx[l * K + k] >= (unsigned)a.g.n_experts) w = 0.0f;
            if constexpr (GUARD) {
                float part = 0.0f;
                for (int j = threadIdx.x; j < H; j += blockDim.x) {
                    float v = fm_ld_shared(eo + (size_t)k * H + j);
                    part = fmaf(v, v, part);
                }
                part = fm_group_sum<64>(part);
                __syncthreads();
                if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
                __syncthreads();
                float er = 0.0f;
                for (int i = 0; i < (int)(blockDim.x >> 6); i++) er += red[i];
                bool keep = isfinite(er) && er < 1e20f;
                if (keep) total += w; else w = 0.0f;
            }
        }
        wk[k] = w;
    }
    float rn = 1.0f;
    if constexpr (GUARD) {
        if (total > 0.0f && total < 0.99f) rn = 1.0f / total;
    }
    float *out = a.out + (size_t)l * H;
    for (int j = j0 + threadIdx.x; j < j1; j += blockDim.x) {
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            if (k < K && wk[k] != 0.0f) acc += wk[k] * fm_ld_shared(eo + (size_t)k * H + j);
        if constexpr (GUARD) acc *= rn;
        out[j] = (a.flags & FM_ACCUMULATE) ? out[j] + acc : acc;
    }
}

// grid: GUARD (n_groups), otherwise (n_groups, ceil(hidden / 256))
template <bool GUARD>
__global__ __launch_bounds__(256) void fm_combine(DecodeArgs a) {
    __shared__ float red[FM_NW];
    const int H = a.g.hidden;
    const int j0 = GUARD ? 0 : blockIdx.y * blockDim.x;
    const int j1 = GUARD ? H : min(H, j0 + (int)blockDim.x);
    fm_combine_rows<GUARD>(a, blockIdx.x, j0, j1, red);
}

// ======================================================================
// Matrix-core path (fm_mfma.h): persistent workgroups over a static partition,
// weight ring in LDS.
//
// All row steps of all pairs form one sequence of "units" (a unit = one wave
// step = 64/LPR rows of one pair).  The launch has a fixed number of
// workgroups; workgroup g takes the contiguous unit range [U*g/G, U*(g+1)/G)
// and its four waves interleave over it — so a wave streams tens of kilobytes
// back to back instead of a few rows, and every wave ends after its own share
// (no queue).  A range is cut into segments that share an input vector (a
// layer for gate/up, a pair for down); per segment the workgroup builds the
// activation registers once in LDS (fm_build_act_lds) and every wave copies
// its own.
//
// Weight ring.  The rows of one wave step are consecutive rows of one matrix,
// so a slice is three contiguous byte runs: 64 lanes' worth of codes (3072 or
// 4096 B), 256 B of scales and 256 B of biases.  The wave copies them with
// LDS-direct loads (global_load_lds: 64 lanes x 16 B or 4 B land back to back
// at the address in M0).  They need no destination registers, so several
// slices per wave are in flight while the multiply keeps the registers, and
// every load instruction covers whole cache lines.  Each lane then reads its
// own 48/64 bytes and its scale/bias words back from the slot.
//
// Ordering.  LDS-direct loads complete in issue order and count in vmcnt.  A
// slice is consumed when RING-1 younger slices have been issued, so waiting
// until at most LOADS*(RING-1) vector-memory operations are outstanding
// guarantees that it has landed (stores only make the wait stricter); once the
// loader has run out of work the wait is for zero.  The compiler does not see
// the dependence between a load into LDS and the consumer's LDS read, so both
// the wait and the read are explicit.
// ======================================================================
// (the one-layer launch that takes the layer tail along keeps eight waves: it is bound by its
// chain of round trips, not by the stream, and with the tail's registers held across the
// experts it does not fit the 168 registers that twelve waves leave a lane)
constexpr int FM_NW_TAIL = 8;
template <int BITS, int NW = FM_NW>
struct FmDma : FmSlot<BITS> {
    // the workgroup's rings must fit in 160 KB of LDS next to the activation image
    static constexpr int RING = 2;
    static constexpr int WG_BYTES = NW * RING * FmSlot<BITS>::BYTES;
};

// Dynamic LDS of the streaming kernels: ring [FM_NW][RING] slots, then the
// activation image, then (gate/up only) the layer's blob table and valid mask.
extern __shared__ __attribute__((aligned(16))) uint8_t fm_dyn_lds[];

// Dependencies of a phase on other workgroups (used by the fused kernel; the
// separate kernels have none):
//   wait_in(s)            before segment s's input vector is read
//   publish(s, first, n)  by wave 0, once units [first, first+n) of segment s are
//                         complete and their stores have completed
struct FmNoDeps {
    __device__ __forceinline__ void wait_in(int) const {}
    __device__ __forceinline__ void publish(int, uint32_t, uint32_t) const {}
};

// What the loaders need to know about a segment (a layer's K experts for gate/up,
// one pair for down) plus the segment's unit counter.  Three of them, used round
// robin: while segment s is multiplied the loaders read those of s and s+1, and
// the one of s+1 is written while slower waves may still be loading s-1.
struct FmSegTable {
    const uint8_t *blob[FM_MAX_K];
    uint32_t valid;          // bit k: slot k has a valid expert index
    uint32_t next_unit;
    uint32_t pad[2];
};

template <int BITS, int LPR>
constexpr size_t fm_phase_lds_bytes() {
    return FmDma<BITS>::WG_BYTES + 2 * sizeof(FmActLds<LPR>) + 3 * sizeof(FmSegTable);
}

// The operator's two streaming phases over this workgroup's shares
// [U*g/G, U*(g+1)/G) of each phase's units:
//   gate/up: unit = RPS rows of gate and of up (two slices), segment = layer,
//            input a.x, output a.act (SwiGLU applied)
//   down   : unit = RPS rows (one slice), segment = pair, input a.act, output
//            a.expert_out
// DO_UP / DO_DOWN select the phases (one of them: the separate kernels).  An
// invalid expert index streams expert 0 and contributes zero.
//
// The shares form one continuous stream of segments, numbered in sequence
// across both phases.  Per segment only the activation image changes, and what
// a change needs is fetched ahead (the next segment's activations into
// registers, its expert indices two segments ahead), while the loaders run on
// into the next segment's units — also from the last gate/up segment into the
// first down segment, whose weights depend on nothing — as soon as the current
// one is handed out.  A slice's tag says which segment it belongs to, and a
// wave that meets a slice of the next segment waits for the workgroup to
// switch image.
// (A struct with inlined member functions rather than nested lambdas: the
// compiler keeps lambda closures that capture one another in private memory,
// and every access to it counts against the vector-memory counter the ring's
// waits rely on.)
template <int BITS, int LPR_UP, int LPR_DOWN, bool FP16, bool DO_UP, bool DO_DOWN, class DepsUp,
          class DepsDown>
struct FmOperatorStream {
    using D = FmDma<BITS>;
    static constexpr int RING = D::RING;
    static constexpr int LPR_MAX = LPR_UP > LPR_DOWN ? LPR_UP : LPR_DOWN;
    static constexpr int RPS_UP = FM_WAVE / LPR_UP, RPS_DN = FM_WAVE / LPR_DOWN;
    struct Raw {            // expert index and layer blob of one slot of a segment
        int e;
        const uint8_t *layer;
    };

    const DecodeArgs &a;
    const DepsUp &deps_up;
    const DepsDown &deps_down;
    int lane, wave;
    uint32_t ring0;
    uint8_t *img_mem;       // two images
    FmSegTable *tab;        // three tables
    // geometry of the two phases: units per pair / per segment, this workgroup's
    // units and segments, bytes per unit in the code and in the scale/bias regions
    uint32_t gu_upp, dn_upp;
    Fm1Split sp;            // this workgroup's shares of both phases (fm_index.h)
    long gu_segu, dn_segu;
    int n_up, n_seq;
    uint32_t gu_wstep, gu_sstep, dn_wstep, dn_sstep;
    // Loader's current phase: bytes per unit, region offsets of a unit's first
    // slice, and how far the second slice (up after gate) lies behind it.  Kept
    // as plain members that are assigned at the phase change: a `c ? m1 : m2` on
    // two members turns into one load from a selected address, which pins the
    // whole object in private memory.
    bool l_gu;
    uint32_t cur_wstep, cur_sstep, cur_w, cur_s, cur_b, d_w, d_s, d_b;
    // loader / multiply state
    int lq, cq;             // segment of the loader / of the multiply
    uint32_t l_first, l_n;
    int hn, wpos, c;
    uint32_t tag_n, rsn, issued, consumed;
    const uint8_t *blob_n;
    bool dry;               // nothing more to hand out for now
    bool once;              // every expert byte is read once in this launch (fm_ring.h, FM_AUX_ONCE)
    Raw raw_next;           // of segment cq + 2
    FmBuildSlot<BITS> bslot;

    __device__ __forceinline__ FmOperatorStream(const DecodeArgs &a_, int n_pairs,
                                                const DepsUp &du, const DepsDown &dd)
        : a(a_), deps_up(du), deps_down(dd) {
        lane = threadIdx.x & 63;
        wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        ring0 = (uint32_t)(uintptr_t)(fm_lptr)fm_dyn_lds + (uint32_t)wave * (RING * D::BYTES);
        img_mem = fm_dyn_lds + D::WG_BYTES;
        tab = reinterpret_cast<FmSegTable *>(fm_dyn_lds + D::WG_BYTES +
                                             2 * sizeof(FmActLds<LPR_MAX>));
        gu_upp = (uint32_t)(a.g.inter / RPS_UP);
        dn_upp = (uint32_t)(a.g.hidden / RPS_DN);
        gu_segu = (long)gu_upp * a.K;
        dn_segu = (long)dn_upp;
        const long gu_total = DO_UP ? (long)n_pairs * gu_upp : 0;
        const long dn_total = DO_DOWN ? (long)n_pairs * dn_upp : 0;
        sp = fm1_split(gu_total, dn_total, gu_segu, dn_segu, blockIdx.x, gridDim.x);
        n_up = sp.n_up;
        n_seq = sp.n_up + sp.n_dn;
        gu_wstep = (uint32_t)(RPS_UP * (a.g.hidden * BITS / 8));
        gu_sstep = (uint32_t)(RPS_UP * (a.g.hidden / 64) * 2);
        dn_wstep = (uint32_t)(RPS_DN * (a.g.inter * BITS / 8));
        dn_sstep = (uint32_t)(RPS_DN * (a.g.inter / 64) * 2);
        d_w = a.g.up_w - a.g.gate_w;
        d_s = a.g.up_s - a.g.gate_s;
        d_b = a.g.up_b - a.g.gate_b;
        if (DO_UP && n_up > 0) {
            l_gu = true;
            cur_wstep = gu_wstep, cur_sstep = gu_sstep;
            cur_w = a.g.gate_w, cur_s = a.g.gate_s, cur_b = a.g.gate_b;
        } else {
            loader_to_down();
        }
        lq = cq = 0;
        l_first = l_n = 0;
        hn = wpos = c = 0;
        tag_n = rsn = issued = consumed = 0;
        blob_n = nullptr;
        dry = false;
        // layers of a step have stores of their own; the positions of a chunk share one layer's experts
        once = a.layer_stride != 0 || n_pairs == a.K;
        raw_next = Raw{0, nullptr};
        bslot.init();
    }

    __device__ __forceinline__ void loader_to_down() {
        l_gu = false;
        cur_wstep = dn_wstep, cur_sstep = dn_sstep;
        cur_w = a.g.down_w, cur_s = a.g.down_s, cur_b = a.g.down_b;
    }
    // segment number q of the sequence -> phase and segment of that phase
    __device__ __forceinline__ bool seq_gu(int q) const { return q < n_up; }
    __device__ __forceinline__ int seq_seg(int q) const { return fm1_seg(sp, q); }
    // this workgroup's part of it: first unit (inside the segment) and count
    template <bool GU>
    __device__ __forceinline__ void seq_part(int q, uint32_t &first, uint32_t &n) const {
        fm1_part(sp, q, GU, &first, &n);
    }
    // the loader enters segment q
    __device__ __forceinline__ void loader_enter(int q) {
        if (l_gu && q >= n_up) loader_to_down();
        if (l_gu) seq_part<true>(q, l_first, l_n);
        else seq_part<false>(q, l_first, l_n);
    }
    // wave 0, lanes < K (gate/up) or lane 0 (down)
    __device__ __forceinline__ Raw load_raw(int q) const {
        Raw r{0, nullptr};
        const bool gu = seq_gu(q);
        const int s = seq_seg(q);
        if (wave == 0 && lane < (gu ? a.K : 1)) {
            const int l = gu ? s : s / a.K;
            r.e = a.idx[gu ? s * a.K + lane : s];
            r.layer = a.layer_ptrs[a.layer0 + l * a.layer_stride];
        }
        return r;
    }
    __device__ __forceinline__ void write_table(int q, const Raw &r) const {
        if (wave == 0) {
            FmSegTable &t = tab[q % 3];
            const int nk = seq_gu(q) ? a.K : 1;
            const bool ok = lane < nk && (unsigned)r.e < (unsigned)a.g.n_experts;
            if (lane < nk) t.blob[lane] = r.layer + (size_t)(ok ? r.e : 0) * a.g.expert_size;
            const uint64_t m = __ballot(ok);
            if (lane == 0) {
                t.valid = (uint32_t)m;
                t.next_unit = 0u;
            }
        }
    }
    template <bool GU>
    __device__ __forceinline__ void publish(int q) const {   // by wave 0, after a barrier
        if (wave == 0) {
            uint32_t pf, pc;
            seq_part<GU>(q, pf, pc);
            if constexpr (GU) deps_up.publish(seq_seg(q), pf, pc);
            else deps_down.publish(seq_seg(q), pf, pc);
        }
    }

    // loader: the next slice of the stream (gate rows, then up rows of the same unit)
    __device__ __forceinline__ void issue() {
        if (dry) return;
        if (!l_gu || hn == 0) {
            uint32_t ul;
            for (;;) {
                ul = fm_claim_unit(&tab[lq % 3].next_unit, lane);
                if (ul < l_n) break;
                if (lq + 1 < n_seq && lq == cq) {       // run on into the next segment
                    lq++;
                    loader_enter(lq);
                    continue;
                }
                dry = true;
                return;
            }
            const uint32_t uq = l_first + ul;                     // unit inside the segment
            const uint32_t pn = l_gu ? uq / gu_upp : 0u;
            rsn = uq - pn * gu_upp;
            tag_n = ((uint32_t)(lq & 1) << 31) | (pn << 28) | ul;
            blob_n = fm_uniform(tab[lq % 3].blob[pn]);
        }
        const uint32_t slot = ring0 + (uint32_t)wpos * D::BYTES;
        fm_slot_tag(slot + D::TAG, tag_n);
        const uint8_t *b = blob_n + (size_t)rsn * cur_wstep;
        const uint8_t *sb = blob_n + (size_t)rsn * cur_sstep;
        const uint32_t second = (uint32_t)hn;                     // 1: the up rows of a unit
        fm_dma_issue_as<BITS>(once, slot, b + cur_w + second * d_w, sb + cur_s + second * d_s,
                           sb + cur_b + second * d_b, lane);
        if (l_gu) hn ^= 1;
        wpos = wpos + 1 == RING ? 0 : wpos + 1;
        issued++;
    }

    // the oldest slice of the ring times the activation registers
    template <int LPR>
    __device__ __forceinline__ float take(uint32_t woff, uint32_t soff, const FmActRegs &ar) {
        FmRowSlice<BITS> t;
        if (issued - consumed == (uint32_t)RING) fm_dma_wait<D::LOADS *(RING - 1)>(false);
        else fm_dma_wait<0>(true);
        fm_dma_read<BITS>(ring0 + (uint32_t)c * D::BYTES, woff, soff, t);
        consumed++;
        c = c + 1 == RING ? 0 : c + 1;
        issue();
        return fm_chunk_sum<LPR>(fm_lane_dot_mfma<BITS, FP16>(t, ar));
    }

    // tables of the first two segments, first loads
    __device__ __forceinline__ void start() {
        loader_enter(0);
        __syncthreads();                              // LDS is free
        const Raw r0 = load_raw(0);
        const Raw r1 = load_raw(n_seq > 1 ? 1 : 0);
        write_table(0, r0);
        if (n_seq > 1) write_table(1, r1);
        raw_next = load_raw(n_seq > 2 ? 2 : 0);
        __syncthreads();
#pragma unroll
        for (int k = 0; k < RING; k++) issue();
    }

    // the segments [cq, q1) of one phase.  xr: the first segment's input vector
    // (gate/up), or nothing yet (down)
    template <int LPR, bool GU, class Deps>
    __device__ __forceinline__ void run_phase(FmActX<LPR> &xr, const Deps &deps, int q1) {
        constexpr int RPS = FM_WAVE / LPR;
        const int q0 = cq;
        const long segu_c = GU ? gu_segu : dn_segu;
        const int in_dim = GU ? a.g.hidden : a.g.inter;
        uint32_t woff, soff;
        int ris, ch;
        fm_unit_lane_offsets<BITS, LPR>(lane, in_dim * BITS / 8, (in_dim / 64) * 2, woff, soff, ris,
                                        ch);
        const float *in_base = GU ? a.x : a.act;
        float *out_vec = GU ? a.act : a.expert_out;
        for (; cq < q1; cq++) {
            const int s = seq_seg(cq);
            FmActLds<LPR> &img = *reinterpret_cast<FmActLds<LPR> *>(
                img_mem + (cq & 1) * sizeof(FmActLds<LPR_MAX>));
            // ---- switch to the image of this segment
            const bool first_down = !GU && cq == q0;
            if (first_down) {
                // the first down vector may be this workgroup's own: it is not fetched
                // ahead, and what the workgroup has produced is published before the wait
                __syncthreads();
                if (cq > 0) publish<true>(cq - 1);
                if (threadIdx.x < 256) {
                    deps.wait_in(s);
                    fm_act_load<BITS, LPR, true>(in_base + (size_t)s * in_dim, bslot, xr);
                }
            }
            if (threadIdx.x < 256) fm_act_build<BITS, LPR>(xr, bslot, img);
            const bool new_table = cq > 0 && cq + 1 < n_seq;
            // every loader has left segment cq-2: its table becomes that of cq+1
            if (new_table) write_table(cq + 1, raw_next);
            __syncthreads();
            if (!first_down && cq > 0) publish<GU>(cq - 1);   // every wave is done with it
            FmActRegs ar;
            fm_read_act_lds<LPR>(img, lane, ar);
            const uint32_t valid = __builtin_amdgcn_readfirstlane(tab[cq % 3].valid);
            uint32_t c_first, c_n;
            seq_part<GU>(cq, c_first, c_n);
            const size_t out0 = (size_t)((long)s * segu_c + c_first) * RPS + ris;
            // fetched now, used at the next switch
            if (cq + 1 < q1 && threadIdx.x < 256) {
                deps.wait_in(s + 1);
                fm_act_load<BITS, LPR, !GU>(in_base + (size_t)(s + 1) * in_dim, bslot, xr);
            }
            if (new_table) raw_next = load_raw(cq + 2 < n_seq ? cq + 2 : cq);
            dry = false;
            while (issued - consumed < (uint32_t)RING && !dry) issue();

            // ---- multiply the slices of this segment
            while (consumed < issued) {
                const uint32_t tag = fm_slot_peek(ring0 + (uint32_t)c * D::BYTES + D::TAG);
                if ((tag >> 31) != (uint32_t)(cq & 1)) break;     // belongs to the next segment
                const uint32_t pc = (tag >> 28) & 7u, ul = tag & 0x0FFFFFFFu;
                float v;
                if constexpr (GU) {
                    const float gv = take<LPR>(woff, soff, ar);
                    const float uv = take<LPR>(woff, soff, ar);
                    v = fm_silu_mul(gv, uv);
                } else {
                    v = take<LPR>(woff, soff, ar);
                }
                if (!((valid >> pc) & 1u)) v = 0.0f;
                // unit (pair, row step): the output is [pair][rows], rows are contiguous
                if (ch == 0) fm_st_shared(out_vec + out0 + (size_t)ul * RPS, v);
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's stores have completed
        }
    }

    __device__ __forceinline__ void run() {
        if (n_seq == 0) return;
        FmActX<LPR_UP> xr_up;
        if (n_up > 0 && threadIdx.x < 256)
            fm_act_load<BITS, LPR_UP, false>(a.x + (size_t)seq_seg(0) * a.g.hidden, bslot, xr_up);
        start();
        if constexpr (DO_UP) run_phase<LPR_UP, true>(xr_up, deps_up, n_up);
        if constexpr (DO_DOWN) {
            FmActX<LPR_DOWN> xr_dn;
            run_phase<LPR_DOWN, false>(xr_dn, deps_down, n_seq);
        }
        __syncthreads();
        publish<!DO_DOWN>(n_seq - 1);
    }
};

template <int BITS, int LPR_UP, int LPR_DOWN, bool FP16, bool DO_UP, bool DO_DOWN, class DepsUp,
          class DepsDown>
__device__ __forceinline__ void fm_stream_operator(const DecodeArgs &a, int n_pairs,
                                                   const DepsUp &deps_up,
                                                   const DepsDown &deps_down) {
    FmOperatorStream<BITS, LPR_UP, LPR_DOWN, FP16, DO_UP, DO_DOWN, DepsUp, DepsDown> st(
        a, n_pairs, deps_up, deps_down);
    st.run();
}

template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(FM_NW * 64) void fm_gate_up_swiglu_lds(DecodeArgs a, int n_pairs) {
    fm_stream_operator<BITS, LPR, LPR, FP16, true, false>(a, n_pairs, FmNoDeps(), FmNoDeps());
}

template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(FM_NW * 64) void fm_down_lds(DecodeArgs a, int n_pairs) {
    fm_stream_operator<BITS, LPR, LPR, FP16, false, true>(a, n_pairs, FmNoDeps(), FmNoDeps());
}

// ======================================================================
// One launch for the whole operator: gate/up, down and combine as three phases
// of one persistent grid.
//
// A phase's weights do not depend on the previous phase, so every wave issues
// the first slices of its next share before it looks at its input: the memory
// pipeline stays full across the phase change, where separate kernels drain
// it, relaunch and refill it.
//
// Dependencies are per vector, not grid-wide: a counter per pair says how many
// units of its activation vector exist, a counter per group how many units of
// its K expert outputs.  Both phases split their units over the workgroups in
// proportion, so a workgroup's down share needs activations that it or its
// neighbours produced a moment ago, and nobody waits for the slowest workgroup
// of the grid.  Producers add to a counter after their stores have completed;
// the vectors themselves are stored and loaded at device scope (fm_st_shared /
// fm_ld_shared), so no cache is written back or invalidated.
//
// Two sets of counters alternate between launches: a launch uses one and
// clears the part of the other that the launch before it used, so nothing has
// to be reset in between and a failed launch leaves no state behind.  Every
// workgroup must be resident at once (the launcher sizes the grid from the
// occupancy query), a workgroup finishes a phase before it starts the next, and
// every wait is bounded: past `spin_limit` polls the thread raises `*err` and
// goes on (the results are then wrong and the host reports the error).
// ======================================================================
struct FmFlags {
    unsigned int *cur;        // [n_pairs] activation units, then [n_groups] expert-output units
    unsigned int *other;      // the set of the previous and of the next launch
    unsigned int clear_n;     // entries of `other` to clear
    unsigned int *err;        // host memory
    unsigned int spin_limit;
};

__device__ __forceinline__ void fm_flag_wait(const FmFlags &f, const unsigned int *flag,
                                             unsigned int target) {
    unsigned int polls = 0;
    while (__hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
        if (++polls > f.spin_limit) {
            __hip_atomic_store(f.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            break;
        }
        __builtin_amdgcn_s_sleep(8);
    }
    // The vector this wait guards is read with relaxed device-scope loads, which carry no
    // ordering of their own: without this the compiler may legally hoist them above the poll
    // loop.  The hardware half: the producer's device-scope (sc1) stores write through to the
    // memory side of the fabric, `s_waitcnt vmcnt(0)` returns only once they have been
    // acknowledged from there, and only then is the counter incremented (an atomic performed
    // at the same place) — so a device-scope load issued after the counter was seen reads the
    // stored value whichever XCD's L2 sits in front of the reader, with no cache maintenance.
    __atomic_signal_fence(__ATOMIC_ACQUIRE);
}

// gate/up: publishes per pair how many of its units this workgroup finished
struct FmGateUpDeps {
    const FmFlags &f;
    int K;
    uint32_t upp;
    __device__ __forceinline__ void wait_in(int) const {}
    __device__ __forceinline__ void publish(int s, uint32_t first, uint32_t n) const {
        const int k = threadIdx.x & 63;
        if (k < K) {
            const uint32_t lo = max(first, (uint32_t)k * upp), hi = min(first + n, (uint32_t)(k + 1) * upp);
            if (hi > lo)
                __hip_atomic_fetch_add(f.cur + (size_t)s * K + k, hi - lo, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        }
    }
};

// down: waits for a pair's activation vector, publishes per group
struct FmDownDeps {
    const FmFlags &f;
    int K, n_pairs;
    uint32_t upp_up;          // units of a complete activation vector
    __device__ __forceinline__ void wait_in(int p) const { fm_flag_wait(f, f.cur + p, upp_up); }
    __device__ __forceinline__ void publish(int p, uint32_t, uint32_t n) const {
        if ((threadIdx.x & 63) == 0)
            __hip_atomic_fetch_add(f.cur + n_pairs + p / K, n, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
    }
};

template <int BITS, int LPR_UP, bool FP16>
__global__ __launch_bounds__(FM_NW * 64)
void fm_moe_fused(DecodeArgs a, int n_pairs, FmFlags f) {
    constexpr int LPR_DOWN = LPR_UP / 4;
    __shared__ float red[FM_NW];
    const int G = gridDim.x, n_groups = n_pairs / a.K, H = a.g.hidden;
    for (unsigned int i = blockIdx.x * blockDim.x + threadIdx.x; i < f.clear_n;
         i += G * blockDim.x)
        f.other[i] = 0u;
    const uint32_t upp_up = (uint32_t)(a.g.inter / (FM_WAVE / LPR_UP));
    const uint32_t upp_down = (uint32_t)(H / (FM_WAVE / LPR_DOWN));
    fm_stream_operator<BITS, LPR_UP, LPR_DOWN, FP16, true, true>(
        a, n_pairs, FmGateUpDeps{f, a.K, upp_up}, FmDownDeps{f, a.K, n_pairs, upp_up});
    // combine: a group's K expert outputs are complete at K * upp_down units
    const unsigned int full = (unsigned int)a.K * upp_down;
    if (a.flags & FM_GUARD) {
        for (int l = blockIdx.x; l < n_groups; l += G) {
            fm_flag_wait(f, f.cur + n_pairs + l, full);
            fm_combine_rows<true>(a, l, 0, H, red);
        }
    } else {
        // column blocks of a group go to neighbouring workgroups, groups in the
        // order in which the down phase finishes them
        const int cols = FM_NW * 64, per = (H + cols - 1) / cols, items = n_groups * per;
        for (int it = (int)((long)blockIdx.x * items / G); it < (int)((long)(blockIdx.x + 1) * items / G); it++) {
            const int l = it / per, j0 = (it - l * per) * cols;
            fm_flag_wait(f, f.cur + n_pairs + l, full);
            fm_combine_rows<false>(a, l, j0, min(H, j0 + cols), red);
        }
    }
}

// ======================================================================
// The operator as one launch when the caller does not want the per-expert vectors and the
// plain combine applies (no finite guard): nothing but `out` leaves the workgroup.
//
// Down phase by row blocks.  A row block is one wave step's rows (64/LPR_DOWN of them) of all
// K experts of a layer; the row blocks are split over the workgroups, so
// a workgroup owns whole output rows: it keeps the K partial vectors of its rows in LDS and
// adds them up itself, w_k * down_k in slot order (the arithmetic of fm_combine_rows<false>),
// when its part of a layer is finished.  The per-expert vectors are never written, there is
// no combine phase, and nothing waits for the slowest workgroup of the grid.  A segment of
// the down phase is a layer: the K activation images of its experts fill the LDS of the two
// gate/up images.  Units of a part are handed out expert by expert, so a wave re-reads its
// activation registers only when the expert changes.
//
// Activations between the phases.  A vector element that has not been produced yet holds
// FM_ACT_EMPTY (a NaN that no arithmetic yields); the consumer polls each element it needs
// until it holds something else.  No counters, so the producer never has to wait for its
// stores (a wait for stores is a wait for every load in flight as well: it would empty the
// ring).  Two activation sets alternate between launches: a launch fills the one it is given
// and marks the part of the other that the launch before it filled as empty again.
//
// The split (see Fm2Stream::run): a workgroup's down rows lie in one layer, and its gate/up
// units are sized so that every workgroup streams the same number of bytes; a gate/up share
// touches at most two layers, whose images are both built before the stream starts, so the
// only workgroup barrier of the steady state is the one between the phases.  The slowest
// workgroup ends the kernel: a workgroup that changed layer more often than the others used
// to be that one.
//
// Nothing in the steady state waits for vector memory except the ring's own waits: all
// segment tables (blob pointers, router weights) are built before the first load of the ring,
// LDS is accessed with explicit instructions (the compiler would order a visible LDS access
// behind every LDS-direct load in flight), barriers likewise.
// ======================================================================
// (FM_ACT_EMPTY and Fm2Sync: fm_common.h)
// FM2_MAX_SEG segments of one workgroup's shares and FM2_PART_BYTES of partial vectors of a part:
// fm_index.h

struct Fm2Seg {
    const uint8_t *blob[FM_MAX_K];
    float w[FM_MAX_K];       // router weight, 0 for an invalid expert index
    uint32_t valid;          // bit k: slot k has a valid expert index
    uint32_t next_unit;
    uint32_t first, n;       // this workgroup's units of the segment
    int layer;               // layer group (layer of a step, position of a chunk)
    int pad;
};

template <int BITS, int LPR, int NW = FM_NW>
constexpr size_t fm2_lds_bytes() {
    return FmDma<BITS, NW>::WG_BYTES + 2 * sizeof(FmActLds<LPR>) + FM2_MAX_SEG * sizeof(Fm2Seg) +
           FM2_PART_BYTES;
}

// (fm_lds_w32 / fm_lds_r32 / fm_wg_barrier: fm_ring.h)

// fm_read_act_lds with explicit instructions; img = LDS address of the image
template <int LPR>
__device__ __forceinline__ void fm_read_act_lds_x(uint32_t img, int lane, FmActRegs &ar) {
    constexpr int NE = 4 * LPR, QS = NE * 16;
    const int e = lane % NE;
    const uint32_t a0 = img + (uint32_t)e * 16u;
    const uint32_t as = img + 16u * QS + (uint32_t)(e >> 2) * 16u;
    fm_u4 q[16], sm;
    asm volatile("ds_read_b128 %0, %17\n\t"
                 "ds_read_b128 %1, %17 offset:%c19\n\t"
                 "ds_read_b128 %2, %17 offset:%c19*2\n\t"
                 "ds_read_b128 %3, %17 offset:%c19*3\n\t"
                 "ds_read_b128 %4, %17 offset:%c19*4\n\t"
                 "ds_read_b128 %5, %17 offset:%c19*5\n\t"
                 "ds_read_b128 %6, %17 offset:%c19*6\n\t"
                 "ds_read_b128 %7, %17 offset:%c19*7\n\t"
                 "ds_read_b128 %8, %17 offset:%c19*8\n\t"
                 "ds_read_b128 %9, %17 offset:%c19*9\n\t"
                 "ds_read_b128 %10, %17 offset:%c19*10\n\t"
                 "ds_read_b128 %11, %17 offset:%c19*11\n\t"
                 "ds_read_b128 %12, %17 offset:%c19*12\n\t"
                 "ds_read_b128 %13, %17 offset:%c19*13\n\t"
                 "ds_read_b128 %14, %17 offset:%c19*14\n\t"
                 "ds_read_b128 %15, %17 offset:%c19*15\n\t"
                 "ds_read_b128 %16, %18\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&v"(q[0]), "=&v"(q[1]), "=&v"(q[2]), "=&v"(q[3]), "=&v"(q[4]), "=&v"(q[5]),
                   "=&v"(q[6]), "=&v"(q[7]), "=&v"(q[8]), "=&v"(q[9]), "=&v"(q[10]), "=&v"(q[11]),
                   "=&v"(q[12]), "=&v"(q[13]), "=&v"(q[14]), "=&v"(q[15]), "=&v"(sm)
                 : "v"(a0), "v"(as), "n"(QS)
                 : "memory");
#pragma unroll
    for (int i = 0; i < 16; i++) {
        ar.a[4 * i + 0] = q[i][0];
        ar.a[4 * i + 1] = q[i][1];
        ar.a[4 * i + 2] = q[i][2];
        ar.a[4 * i + 3] = q[i][3];
    }
    ar.xsum[0] = __uint_as_float(sm[0]);
    ar.xsum[1] = __uint_as_float(sm[1]);
    ar.xoff[0] = __uint_as_float(sm[2]);
    ar.xoff[1] = __uint_as_float(sm[3]);
    ar.ones = fm_opaque(0x3F803F80u);
}

// fm_act_build for one (chunk, image) with explicit LDS writes: this wave's 64 lanes hold
// the 64 register slots of chunk `ch` (xl, xh: the slot's two activations), img = LDS address
template <int BITS, int LPR>
__device__ __forceinline__ void fm2_build_chunk(float xl, float xh, const FmBuildSlot<BITS> &bs,
                                                uint32_t img, int ch, bool on) {
    constexpr int NE = 4 * LPR;
    const int w = threadIdx.x & 63;
    float vl = xl * bs.slo, vh = xh * bs.shi;
    uint32_t l0 = __float_as_uint(vl) & 0xFFFF0000u, h0 = __float_as_uint(vh) & 0xFFFF0000u;
    float rl = vl - __uint_as_float(l0), rh = vh - __uint_as_float(h0);
    uint32_t l1 = __float_as_uint(rl) & 0xFFFF0000u, h1 = __float_as_uint(rh) & 0xFFFF0000u;
    rl -= __uint_as_float(l1);
    rh -= __uint_as_float(h1);
    uint32_t l2 = __float_as_uint(rl), h2 = __float_as_uint(rh) & 0xFFFF0000u;
    float xs = fm_group_sum<32>(xl + xh);
    float xo = fm_group_sum<32>(vl + vh);
    if (on) {
        const uint32_t dst = img + (uint32_t)((((w >> 2) * NE + 4 * ch) * 4 + (w & 3)) * 4);
        fm_lds_w32(dst, (l0 >> 16) | h0);
        fm_lds_w32(dst + 16, (l1 >> 16) | h1);
        fm_lds_w32(dst + 32, (l2 >> 16) | h2);
        fm_lds_w32(dst + 48, 0u);
        if ((w & 31) == 0) {
            const uint32_t sp = img + (uint32_t)(16 * NE * 16 + ch * 16 + (w >> 5) * 4);
            fm_lds_w32(sp, __float_as_uint(xs));
            fm_lds_w32(sp + 8, __float_as_uint(xo));
        }
    }
}


template <int BITS, int LPR_UP, bool FP16, int NW = FM_NW>
struct Fm2Stream {
    using D = FmDma<BITS, NW>;
    static constexpr int RING = D::RING;
    static constexpr int LPR_DN = LPR_UP / 4;
    static constexpr int RPS_UP = FM_WAVE / LPR_UP, RPS_DN = FM_WAVE / LPR_DN;
    static constexpr int IMG_UP = (int)sizeof(FmActLds<LPR_UP>), IMG_DN = (int)sizeof(FmActLds<LPR_DN>);
    static_assert(FM_MAX_K * IMG_DN <= 2 * IMG_UP, "the K down images use the two gate/up images");

    const DecodeArgs &a;
    const Fm2Sync &sy;
    int lane, wave;
    uint32_t ring0, img0, part0;
    Fm2Seg *tab;
    uint32_t gu_upp, dn_upp;
    FmDiv by_gu_upp, by_K;
    int n_up, n_seq;
    uint32_t gu_wstep, gu_sstep, dn_wstep, dn_sstep;
    // loader's phase (plain members assigned at the phase change, see FmOperatorStream)
    bool l_gu;
    uint32_t cur_wstep, cur_sstep, cur_w, cur_s, cur_b, d_w, d_s, d_b;
    int lq, cq;
    uint32_t l_first, l_n, l_nrb;
    float l_inv;
    int hn, wpos, c;
    uint32_t tag_n, rsn, issued, consumed;
    const uint8_t *blob_n;
    bool dry;
    bool once;              // every expert byte is read once in this launch (fm_ring.h, FM_AUX_ONCE)
    FmBuildSlot<BITS> bslot;

    __device__ __forceinline__ Fm2Stream(const DecodeArgs &a_, const Fm2Sync &sy_) : a(a_), sy(sy_) {
        lane = threadIdx.x & 63;
        wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const uint32_t lds0 = fm_lds_addr(fm_dyn_lds);
        ring0 = lds0 + (uint32_t)wave * (RING * D::BYTES);
        img0 = lds0 + D::WG_BYTES;
        tab = reinterpret_cast<Fm2Seg *>(fm_dyn_lds + D::WG_BYTES + 2 * IMG_UP);
        part0 = img0 + 2 * IMG_UP + FM2_MAX_SEG * (uint32_t)sizeof(Fm2Seg);
        gu_upp = (uint32_t)(a.g.inter / RPS_UP);
        dn_upp = (uint32_t)(a.g.hidden / RPS_DN);
        gu_wstep = (uint32_t)(RPS_UP * (a.g.hidden * BITS / 8));
        gu_sstep = (uint32_t)(RPS_UP * (a.g.hidden / 64) * 2);
        dn_wstep = (uint32_t)(RPS_DN * (a.g.inter * BITS / 8));
        dn_sstep = (uint32_t)(RPS_DN * (a.g.inter / 64) * 2);
        d_w = a.g.up_w - a.g.gate_w;
        d_s = a.g.up_s - a.g.gate_s;
        d_b = a.g.up_b - a.g.gate_b;
        lq = cq = 0;
        l_first = l_n = l_nrb = 0;
        l_inv = 0.0f;
        hn = wpos = c = 0;
        tag_n = rsn = issued = consumed = 0;
        blob_n = nullptr;
        dry = false;
        once = a.layer_stride != 0;      // (one group: run() says so, it knows the number of groups)
        l_gu = true;
        bslot.init();
    }

    __device__ __forceinline__ void loader_enter(int q) {
        if (l_gu && q >= n_up) {
            l_gu = false;
            cur_wstep = dn_wstep, cur_sstep = dn_sstep;
            cur_w = a.g.down_w, cur_s = a.g.down_s, cur_b = a.g.down_b;
        }
        const uint32_t ta = fm_lds_addr(&tab[q].first);
        l_first = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta));
        l_n = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + 4));
        if (!l_gu) {
            l_nrb = fm_div(by_K, l_n);
            l_first = fm_div(by_K, l_first);            // first row block of the part
            l_inv = 1.0f / (float)(l_nrb ? l_nrb : 1u);
        }
    }

    __device__ __forceinline__ void issue() {
        if (dry) return;
        if (!l_gu || hn == 0) {
            uint32_t ul;
            for (;;) {
                ul = fm_claim_unit(&tab[lq].next_unit, lane);
                if (ul < l_n) break;
                if (lq + 1 < n_seq && lq == cq) {       // run on into the next segment
                    lq++;
                    loader_enter(lq);
                    continue;
                }
                dry = true;
                return;
            }
            uint32_t pn;
            if (l_gu) fm2_gu_unit(l_first, ul, by_gu_upp, &pn, &rsn);
            else fm2_dn_unit(l_first, l_nrb, l_inv, ul, &pn, &rsn);     // expert by expert
            tag_n = ((uint32_t)(lq & 1) << 31) | (pn << 28) | ul;
            const uint32_t ba = fm_lds_addr(&tab[lq].blob[pn]);
            const uint32_t lo = __builtin_amdgcn_readfirstlane(fm_lds_r32(ba));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(fm_lds_r32(ba + 4));
            blob_n = (const uint8_t *)(((uintptr_t)hi << 32) | lo);
        }
        const uint32_t slot = ring0 + (uint32_t)wpos * D::BYTES;
        fm_slot_tag(slot + D::TAG, tag_n);
        const uint8_t *b = blob_n + (size_t)rsn * cur_wstep;
        const uint8_t *sb = blob_n + (size_t)rsn * cur_sstep;
        const uint32_t second = (uint32_t)hn;
        fm_dma_issue_as<BITS>(once, slot, b + cur_w + second * d_w, sb + cur_s + second * d_s,
                           sb + cur_b + second * d_b, lane);
        if (l_gu) hn ^= 1;
        wpos = wpos + 1 == RING ? 0 : wpos + 1;
        issued++;
    }

    template <int LPR>
    __device__ __forceinline__ float take(uint32_t woff, uint32_t soff, const FmActRegs &ar) {
        FmRowSlice<BITS> t;
        if (issued - consumed == (uint32_t)RING) fm_dma_wait<D::LOADS *(RING - 1)>(false);
        else fm_dma_wait<0>(true);
        fm_dma_read<BITS>(ring0 + (uint32_t)c * D::BYTES, woff, soff, t);
        consumed++;
        c = c + 1 == RING ? 0 : c + 1;
        issue();
        return fm_chunk_sum<LPR>(fm_lane_dot_mfma<BITS, FP16>(t, ar));
    }

    __device__ __forceinline__ int seg_layer(int q) const {
        return __builtin_amdgcn_readfirstlane((int)fm_lds_r32(fm_lds_addr(&tab[q].layer)));
    }

    // an activation produced in this launch: polled until it is there
    __device__ __forceinline__ float act_get(const float *p) const {
        unsigned int polls = 0;
        for (;;) {
            const float v = fm_ld_shared(p);
            if (__float_as_uint(v) != FM_ACT_EMPTY) return v;
            if (++polls > sy.spin_limit) {
                __hip_atomic_store(sy.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                return 0.0f;
            }
            __builtin_amdgcn_s_sleep(8);
        }
    }

    // w_k * partial_k over the part's rows, in slot order -> out (fm_combine_rows<false>)
    __device__ __forceinline__ void reduce_part(int q) {
        const int K = a.K;
        const uint32_t ta = fm_lds_addr(&tab[q]);
        const uint32_t first = fm_lds_r32(ta + (uint32_t)offsetof(Fm2Seg, first));
        const uint32_t n = fm_lds_r32(ta + (uint32_t)offsetof(Fm2Seg, n));
        float wk[FM_MAX_K];
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            wk[k] = k < K ? __uint_as_float(fm_lds_r32(ta + (uint32_t)offsetof(Fm2Seg, w) + 4u * k)) : 0.0f;
        const int rows = (int)fm_div(by_K, n) * RPS_DN;
        const int l = seg_layer(q);
        float *out = a.out + (size_t)l * a.g.hidden + (size_t)fm_div(by_K, first) * RPS_DN;
        for (int r = threadIdx.x; r < rows; r += NW * 64) {
            const int rbi = r / RPS_DN, ris = r - rbi * RPS_DN;
            float acc = 0.0f;
#pragma unroll
            for (int k = 0; k < FM_MAX_K; k++)
                if (k < K && wk[k] != 0.0f)
                    acc += wk[k] * __uint_as_float(fm_lds_r32(part0 + 4u * (uint32_t)((rbi * K + k) * RPS_DN + ris)));
            out[r] = (a.flags & FM_ACCUMULATE) ? out[r] + acc : acc;
        }
    }

    // dm: the launch's dimensions with their divisions prepared (fm2_dims on the host).
    // TAIL (one layer, one down part per workgroup): the layer's tail in the same launch — the
    // workgroup that owns rows of the experts' sum also runs those rows of the shared expert's
    // down projection and writes hidden = h_mid + sum + sigmoid(score) * shared; the workgroup
    // that finishes last normalises (fm_layer_tail's arithmetic, operation for operation).
    template <bool TAIL>
    __device__ __forceinline__ void run(const Fm2Dims &dm, const FmTailArgs *tp) {
        const int K = a.K, G = gridDim.x, g = blockIdx.x;
        // The split.  Down: a workgroup's row blocks lie in ONE layer whenever there are at
        // least as many workgroups as layers (layer l gets the workgroups g with g*L/G == l, its
        // row blocks divided evenly among them), so the down phase has one segment and no
        // workgroup pays for a change of layer that others do not have.  Gate/up: contiguous unit
        // ranges sized so that gate/up + down bytes are the same for every workgroup (a
        // workgroup with fewer down rows takes more gate/up units).
        // (32-bit arithmetic: the launcher checks that slices x workgroups stays below 2^31)
        by_gu_upp = dm.by_gu_upp, by_K = dm.by_K;
        if (dm.L == 1u) once = true;
        const Fm2Split sp = fm2_split(dm, (uint32_t)g);
        const uint32_t gu_segu = dm.gu_segu;
        const int gu_s0 = sp.gu_s0;
        n_up = sp.n_up;
        n_seq = sp.n_up + sp.n_dn;
        const int qq = threadIdx.x >> 3;        // the segment this thread looks up below
        const bool mine = qq < n_seq;
        const Fm2Part mp = fm2_part(dm, sp, mine ? qq : 0);
        const uint32_t mine_s = mp.seg, mine_first = mp.first, mine_n = mp.n;

        // the other activation set becomes empty again (plain stores, nobody reads it now)
        for (unsigned int i = blockIdx.x * blockDim.x + threadIdx.x; i < sy.clear_n; i += G * blockDim.x)
            sy.act_other[i] = __uint_as_float(FM_ACT_EMPTY);
        if (n_seq == 0) return;

        // the first gate/up segment's input, then the tables of every segment: thread 8q + k
        // looks up slot k of segment q (ordinary loads and LDS stores: nothing is in flight yet)
        // (every thread loads, and the values are used unconditionally further down: a load
        // whose result is still pending on some path of the control flow makes the compiler
        // wait for every load in flight at the register's next use, in the middle of the stream)
        FmActX<LPR_UP> xr0, xr1;
        fm_act_load<BITS, LPR_UP, false>(a.x + (size_t)(n_up > 0 ? gu_s0 : 0) * a.g.hidden, bslot, xr0);
        fm_act_load<BITS, LPR_UP, false>(a.x + (size_t)(n_up > 1 ? gu_s0 + 1 : 0) * a.g.hidden, bslot, xr1);
        // TAIL with the routing inside: wave 0 of every workgroup routes the token (the same wave
        // function as the routing kernel, on the same logits: the same indices and weights
        // everywhere), into LDS; workgroup 0 also leaves them in memory for the caller
        const int32_t *idx_src = a.idx;
        const float *w_src = a.w;
        if constexpr (TAIL) {
            if (tp->route_logits) {
                uint8_t *part_mem = fm_dyn_lds + D::WG_BYTES + 2 * IMG_UP + FM2_MAX_SEG * sizeof(Fm2Seg);
                int32_t *r_idx = reinterpret_cast<int32_t *>(part_mem + FM2_PART_BYTES - FM2_ROUTE_WORDS);
                float *r_w = reinterpret_cast<float *>(part_mem + FM2_PART_BYTES - FM2_ROUTE_WORDS + 32);
                float *r_par = reinterpret_cast<float *>(part_mem + FM2_PART_BYTES - FM2_ROUTE_WORDS + 64);
                if (wave == 0) {
                    const RouteArgs ra{tp->route_logits, tp->route_n, K, tp->route_seg, r_idx, r_w, r_par};
                    fm_route_wave<false>(ra, reinterpret_cast<float *>(part_mem));
                    if (blockIdx.x == 0) {
                        if (lane < K) {
                            tp->route_idx[lane] = r_idx[lane];
                            tp->route_w[lane] = r_w[lane];
                        }
                        if (tp->route_params && lane < 10) tp->route_params[lane] = r_par[lane];
                    }
                }
                __syncthreads();
                idx_src = r_idx;
                w_src = r_w;
            }
        }
        if (mine) {
            const int k = threadIdx.x & 7;
            const size_t sg = mine_s;                              // layer group of the segment
            Fm2Seg &t = tab[qq];
            bool ok = false;
            if (k < K) {
                const int e = idx_src[sg * K + k];
                const float wv = w_src[sg * K + k];
                ok = (unsigned)e < (unsigned)a.g.n_experts;
                t.blob[k] = a.layer_ptrs[a.layer0 + (int)sg * a.layer_stride] + (size_t)(ok ? e : 0) * a.g.expert_size;
                t.w[k] = ok ? wv : 0.0f;
            }
            const uint64_t m = __ballot(ok);
            if (k == 0) {
                t.valid = (uint32_t)(m >> (threadIdx.x & 56)) & 0xFFu;
                t.next_unit = 0u;
                t.first = mine_first;
                t.n = mine_n;
                t.layer = (int)sg;
            }
        }
        // TAIL: what the tail needs from memory is requested here too (the shared expert's codes
        // for this workgroup's rows stay in registers until the experts are done)
        FmRowSlice<4> tw;
        float t_hm = 0.0f, t_score = 0.0f;
        uint32_t t_nw = 0u;
        int t_row0 = 0, t_nrb = 0;
        Fm2TailLds tl{};
        if constexpr (TAIL) {
            t_nrb = (int)fm_div(dm.by_K, sp.dn_wg1 - sp.dn_wg0);
            t_row0 = (int)fm_div(dm.by_K, sp.dn_wg0) * RPS_DN;
            tl = fm2_tail_lds(t_nrb, K, RPS_DN, tp->inter, tp->hidden);
            const int tw_row = t_row0 + (wave < t_nrb ? wave : 0) * RPS_DN + lane / LPR_DN, tc = lane % LPR_DN;
            const int trb = tp->inter / 2, tsb = (tp->inter / 64) * 2;
            fm_load_slice<4>(tw, tp->W + (size_t)tw_row * trb + (size_t)tc * 64, tp->S + (size_t)tw_row * tsb + (size_t)tc * 4,
                             tp->B + (size_t)tw_row * tsb + (size_t)tc * 4);
            const int rows = t_nrb * RPS_DN, tr = (int)threadIdx.x < rows ? (int)threadIdx.x : (rows > 0 ? rows - 1 : 0);
            t_hm = tp->h_mid[t_row0 + tr];
            t_score = tp->route_logits ? (tp->route_seg ? *tp->route_seg : 0.0f) : tp->params[8];
            t_nw = tp->next_in ? (uint32_t)tp->norm_w[t_row0 + tr] : 0u;
            const int tj = (int)threadIdx.x < tp->inter ? (int)threadIdx.x : tp->inter - 1;
            const float tact = fm_silu_mul(tp->shared_gate[tj], tp->shared_up[tj]);
            if ((int)threadIdx.x < tp->inter) fm_lds_w32(part0 + tl.act + 4u * (uint32_t)tj, __float_as_uint(tact));
#pragma unroll
            for (int i = 0; i < FmRowSlice<4>::NQ; i++) asm volatile("" ::"v"(tw.q[i]));
            asm volatile("" ::"v"(tw.s), "v"(tw.b), "v"(t_hm), "v"(t_score), "v"(t_nw));
        }
#pragma unroll
        for (int i = 0; i < FmActX<LPR_UP>::NIT; i++)
            asm volatile("" ::"v"(xr0.xl[i]), "v"(xr0.xh[i]), "v"(xr1.xl[i]), "v"(xr1.xh[i]));
        if (n_up > 0) {
            cur_wstep = gu_wstep, cur_sstep = gu_sstep;
            cur_w = a.g.gate_w, cur_s = a.g.gate_s, cur_b = a.g.gate_b;
        }
        __syncthreads();
        loader_enter(0);
#pragma nounroll
        for (int k = 0; k < RING; k++) {
            issue();
        }
        // the images of both gate/up segments (from registers: no load is waited for here); a
        // wave then changes segment on its own, without a barrier
        if (n_up > 0 && threadIdx.x < 256) {
#pragma unroll
            for (int i = 0; i < FmActX<LPR_UP>::NIT; i++) {
                const int chn = (threadIdx.x >> 6) + 4 * i;
                fm2_build_chunk<BITS, LPR_UP>(xr0.xl[i], xr0.xh[i], bslot, img0, chn, chn < LPR_UP);
                fm2_build_chunk<BITS, LPR_UP>(xr1.xl[i], xr1.xh[i], bslot, img0 + IMG_UP, chn, chn < LPR_UP && n_up > 1);
            }
        }
        fm_wg_barrier();

        // ---------------------------------------------------------- gate/up
        {
            uint32_t woff, soff;
            int ris, ch;
            fm_unit_lane_offsets<BITS, LPR_UP>(lane, a.g.hidden * BITS / 8, (a.g.hidden / 64) * 2, woff,
                                               soff, ris, ch);
            for (; cq < n_up; cq++) {
                const int s = seg_layer(cq);
                const uint32_t img = img0 + (uint32_t)(cq & 1) * IMG_UP;
                FmActRegs ar;
                fm_read_act_lds_x<LPR_UP>(img, lane, ar);
                const uint32_t ta = fm_lds_addr(&tab[cq]);
                const uint32_t valid = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + (uint32_t)offsetof(Fm2Seg, valid)));
                const uint32_t c_first = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + (uint32_t)offsetof(Fm2Seg, first)));
                const size_t out0 = ((size_t)s * gu_segu + c_first) * RPS_UP + ris;
                dry = false;
                while (issued - consumed < (uint32_t)RING && !dry) issue();
                while (consumed < issued) {
                    const uint32_t tag = fm_slot_peek(ring0 + (uint32_t)c * D::BYTES + D::TAG);
                    if ((tag >> 31) != (uint32_t)(cq & 1)) break;
                    const uint32_t pc = (tag >> 28) & 7u, ul = tag & 0x0FFFFFFFu;
                    const float gv = take<LPR_UP>(woff, soff, ar);
                    const float uv = take<LPR_UP>(woff, soff, ar);
                    float v = fm_silu_mul(gv, uv);
                    if (!((valid >> pc) & 1u)) v = 0.0f;
                    if (ch == 0) fm_st_shared(a.act + out0 + (size_t)ul * RPS_UP, v);
                }
            }
        }
        // ---------------------------------------------------------- down
        {
            uint32_t woff, soff;
            int ris, ch;
            fm_unit_lane_offsets<BITS, LPR_DN>(lane, a.g.inter * BITS / 8, (a.g.inter / 64) * 2, woff,
                                               soff, ris, ch);
            for (; cq < n_seq; cq++) {
                const int l = seg_layer(cq);
                fm_wg_barrier();                       // images and partial vectors are free
                if (cq > n_up) reduce_part(cq - 1);
                // the K activation vectors of the layer -> K images; wave slot (tid / 64) takes
                // the (expert, chunk) combinations slot, slot + 8, ...
                float xl[LPR_DN], xh[LPR_DN];
#pragma unroll
                for (int i = 0; i < LPR_DN; i++) {       // all loads first, polls where needed after
                    const int cmb = (threadIdx.x >> 6) + NW * i;
                    const int k = cmb / LPR_DN, chn = cmb - k * LPR_DN;
                    const float *src = a.act + ((size_t)l * K + (k < K ? k : 0)) * a.g.inter + chn * FM_CPL;
                    xl[i] = fm_ld_shared(src + bslot.lo);
                    xh[i] = fm_ld_shared(src + bslot.hi);
                }
#pragma unroll
                for (int i = 0; i < LPR_DN; i++) {
                    const int cmb = (threadIdx.x >> 6) + NW * i;
                    const int k = cmb / LPR_DN, chn = cmb - k * LPR_DN;
                    const bool on = k < K;
                    const float *src = a.act + ((size_t)l * K + (on ? k : 0)) * a.g.inter + chn * FM_CPL;
                    if (__float_as_uint(xl[i]) == FM_ACT_EMPTY) xl[i] = act_get(src + bslot.lo);
                    if (__float_as_uint(xh[i]) == FM_ACT_EMPTY) xh[i] = act_get(src + bslot.hi);
                    fm2_build_chunk<BITS, LPR_DN>(xl[i], xh[i], bslot, img0 + (uint32_t)(on ? k : 0) * IMG_DN, chn, on);
                }
                fm_wg_barrier();
                const uint32_t ta = fm_lds_addr(&tab[cq]);
                const uint32_t valid = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + (uint32_t)offsetof(Fm2Seg, valid)));
                const uint32_t c_nrb = fm_div(by_K, __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + (uint32_t)offsetof(Fm2Seg, n))));
                FmActRegs ar;
                uint32_t k_cur = 0xFFFFFFFFu;
                dry = false;
                while (issued - consumed < (uint32_t)RING && !dry) issue();
                while (consumed < issued) {
                    const uint32_t tag = fm_slot_peek(ring0 + (uint32_t)c * D::BYTES + D::TAG);
                    if ((tag >> 31) != (uint32_t)(cq & 1)) break;
                    const uint32_t pc = (tag >> 28) & 7u, ul = tag & 0x0FFFFFFFu;
                    if (pc != k_cur) {
                        fm_read_act_lds_x<LPR_DN>(img0 + pc * IMG_DN, lane, ar);
                        k_cur = pc;
                    }
                    float v = take<LPR_DN>(woff, soff, ar);
                    if (!((valid >> pc) & 1u)) v = 0.0f;
                    const uint32_t rbi = ul - pc * c_nrb;
                    if (ch == 0)
                        fm_lds_w32(part0 + 4u * ((rbi * (uint32_t)K + pc) * RPS_DN + (uint32_t)ris), __float_as_uint(v));
                }
            }
            if (n_seq > n_up) {
                fm_wg_barrier();
                if constexpr (TAIL) tail_part(n_seq - 1, *tp, tw, t_hm, t_score, t_nw, t_row0, t_nrb, tl);
                else reduce_part(n_seq - 1);
            }
        }
    }

    // The tail for the rows of part q (the workgroup's only down part).  The rings are empty by now.
    __device__ __forceinline__ void tail_part(int q, const FmTailArgs &ta, const FmRowSlice<4> &tw, float hm,
                                              float score, uint32_t nw, int row0, int nrb, const Fm2TailLds &tl) {
        const int K = a.K;
        const int r_in = lane / LPR_DN, tc = lane % LPR_DN;
        // the shared expert's down projection for these rows: fm_layer_tail's lane map and arithmetic
        if (wave < nrb) {
            float xs[FM_CPL], xsum0, xsum1;
            const uint8_t *part_mem = fm_dyn_lds + D::WG_BYTES + 2 * IMG_UP + FM2_MAX_SEG * sizeof(Fm2Seg);
            fm_load_x<4>(reinterpret_cast<const float *>(part_mem + tl.act) + tc * FM_CPL, xs, xsum0, xsum1);
            const float d = ta.scale_fp16 ? fm_lane_dot<4, true>(tw, xs, xsum0, xsum1)
                                          : fm_lane_dot<4, false>(tw, xs, xsum0, xsum1);
            const float so = fm_group_sum<LPR_DN>(d);
            if (tc == 0) fm_lds_w32(part0 + tl.so + 4u * (uint32_t)(wave * RPS_DN + r_in), __float_as_uint(so));
        }
        fm_wg_barrier();
        const uint32_t tq = fm_lds_addr(&tab[q]);
        float wk[FM_MAX_K];
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            wk[k] = k < K ? __uint_as_float(fm_lds_r32(tq + (uint32_t)offsetof(Fm2Seg, w) + 4u * k)) : 0.0f;
        const int rows = nrb * RPS_DN;
        const bool mine = (int)threadIdx.x < rows;
        float hv = 0.0f;
        if (mine) {
            const int r = threadIdx.x, rbi = r / RPS_DN, ris = r - rbi * RPS_DN;
            float acc = 0.0f;
#pragma unroll
            for (int k = 0; k < FM_MAX_K; k++)
                if (k < K && wk[k] != 0.0f)
                    acc += wk[k] * __uint_as_float(fm_lds_r32(part0 + 4u * (uint32_t)((rbi * K + k) * RPS_DN + ris)));
            const float shared_out = __uint_as_float(fm_lds_r32(part0 + tl.so + 4u * (uint32_t)r));
            const float moe = acc;
            const float shared_gate = 1.0f / (1.0f + expf(-score));
            hv = hm + moe + shared_gate * shared_out;
            fm_st_shared(ta.hidden_out + row0 + r, hv);
            fm_lds_w32(part0 + tl.so + 4u * (uint32_t)r, __float_as_uint(hv));    // (its shared_out is used up)
        }
        if (!ta.next_in) return;
        // The norm needs the sum of squares over all rows.  fm_layer_tail adds them per wave of 16
        // rows (lane 4 r holds row r's square), per workgroup of four such waves, then over the
        // workgroups in order; a row block here is one such wave.  Every workgroup publishes its
        // row blocks' sums (a word that holds the not-yet-produced marker until then), gathers all
        // of them, adds them in that order and normalises its own rows: nothing waits for a last
        // workgroup, and no ticket is drawn.
        fm_wg_barrier();
        if (wave < nrb) {
            const float v = tc == 0 ? __uint_as_float(fm_lds_r32(part0 + tl.so + 4u * (uint32_t)(wave * RPS_DN + r_in))) : 0.0f;
            const float sq = fm_group_sum<64>(v * v);
            if (lane == 0) fm_st_shared(ta.partial + row0 / RPS_DN + wave, sq);
        }
        const int n_vw = ta.hidden / RPS_DN;
        for (int v = threadIdx.x; v < n_vw; v += NW * 64)
            fm_lds_w32(part0 + tl.red + 4u * (uint32_t)v, __float_as_uint(act_get(ta.partial + v)));
        fm_wg_barrier();
        if (wave == 0) {
            float sum_sq = 0.0f;
            for (int b0 = 0; b0 < n_vw / 4; b0 += 64) {
                const int b = b0 + lane;
                float p = 0.0f;
                if (b < n_vw / 4) {
                    const uint32_t ra = part0 + tl.red + 16u * (uint32_t)b;
                    uint2 q01, q23;
                    asm volatile("ds_read2_b32 %0, %2 offset1:1\n\tds_read2_b32 %1, %2 offset0:2 offset1:3\n\ts_waitcnt lgkmcnt(0)"
                                 : "=&v"(q01), "=&v"(q23)
                                 : "v"(ra)
                                 : "memory");
                    p = ((__uint_as_float(q01.x) + __uint_as_float(q01.y)) + __uint_as_float(q23.x)) + __uint_as_float(q23.y);
                }
                const int nb = n_vw / 4 - b0 < 64 ? n_vw / 4 - b0 : 64;
                for (int i = 0; i < nb; i++) sum_sq += __shfl(p, i);
            }
            if (lane == 0) fm_lds_w32(part0 + tl.word, __float_as_uint(sum_sq));
        }
        fm_wg_barrier();
        const float sum_sq = __uint_as_float(fm_lds_r32(part0 + tl.word));
        const float inv_rms = 1.0f / sqrtf(sum_sq / (float)ta.hidden + ta.eps);   // infer.m:1771-1772
        if (mine) {
            const int row = row0 + (int)threadIdx.x;
            ta.next_in[row] = hv * inv_rms * __uint_as_float(nw << 16);
        }
    }
};

template <int BITS, int LPR_UP, bool FP16>
__global__ __launch_bounds__(FM_NW * 64)
void fm_moe_fused_rows(DecodeArgs a, Fm2Dims dm, Fm2Sync sy) {
    Fm2Stream<BITS, LPR_UP, FP16> st(a, sy);
    st.template run<false>(dm, nullptr);
}

// one layer's experts with the layer's tail behind them (Fm2Stream::run<true>)
template <int BITS, int LPR_UP, bool FP16>
__global__ __launch_bounds__(FM_NW_TAIL * 64)
void fm_moe_fused_rows_tail(DecodeArgs a, Fm2Dims dm, Fm2Sync sy, FmTailArgs ta) {
    Fm2Stream<BITS, LPR_UP, FP16, FM_NW_TAIL> st(a, sy);
    st.template run<true>(dm, &ta);
}

// fills n words with v (counters to zero, activations to FM_ACT_EMPTY)
__global__ __launch_bounds__(256) void fm_fill_words(unsigned int *p, unsigned int n, unsigned int v) {
    const unsigned int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

__global__ __launch_bounds__(256) void fm_clear_counters(unsigned int *p, unsigned int n) {
    const unsigned int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// per kernel and device: dynamic LDS limit raised, resident workgroups per CU asked
constexpr int FM_MAX_DEVICES = 64;
struct FmKernelSetup {
    FmLdsAttr lds;
    int per_cu[FM_MAX_DEVICES] = {};   // resident workgroups per CU, 0 = not asked yet
};

int fm_current_device() {
    int d = 0;
    (void)hipGetDevice(&d);
    return d >= 0 && d < FM_MAX_DEVICES ? d : -1;
}

bool fm_dyn_lds_ok(FmKernelSetup &ks, const void *fn, size_t bytes) {
    return fm_dyn_lds_ready(ks.lds, fn, bytes);
}

// workgroups of a streaming launch: one per CU (LDS budget), fewer when there
// are not enough units to give every wave `per_wave` of them
dim3 fm_stream_grid(long units, int n_cu, int per_wave) {
    return dim3((unsigned)fm_stream_wgs(units, n_cu, per_wave, FM_NW));
}

// One fused launch.  Returns FM_ERR_UNSUPPORTED when the grid cannot be made
// fully resident (the caller then uses separate kernels).
template <int BITS, int LPR_UP, bool FP16>
int launch_fused(const DecodeArgs &a, int n_pairs, int n_cu, hipStream_t st, const FmFlags &f) {
    auto kfn = fm_moe_fused<BITS, LPR_UP, FP16>;
    const size_t sh = fm_phase_lds_bytes<BITS, LPR_UP>();
    static FmKernelSetup ks;
    if (!fm_dyn_lds_ok(ks, (const void *)kfn, sh)) return FM_ERR_HIP;
    const int dev = fm_current_device();
    int per_cu = dev >= 0 ? ks.per_cu[dev] : 0;
    if (per_cu == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kfn, FM_NW * 64, sh) !=
            hipSuccess)
            per_cu = 0;
        if (per_cu < 1) per_cu = -1;
        if (dev >= 0) ks.per_cu[dev] = per_cu;
    }
    if (per_cu < 1) return FM_ERR_UNSUPPORTED;   // the grid could not be resident at once
    per_cu = 1;
    const long up_units = (long)n_pairs * (a.g.inter / (FM_WAVE / LPR_UP));
    const long down_units = (long)n_pairs * (a.g.hidden / (FM_WAVE / (LPR_UP / 4)));
    const long wgs = fm1_fused_wgs(up_units, down_units, n_cu);
    hipLaunchKernelGGL(kfn, dim3((unsigned)wgs), dim3(FM_NW * 64), sh, st, a, n_pairs, f);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

// The launch that keeps the per-expert vectors in LDS.  FM_ERR_UNSUPPORTED when the shape does
// not fit its fixed tables (the caller then takes the launch with counters).
template <int BITS, int LPR_UP, bool FP16>
int launch_fused_rows_tail(const DecodeArgs &a, int n_pairs, int n_cu, hipStream_t st, const Fm2Sync &sy,
                           const FmTailArgs &ta) {
    auto kfn = fm_moe_fused_rows_tail<BITS, LPR_UP, FP16>;
    const size_t sh = fm2_lds_bytes<BITS, LPR_UP, FM_NW_TAIL>();
    static FmKernelSetup ks;
    if (!fm_dyn_lds_ok(ks, (const void *)kfn, sh)) return FM_ERR_HIP;
    const int dev = fm_current_device();
    int per_cu = dev >= 0 ? ks.per_cu[dev] : 0;
    if (per_cu == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kfn, FM_NW_TAIL * 64, sh) != hipSuccess)
            per_cu = 0;
        if (per_cu < 1) per_cu = -1;
        if (dev >= 0) ks.per_cu[dev] = per_cu;
    }
    if (per_cu < 1) return FM_ERR_UNSUPPORTED;
    // one layer; the shared expert's down projection has the experts' down shape (its rows are
    // the rows of the experts' sum, its wave step their row block), 4-bit; every workgroup owns
    // at least one row block and the tail's tables fit beside its partial vectors
    if (n_pairs != a.K || ta.hidden != a.g.hidden || ta.inter != a.g.inter || ta.K != 0) return FM_ERR_UNSUPPORTED;
    if (ta.route_logits && (!fm2_route_fits(ta.route_n) || ta.route_n > FM_ROUTE_MAX || a.K > ta.route_n)) return FM_ERR_UNSUPPORTED;
    const Fm2Plan plan = fm2_plan(n_pairs, a.K, a.g.inter, a.g.hidden, LPR_UP, n_cu);
    if (!plan.ok) return FM_ERR_UNSUPPORTED;
    const int rps_dn = FM_WAVE / (LPR_UP / 4), dn_rbs = a.g.hidden / rps_dn;
    if (plan.wgs > dn_rbs) return FM_ERR_UNSUPPORTED;
    const int nrb_max = (dn_rbs + plan.wgs - 1) / plan.wgs;
    if (!fm2_tail_lds(nrb_max, a.K, rps_dn, ta.inter, ta.hidden).ok) return FM_ERR_UNSUPPORTED;
    const Fm2Dims dm = fm2_dims(n_pairs, a.K, plan.wgs, a.g.inter, a.g.hidden, LPR_UP);
    hipLaunchKernelGGL(kfn, dim3((unsigned)plan.wgs), dim3(FM_NW_TAIL * 64), sh, st, a, dm, sy, ta);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

template <int BITS, int LPR_UP, bool FP16>
int launch_fused_rows(const DecodeArgs &a, int n_pairs, int n_cu, hipStream_t st, const Fm2Sync &sy) {
    auto kfn = fm_moe_fused_rows<BITS, LPR_UP, FP16>;
    const size_t sh = fm2_lds_bytes<BITS, LPR_UP>();
    static FmKernelSetup ks;
    if (!fm_dyn_lds_ok(ks, (const void *)kfn, sh)) return FM_ERR_HIP;
    const int dev = fm_current_device();
    int per_cu = dev >= 0 ? ks.per_cu[dev] : 0;
    if (per_cu == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kfn, FM_NW * 64, sh) != hipSuccess)
            per_cu = 0;
        if (per_cu < 1) per_cu = -1;
        if (dev >= 0) ks.per_cu[dev] = per_cu;
    }
    if (per_cu < 1) return FM_ERR_UNSUPPORTED;   // the grid could not be resident at once
    // the kernel's split (Fm2Stream::run): at most two gate/up segments, and the down segments
    // and the row blocks of one part within the fixed tables
    const Fm2Plan plan = fm2_plan(n_pairs, a.K, a.g.inter, a.g.hidden, LPR_UP, n_cu);
    if (!plan.ok) return FM_ERR_UNSUPPORTED;
    const long wgs = plan.wgs;
    const Fm2Dims dm = fm2_dims(n_pairs, a.K, (int)wgs, a.g.inter, a.g.hidden, LPR_UP);
    hipLaunchKernelGGL(kfn, dim3((unsigned)wgs), dim3(FM_NW * 64), sh, st, a, dm, sy);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

template <int BITS, bool FP16>
int launch_decode_t(const DecodeArgs &a, int n_pairs, int rpi_up, int n_cu,
                    hipStream_t st, hipEvent_t *kev, const FmFlags *fl, bool *fused,
                    const Fm2Sync *sy = nullptr, float *act_rows = nullptr, bool *rows = nullptr,
                    const FmTailArgs *tail = nullptr) {
    dim3 b(256);
    const int lpr_up = a.g.hidden / FM_CPL, lpr_down = a.g.inter / FM_CPL;
    const bool lds_up = lpr_up >= 4 && lpr_up <= 16, lds_down = lpr_down <= 16;
    if (!lds_down) return FM_ERR_UNSUPPORTED;
    if (tail) {      // only the launch that sums the experts itself can take the tail along
        if (!(sy && lds_up && lpr_down * 4 == lpr_up)) return FM_ERR_UNSUPPORTED;
        DecodeArgs a2 = a;
        a2.act = act_rows;
        a2.expert_out = nullptr;
        int rc = FM_ERR_UNSUPPORTED;
        switch (lpr_up) {
            case 4: rc = launch_fused_rows_tail<BITS, 4, FP16>(a2, n_pairs, n_cu, st, *sy, *tail); break;
            case 8: rc = launch_fused_rows_tail<BITS, 8, FP16>(a2, n_pairs, n_cu, st, *sy, *tail); break;
            case 16: rc = launch_fused_rows_tail<BITS, 16, FP16>(a2, n_pairs, n_cu, st, *sy, *tail); break;
        }
        if (rows) *rows = rc == FM_OK;
        return rc;
    }
    if (kev) (void)hipEventRecord(kev[0], st);
    if (sy && lds_up && lpr_down * 4 == lpr_up) {
        DecodeArgs a2 = a;
        a2.act = act_rows;
        a2.expert_out = nullptr;
        int rc = FM_ERR_UNSUPPORTED;
        switch (lpr_up) {
            case 4: rc = launch_fused_rows<BITS, 4, FP16>(a2, n_pairs, n_cu, st, *sy); break;
            case 8: rc = launch_fused_rows<BITS, 8, FP16>(a2, n_pairs, n_cu, st, *sy); break;
            case 16: rc = launch_fused_rows<BITS, 16, FP16>(a2, n_pairs, n_cu, st, *sy); break;
        }
        if (rc != FM_ERR_UNSUPPORTED) {
            *rows = rc == FM_OK;
            if (kev) {
                (void)hipEventRecord(kev[1], st);
                (void)hipEventRecord(kev[2], st);
            }
            return rc;
        }
    }
    if (fl && lds_up && lpr_down * 4 == lpr_up) {
        int rc = FM_ERR_UNSUPPORTED;
        switch (lpr_up) {
            case 4: rc = launch_fused<BITS, 4, FP16>(a, n_pairs, n_cu, st, *fl); break;
            case 8: rc = launch_fused<BITS, 8, FP16>(a, n_pairs, n_cu, st, *fl); break;
            case 16: rc = launch_fused<BITS, 16, FP16>(a, n_pairs, n_cu, st, *fl); break;
        }
        if (rc != FM_ERR_UNSUPPORTED) {
            *fused = rc == FM_OK;
            if (kev) {
                (void)hipEventRecord(kev[1], st);
                (void)hipEventRecord(kev[2], st);
            }
            return rc;
        }
    }
    if (lds_up) {
        const long units = (long)n_pairs * (a.g.inter / (FM_WAVE / lpr_up));
        const dim3 g = fm_stream_grid(units, n_cu, 2);
#define FM_UP(L)                                                                   \
    do {                                                                           \
        auto kfn = fm_gate_up_swiglu_lds<BITS, L, FP16>;                           \
        const size_t sh = fm_phase_lds_bytes<BITS, L>();                           \
        static FmKernelSetup ks;                                                   \
        if (!fm_dyn_lds_ok(ks, (const void *)kfn, sh)) return FM_ERR_HIP;          \
        hipLaunchKernelGGL(kfn, g, dim3(FM_NW * 64), sh, st, a, n_pairs);          \
    } while (0)
        switch (lpr_up) {
            case 4: FM_UP(4); break;
            case 8: FM_UP(8); break;
            default: FM_UP(16); break;
        }
#undef FM_UP
    } else if (lpr_up == 32) {
        DecodeArgs a1 = a;
        a1.rows_per_item = rpi_up;
        a1.items_per_pair = a.g.inter / rpi_up;
        hipLaunchKernelGGL((fm_gate_up_swiglu<BITS, 32, FP16>), dim3(n_pairs * a1.items_per_pair),
                           b, 0, st, a1);
    } else {
        return FM_ERR_UNSUPPORTED;
    }
    if (kev) (void)hipEventRecord(kev[1], st);
    {
        const long units = (long)n_pairs * (a.g.hidden / (FM_WAVE / lpr_down));
        const dim3 g = fm_stream_grid(units, n_cu, 2);
#define FM_DOWN(L)                                                                 \
    do {                                                                           \
        auto kfn = fm_down_lds<BITS, L, FP16>;                                     \
        const size_t sh = fm_phase_lds_bytes<BITS, L>();                           \
        static FmKernelSetup ks;                                                   \
        if (!fm_dyn_lds_ok(ks, (const void *)kfn, sh)) return FM_ERR_HIP;          \
        hipLaunchKernelGGL(kfn, g, dim3(FM_NW * 64), sh, st, a, n_pairs);          \
    } while (0)
        switch (lpr_down) {
            case 1: FM_DOWN(1); break;
            case 2: FM_DOWN(2); break;
            case 4: FM_DOWN(4); break;
            case 8: FM_DOWN(8); break;
            default: FM_DOWN(16); break;
        }
#undef FM_DOWN
    }
    const int n_groups = n_pairs / a.K;
    if (a.flags & FM_GUARD)
        hipLaunchKernelGGL(fm_combine<true>, dim3(n_groups), b, 0, st, a);
    else
        hipLaunchKernelGGL(fm_combine<false>, dim3(n_groups, (a.g.hidden + 255) / 256), b, 0, st, a);
    if (kev) (void)hipEventRecord(kev[2], st);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

// rows per workgroup: min_rows * 2^j dividing `rows`, as large as possible (at
// most `cap`) while the launch still has at least `want` workgroups
int pick_rows_per_item(int rows, int n_pairs, int min_rows, int cap, int want) {
    int rpi = min_rows;
    while (rpi * 2 <= cap && rows % (rpi * 2) == 0 && (rows / (rpi * 2)) * n_pairs >= want)
        rpi *= 2;
    return rpi;
}

}  // namespace


// Enqueue the operator for n_layers x K pairs (n_layers groups of K slots: the
// layers of a decode step, or with layer_stride 0 the positions of a chunk).  Shapes are validated by the
// caller (fm_api.cpp): hidden, inter multiples of 128 with a supported
// lanes-per-row, every layer resident.
extern "C" int fm_launch_decode_affine(const uint8_t *const *d_layer_ptrs,
                                       const FmExpertGeom *g, int layer0, int layer_stride,
                                       int n_layers, const float *d_x, const int32_t *d_idx,
                                       const float *d_w, int K, float *d_act,
                                       float *d_expert_out, float *d_out,
                                       FmDecodeFlags *df, int flags, int n_cu,
                                       hipStream_t st, hipEvent_t *kev, const FmTailArgs *tail) {
    DecodeArgs a;
    a.layer_ptrs = d_layer_ptrs;
    a.g = *g;
    a.layer0 = layer0;
    a.layer_stride = layer_stride;
    a.K = K;
    a.x = d_x;
    a.idx = d_idx;
    a.w = d_w;
    a.act = d_act;
    a.expert_out = d_expert_out;
    a.out = d_out;
    a.flags = flags;
    a.rows_per_item = a.items_per_pair = 0;
    const int n_pairs = n_layers * K;
    const int lpr_up = g->hidden / FM_CPL, lpr_down = g->inter / FM_CPL;
    if (lpr_up < 1 || lpr_down < 1) return FM_ERR_UNSUPPORTED;
    // a wave step covers 64/LPR rows and a workgroup has 4 waves
    const int min_up = 4 * (FM_WAVE / lpr_up), min_down = 4 * (FM_WAVE / lpr_down);
    if (g->inter % min_up || g->hidden % min_down) return FM_ERR_UNSUPPORTED;
    const int want = 4 * n_cu;
    const int rpi_up = pick_rows_per_item(g->inter, n_pairs, min_up, 64, want);
    // with dependency counters (and room in them) the operator is one launch,
    // otherwise the phases run as separate kernels
    const unsigned int need = (unsigned int)(n_pairs + n_layers);
    FmFlags fl{};
    const FmFlags *flp = nullptr;
    // A launch that is being captured into a graph will be replayed without this function: it
    // gets the counter set kept for graphs and, recorded in front of it, a kernel that clears it.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (df && df->set[0]) (void)hipStreamIsCapturing(st, &capture);
    const bool captured = capture == hipStreamCaptureStatusActive;
    // (the entry point that allocates nothing has one counter set only: it takes the graph's
    // route whether or not the stream is capturing)
    const bool own_clear = captured || (df && df->always_graph_set);
    if (tail && (own_clear || !df)) return FM_ERR_UNSUPPORTED;    // (the caller chains the two launches)
    if (df && (df->set[0] || df->always_graph_set) && need <= df->cap) {
        if (own_clear) {
            hipLaunchKernelGGL(fm_clear_counters, dim3((need + 255) / 256), dim3(256), 0, st,
                               df->graph_set, need);
            fl.cur = df->graph_set;
            fl.other = df->graph_set;
            fl.clear_n = 0u;
        } else {
            fl.cur = df->set[df->parity];
            fl.other = df->set[df->parity ^ 1];
            fl.clear_n = df->used[df->parity ^ 1];
        }
        fl.err = df->err;
        fl.spin_limit = df->spin_limit;
        flp = &fl;
    }
    // without per-expert vectors and without the finite guard: the launch that sums in LDS
    Fm2Sync sy{};
    const Fm2Sync *syp = nullptr;
    float *act_rows = nullptr;
    // (with the tail along: one more vector for the row blocks' sums of squares, behind the activations)
    const unsigned int act_need = (unsigned int)n_pairs * (unsigned int)g->inter + (tail ? (unsigned int)g->hidden : 0u);
    if (flp && (flags & FM_INT_NO_EXPERT_OUT) && !(flags & FM_GUARD) && df->act_cap >= act_need &&
        df->act_set[0]) {
        if (own_clear) {
            if (df->act_graph) {
                hipLaunchKernelGGL(fm_fill_words, dim3((act_need + 255) / 256), dim3(256), 0, st,
                                   (unsigned int *)df->act_graph, act_need, FM_ACT_EMPTY);
                act_rows = df->act_graph;
                sy.act_other = df->act_graph;
                sy.clear_n = 0u;
            }
        } else {
            act_rows = df->act_set[df->act_parity];
            sy.act_other = df->act_set[df->act_parity ^ 1];
            sy.clear_n = df->act_used[df->act_parity ^ 1];
        }
        if (act_rows) {
            sy.err = df->err;
            sy.spin_limit = df->spin_limit;
            syp = &sy;
        }
    }
    a.flags = flags & ~FM_INT_NO_EXPERT_OUT;
    bool fused = false, rows = false;
    FmTailArgs tail_args{};
    if (tail) {
        if (!syp) return FM_ERR_UNSUPPORTED;      // (the caller chains the two launches)
        tail_args = *tail;
        tail_args.partial = act_rows + (size_t)n_pairs * g->inter;
        tail = &tail_args;
    }
#define FM_DEC(B, F) launch_decode_t<B, F>(a, n_pairs, rpi_up, n_cu, st, kev, flp, &fused, syp, act_rows, &rows, tail)
    int rc = FM_ERR_UNSUPPORTED;
    if (g->bits == 3) rc = g->scale_fp16 ? FM_DEC(3, true) : FM_DEC(3, false);
    else if (g->bits == 4) rc = g->scale_fp16 ? FM_DEC(4, true) : FM_DEC(4, false);
#undef FM_DEC
    if (rows && !own_clear) {    // the set just filled is in use, the other one is all markers again
        df->act_used[df->act_parity] = act_need;
        df->act_used[df->act_parity ^ 1] = 0u;
        df->act_parity ^= 1;
    }
    if (fused && !own_clear) {   // the set just used is dirty, the other one is clean again
        df->used[df->parity] = need;
        df->used[df->parity ^ 1] = 0u;
        df->parity ^= 1;
    }
    return rc;
}
