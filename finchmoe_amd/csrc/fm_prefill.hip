// fm_prefill.hip — chunks of many positions on the matrix cores: the routed experts' products
// grouped by expert (affine 3-/4-bit stores and GGUF Q4_K / Q6_K stores), and dense affine
// tensors against M positions.
//
// The reference has no GEMM here: prefill_chunk_cmd3_encode (finchmoe/infer.m:
// 10704-10765) runs the per-position GEMV chain for each of the M positions, so two
// positions routed to the same expert read its weights twice.  This file groups
// the M*K (position, slot) pairs by expert and multiplies each expert's weights
// once against a group of its positions.  Numerical contract: the per-position
// result (fm_decode.hip, fm_gguf.hip) within the parity bar.
//
// Why not "dequantize to bf16 and multiply": rounding (q*s + b) to bf16 misses
// the bar (max relative error 1.8e-3 on the benchmark's weight distribution).
// Instead
//   * the CODES are the MFMA operand, as exact bf16 numbers 1 + q*2^t/128 (the
//     mantissa trick of fm_mfma.h: one V_AND_OR_B32 per two codes);
//   * each quantization group is accumulated by its own MFMA chain and its scale is
//     applied to the result in fp32: acc += s[row][g] * D_g;
//   * fp32 activations are split hi + lo (two bf16 pieces, 16 significant bits), bf16
//     activations are operands as they are;
//   * the bias term sum_g b[row][g] * xsum[pos][g] and the offset the "1 +" adds are
//     small products over the group index (affine stores: on MFMA as well, the bf16 bits
//     of b and s being operands as they are; GGUF stores: in fp32 on the accumulators).
//
// Kernels of a chunk of routed experts:
//   fm_pf_group        one workgroup groups the pairs by expert and cuts every expert's
//                      positions into items (two lists: gate/up and down items may differ
//                      in size)
//   fm_pf_rows<GATE_UP>, fm_pf_rows<DOWN>     affine stores: row-tile kernels, see below
//   fm_gq_gate_up, fm_gq_down                 GGUF stores
//   fm_pf_combine      weighted sum of a position's K expert outputs in slot order
// Dense tensors: fm_pf_dense_prep (X -> operand registers, once per chunk) and fm_pf_gemm
// (V_MFMA_F32_32X32X16_BF16, K split over the waves of a workgroup, partial tiles summed
// through LDS).
#include "fm_index.h"
#include "fm_mfma.h"
#include "fm_ring.h"

#include <type_traits>

namespace {

typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef const __attribute__((address_space(1))) uint8_t *gptr;

#define PF_TM FM_PF_TM    // positions per item
#define PF_MAX_EXPERTS 1024

struct PfItem { int expert, start, count, pad; };

struct PfArgs {
    const uint8_t *layer;
    FmExpertGeom g;
    const float *X;
    const int32_t *idx;
    const float *w;
    int M, K;
    int *sorted;       // [M*K] pair ids grouped by expert
    PfItem *items;     // [n_experts + M*K/PF_TM]
    int *n_items;
    float *act;        // [M*K][inter], by sorted position
    float *eo;         // [M*K][hidden], by pair id
    uint4 *xop;        // [M][hidden/64][k step 4][half 2][piece 2]: X as MFMA operand registers
    float2 *xsums;     // [M][hidden/64]: (xsum, xoff) of every group of every position
    // dense tensor (PF_DENSE): out[M][d_rows] = X[M][d_cols] * W^T, scales / biases d_sb bytes
    // behind / before W; one launch covers the 2048 columns of pass d_pass
    const uint8_t *d_w;
    ptrdiff_t d_s, d_b;
    int d_rows, d_cols, d_pass, d_flags;
    float *d_out;
    // row-tile kernels (fm_pf_rows): X as bf16 bits when the caller has them, the two item
    // lists (gate/up and down may cut an expert's positions into items of different size)
    const uint16_t *Xbf;
    PfItem *items_up, *items_dn;
    int *n_items_up, *n_items_dn;
    int tm_up, tm_dn;
    // GGUF experts (fm_gq_gate_up / fm_gq_down): the layer's three slabs
    const uint8_t *gq_gate, *gq_up, *gq_down;
};

enum { PF_DENSE = 2, PF_DENSE_TEAMS = 3 };

// ---- pairing of the 32 codes a lane holds for one group -------------------
// Pair p fills k slots 2p (low half of the register, code lo(p) at mantissa bit tl(p)) and
// 2p+1 (high half, code hi(p) at bit th(p)); the pair is cut out of the lane's DW dwords at
// stream bit start(p) with one mask.
template <int BITS>
struct PfCode;
// 3 bits: two blocks of 10 codes 5 apart (tl=4, th=3), one block of 12 codes 6 apart (tl=2, th=4)
template <>
struct PfCode<3> {
    static constexpr int DW = 3;
    static constexpr int lo(int p) { return p < 10 ? 10 * (p / 5) + p % 5 : 20 + (p - 10); }
    static constexpr int hi(int p) { return lo(p) + (p < 10 ? 5 : 6); }
    static constexpr int tl(int p) { return p < 10 ? 4 : 2; }
    static constexpr int th(int p) { return p < 10 ? 3 : 4; }
    static constexpr int start(int p) { return 3 * lo(p) - tl(p); }
    static constexpr uint32_t mask(int p) { return (7u << tl(p)) | (7u << (16 + th(p))); }
};
// 4 bits: nibbles a and a + 4 of a dword are 16 bits apart already
template <>
struct PfCode<4> {
    static constexpr int DW = 4;
    static constexpr int lo(int p) { return 8 * (p / 4) + p % 4; }
    static constexpr int hi(int p) { return lo(p) + 4; }
    static constexpr int tl(int) { return 0; }
    static constexpr int th(int) { return 0; }
    static constexpr int start(int p) { return 4 * lo(p); }
    static constexpr uint32_t mask(int) { return 0x000F000Fu; }
};

template <int BITS, int P>
__device__ __forceinline__ uint32_t pf_pair(const uint32_t *d, uint32_t ones) {
    using C = PfCode<BITS>;
    uint32_t w = fm_window<C::start(P), C::DW>(d);
    return (w & C::mask(P)) | ones;
}

// the 16 operand registers of a lane's 32 codes
template <int BITS, int P>
__device__ __forceinline__ void pf_unpack(const uint32_t *d, uint32_t ones, uint32_t *v) {
    if constexpr (P < 16) {
        v[P] = pf_pair<BITS, P>(d, ones);
        pf_unpack<BITS, P + 1>(d, ones, v);
    }
}

template <int BITS, int S, int Q>
__device__ __forceinline__ void pf_stage_pair(const float *x, uint32_t *hi, uint32_t *lo, float &xs,
                                              float &xo) {
    using C = PfCode<BITS>;
    constexpr int p = 4 * S + Q;
    constexpr float cl = (float)(128 >> C::tl(p)), ch = (float)(128 >> C::th(p));
    float vl = x[C::lo(p)] * cl, vh = x[C::hi(p)] * ch;
    // exact split into bf16 pieces; hi + lo = the value truncated to 16 significant bits
    uint32_t l0 = __float_as_uint(vl) & 0xFFFF0000u, h0 = __float_as_uint(vh) & 0xFFFF0000u;
    float rl = vl - __uint_as_float(l0), rh = vh - __uint_as_float(h0);
    uint32_t l1 = __float_as_uint(rl) & 0xFFFF0000u, h1 = __float_as_uint(rh) & 0xFFFF0000u;
    hi[Q] = (l0 >> 16) | h0;
    lo[Q] = (l1 >> 16) | h1;
    float tl = __uint_as_float(l0) + __uint_as_float(l1), th = __uint_as_float(h0) + __uint_as_float(h1);
    xo += tl + th;
    xs += tl * (1.0f / cl) + th * (1.0f / ch);
}

// ---------------------------------------------------------------- kernels
// X in the form the dense kernel multiplies with: per position, group, k step and column
// half the four operand registers of the hi pieces and of the lo pieces (pf_stage_pair), and
// per position and group the two sums the bias and offset terms need.  Done once per chunk:
// a position is multiplied by K experts, and splitting it inside the multiply kernel cost a
// fifth of that kernel's time.  Task = (position, group, half).
template <int BITS, int S>
__device__ __forceinline__ void pf_prepare_steps(const float *x, uint4 *dst, float &xs, float &xo) {
    if constexpr (S < 4) {
        uint32_t hi[4], lo[4];
        pf_stage_pair<BITS, S, 0>(x, hi, lo, xs, xo);
        pf_stage_pair<BITS, S, 1>(x, hi, lo, xs, xo);
        pf_stage_pair<BITS, S, 2>(x, hi, lo, xs, xo);
        pf_stage_pair<BITS, S, 3>(x, hi, lo, xs, xo);
        dst[4 * S] = make_uint4(hi[0], hi[1], hi[2], hi[3]);          // [k step][half][piece]
        dst[4 * S + 1] = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        pf_prepare_steps<BITS, S + 1>(x, dst, xs, xo);
    }
}

template <int BITS>
__device__ __forceinline__ void pf_prepare(const float *src, int rows, int cols, uint4 *dst_op,
                                           float2 *dst_sums, int task) {
    const int NG = cols / 64;
    const FmPfPrepTask pt = fm_pf_prep_task(task, NG);
    const int h = pt.h, g = pt.g, m = pt.m;
    const bool on = m < rows;
    float x[32];
    if (on) {
        const float4 *xp = reinterpret_cast<const float4 *>(src + (size_t)m * cols + 64 * g + 32 * h);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float4 v = xp[i];
            x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 32; i++) x[i] = 0.0f;
    }
    float xs = 0.0f, xo = 0.0f;
    // this half's registers: index ((m*NG + g)*4 + k)*4 + 2*half + piece
    uint4 regs[16];
    pf_prepare_steps<BITS, 0>(x, regs, xs, xo);
    // the two halves of a group sit in adjacent lanes
    xs += fm_dpp<0xB1>(xs);
    xo += fm_dpp<0xB1>(xo);
    if (on) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            dst_op[fm_pf_xop_index((size_t)m, NG, g, k, h, 0)] = regs[4 * k];
            dst_op[fm_pf_xop_index((size_t)m, NG, g, k, h, 1)] = regs[4 * k + 1];
        }
        if (h == 0) dst_sums[(size_t)m * NG + g] = make_float2(xs, xo);
    }
}

// ======================================================================
// The GEMM kernel (fm_pf_gemm): 512 threads, one workgroup per CU.
//
// The K dimension is cut into slabs of four groups (256 columns) and a wave
// owns one slab of every row it visits: gate/up has eight slabs, one per wave;
// down has two, and the eight waves form four teams on different rows.
//   * A wave's share of the activation operand is 16 registers per group,
//     loaded ready-made (pf_prepare) once per item; LDS holds no activations.
//     (An earlier form kept the whole operand of an item in LDS and let every
//     wave sweep row tiles over the full K with per-lane 12-byte weight loads:
//     the address unit, not the matrix core, was its busiest part.)
//   * A tile-matrix (32 rows of one matrix) x slab is 32 runs of 96 bytes: the
//     wave copies them, with the rows' scales and biases, into a ring slot with
//     LDS-direct loads (whole runs, several slots in flight), and every lane
//     reads its 12-byte pieces back.
//   * Bias and offset terms ride in two extra MFMAs per tile-matrix whose K
//     slots are (piece, group) of the wave's own groups.
//   * The partial tiles of a row tile's slabs are summed through LDS in slab
//     order; SwiGLU / store happen there.  One barrier per step (two
//     tile-matrices per wave), two partial buffers.
// ======================================================================
template <int BITS>
struct PfSlab {
    static constexpr FmPfSlab G = fm_pf_slab(BITS);     // shared with the host-side bounds walk
    static constexpr int GPW = 4;                       // groups per wave
    static constexpr int CB = G.cb;                     // code bytes of a row inside the slab: 96 / 128
    static constexpr int PS = 16;                       // bytes a lane copies per load
    static constexpr int RP = G.rp;                     // pieces per row: 6 / 8
    // a row takes one piece slot more in LDS (it stays empty): with 96- or 128-byte rows the
    // 128-bit reads of neighbouring rows would hit the same banks
    static constexpr int RS = G.rs;                     // piece slots per row in LDS: 7 / 9
    static constexpr int PIECES = G.pieces;             // piece slots of a tile-matrix: 224 / 288
    static constexpr int NQ = G.nq;                     // LDS-direct loads for the codes
    static constexpr int LDS_CODE = G.lds_code;         // 3584 / 4608
    static constexpr int SLOT = G.slot;                 // + scales 256 + biases 256
    static constexpr int LOADS = NQ + 2;
    static constexpr int RED_BYTES = 2 * 2 * 8 * 8 * 64 * 4;   // [buffer][matrix][wave][reg][lane]
    // what is left of the 160 KB for the eight waves' rings: 3 slots of 4096 B / 2 of 5120 B
    static constexpr int RING = G.ring;
    static constexpr int LDS_BYTES = G.lds_bytes;
    static_assert(RING >= 2, "a ring needs a slot in flight beside the one being multiplied");
    static_assert(LDS_BYTES == 8 * RING * SLOT + RED_BYTES && LDS_BYTES <= 160 * 1024, "LDS layout");
};

// three bf16 pieces (bit patterns) of v, the last one truncated
__device__ __forceinline__ void pf_pieces(float v, uint32_t *pc) {
    uint32_t b = __float_as_uint(v) & 0xFFFF0000u;
    pc[0] = b >> 16;
    v -= __uint_as_float(b);
    b = __float_as_uint(v) & 0xFFFF0000u;
    pc[1] = b >> 16;
    v -= __uint_as_float(b);
    pc[2] = __float_as_uint(v) >> 16;
}

// B operands of the bias / offset MFMAs: the slab's four 16-bit values of a row (w0 = groups
// 0, 1; w1 = groups 2, 3) against the K slots of this half lane — hh = 0: piece 0 and piece 1
// of the activation sums, hh = 1: piece 2 and piece 0 again.  BF16 values are operands as they
// are (the fourth slot group stays empty).  An FP16 value (11 significant bits) is split exactly
// into a bf16 head (8 bits) and tail (3 bits): heads everywhere, the tails in the fourth slot
// group; tail x piece 1, as large as head x piece 2, goes into one more MFMA for both terms
// (`tails`); tail x piece 2 is below fp32 precision.
template <bool FP16>
__device__ __forceinline__ uint4 pf_side_b(uint32_t w0, uint32_t w1, int hh, uint2 &tails) {
    if constexpr (!FP16) {
        tails = make_uint2(0u, 0u);
        return hh ? make_uint4(w0, w1, 0u, 0u) : make_uint4(w0, w1, w0, w1);
    } else {
        uint32_t head[4], tail[4];
        const float f[4] = {fm_fp16_bits(w0 & 0xFFFFu), fm_fp16_bits(w0 >> 16), fm_fp16_bits(w1 & 0xFFFFu),
                            fm_fp16_bits(w1 >> 16)};
#pragma unroll
        for (int g = 0; g < 4; g++) {
            head[g] = __float_as_uint(f[g]) & 0xFFFF0000u;
            tail[g] = __float_as_uint(f[g] - __uint_as_float(head[g]));
        }
        const uint32_t h0 = (head[0] >> 16) | head[1], h1 = (head[2] >> 16) | head[3];
        tails = make_uint2((tail[0] >> 16) | (tail[1] & 0xFFFF0000u), (tail[2] >> 16) | (tail[3] & 0xFFFF0000u));
        return hh ? make_uint4(h0, h1, tails.x, tails.y) : make_uint4(h0, h1, h0, h1);
    }
}

// MODE PF_DENSE: one dense tensor against M positions, 2048 of its columns per launch (eight
//   slabs, wave w owns slab w, all waves work on the same rows; column pass d_pass adds to what
//   the passes before it stored); an item is a block of 16 positions, a step = two row tiles
//   (64 rows), the partial tiles of the eight waves are summed through LDS; the operand comes
//   from xop (fm_pf_dense_prep).
// MODE PF_DENSE_TEAMS: a dense tensor of 512 columns: two slabs, the workgroup is four teams of
//   two waves (slab = wave & 1), every team on its own 64 rows of a step's 256; operand and
//   output as in PF_DENSE.
template <int MODE, int BITS, bool FP16>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void fm_pf_gemm(PfArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // (the host pass cannot allocate the registers of the asm blocks)
    using P = PfSlab<BITS>;
    constexpr int DW = PfCode<BITS>::DW;
    // TEAMS: 512 columns as two slabs, four teams of two waves; DENSE: 2048 columns per pass
    constexpr bool TEAMS = MODE == PF_DENSE_TEAMS, DENSE = MODE == PF_DENSE;
    static_assert(TEAMS || DENSE, "dense tensors only (the expert products are fm_pf_rows)");
    constexpr int GPW = P::GPW;
    constexpr int RING = P::RING;
    extern __shared__ __attribute__((aligned(16))) uint8_t pf2_smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 31, hh = lane >> 5;
    const uint32_t lds0 = fm_lds_addr(pf2_smem);
    const uint32_t ring0 = lds0 + (uint32_t)wave * (RING * P::SLOT);
    const uint32_t red0 = lds0 + 8 * RING * P::SLOT;
    const int n_items = *a.n_items;
    const int in_dim = a.d_cols;
    const int row_bytes = in_dim * BITS / 8, sb_bytes = (in_dim / 64) * 2;
    const int slab = DENSE ? wave + 8 * a.d_pass : TEAMS ? (wave & 1) : wave, team = TEAMS ? (wave >> 1) : 0;
    const int n_steps = DENSE ? a.d_rows / 64 : a.d_rows / 256;
    const uint32_t ones = fm_opaque(0x3F803F80u);
    // region offsets of the first tile-matrix of a step (this team's), the distance to the
    // second one, rows per step
    // (byte offsets from the blob's — the dense tensor's W — first byte, modulo 2^64)
    const size_t s_off0 = (size_t)a.d_s, b_off0 = (size_t)a.d_b;
    const uint8_t *store = a.d_w;       // (an item's "expert" is 0: one tensor)
    const size_t expert_size = 0;
    // this lane's pieces of a slot copy
    uint32_t coff[P::NQ];
    bool cvalid[P::NQ];
#pragma unroll
    for (int j = 0; j < P::NQ; j++) {
        int v;
        coff[j] = fm_pf_piece_off(P::G, j, lane, row_bytes, slab, &v);
        cvalid[j] = v != 0;
    }
    // scales / biases of the slab: 2*GPW bytes per row, fetched as whole dwords
    const uint32_t soff = fm_pf_sb_off(lane, sb_bytes, slab);

    // ---- this workgroup's share of the launch: steps [t0, t1) of the sequence
    // (item, step), items in order — every workgroup gets the same number of steps
    // (within one) whatever the number of items, at the price of building the
    // activation operand of an item in two workgroups when a share ends inside it
    // Workgroups are dealt out to the eight XCDs in turn and every XCD has an L2 of its own:
    // workgroup b takes share (b % 8) * (grid / 8) + b / 8, so that neighbouring shares — the
    // items of one expert — run behind the same L2 and its weights come from HBM once.
    const FmRange tr = fm_share((long)n_items * n_steps, fm_xcd_share(blockIdx.x, gridDim.x), gridDim.x);
    const int t0 = (int)tr.lo, t1 = (int)tr.hi;

    // ---- loader: tile-matrices of the share, in order
    int l_t = t0, l_it = t0 / n_steps, l_mat = 0, wpos = 0;
    int l_s = t0 - l_it * n_steps;
    uint32_t issued = 0, consumed = 0;
    bool l_done = t0 >= t1;
    const uint8_t *l_blob = nullptr;
    // expert of the item after the one being multiplied: the loader enters that item a few
    // slices before the multiply does, and a load here would wait for the whole ring
    int e_ahead = 0;
    if (!l_done) {
        l_blob = fm_uniform(store + (size_t)a.items[l_it].expert * expert_size);
        if (l_it + 1 < n_items) e_ahead = a.items[l_it + 1].expert;
    }
    auto issue = [&]() __attribute__((always_inline)) {
        if (l_done) return;
        const uint32_t slot = ring0 + (uint32_t)wpos * P::SLOT;
        const size_t row0 = fm_pf_dense_row(l_s, l_mat, team, TEAMS);
        const uint8_t *wb = l_blob + row0 * row_bytes;
        const uint8_t *sb = l_blob + (s_off0 + row0 * sb_bytes);
        const uint8_t *bb = l_blob + (b_off0 + row0 * sb_bytes);
#pragma unroll
        for (int j = 0; j < P::NQ; j++)
            if (cvalid[j])
                __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(wb + coff[j]),
                                                 (fm_lptr)(uintptr_t)(slot + 64 * P::PS * j),
                                                 P::PS, 0, 0);
        __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(sb + soff),
                                         (fm_lptr)(uintptr_t)(slot + P::LDS_CODE), 4, 0, 0);
        __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(bb + soff),
                                         (fm_lptr)(uintptr_t)(slot + P::LDS_CODE + 256), 4, 0, 0);
        wpos = wpos + 1 == RING ? 0 : wpos + 1;
        issued++;
        l_mat ^= 1;
        if (l_mat == 0) {
            if (++l_t >= t1) {
                l_done = true;
            } else if (++l_s == n_steps) {
                l_s = 0;
                l_it++;
                l_blob = fm_uniform(store + (size_t)e_ahead * expert_size);
            }
        }
    };
#pragma unroll
    for (int k = 0; k < RING; k++) issue();

    int c = 0, buf = 0;
    // What an item's start needs is fetched one item ahead — the item itself, the position
    // (row of X) this lane multiplies, the next expert for the loader — so that the start
    // costs one memory round trip (the operand registers) instead of a chain of three, each
    // of which would also drain the ring.
    PfItem item_next = PfItem{0, 0, 0, 0};
    if (t0 < t1) item_next = a.items[t0 / n_steps];
    for (int t = t0; t < t1;) {
        const int it = t / n_steps, s_begin = t - it * n_steps;
        const int s_end = t1 - t < n_steps - s_begin ? s_begin + (t1 - t) : n_steps;
        t += s_end - s_begin;
        const PfItem item = item_next;
        const bool more = t < t1;                  // this workgroup goes on to item it + 1
        if (more) item_next = a.items[it + 1];
        // ---- this wave's share of the activation operand, straight into registers:
        // lane (m, hh): M row m = hi piece of position m (m < 16) or lo piece of position
        // m - 16; k slots 8*hh .. 8*hh+7 of every k step = columns 32*hh .. 32*hh+31 of the group
        uint4 A[GPW][4];
        uint32_t sideA[2][4];
        {
            const int pos = n & 15;
            const bool on = pos < item.count;
            float xs[GPW], xo[GPW];
            {
                // X was turned into operand registers once per chunk (pf_prepare): lane (m, hh)
                // takes the hi (m < 16) or lo registers of its position, its groups, its half
                const int piece = n < 16 ? 0 : 1;
                const size_t m = !on ? 0 : (size_t)(item.start + pos);
                const int ng = in_dim / 64;
                const float2 *sm = a.xsums + m * ng + GPW * slab;
#pragma unroll
                for (int gi = 0; gi < GPW; gi++) {
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        A[gi][k] = a.xop[fm_pf_xop_index(m, ng, GPW * slab + gi, k, hh, piece)];
                    const float2 v = sm[gi];
                    xs[gi] = on ? v.x : 0.0f;
                    xo[gi] = on ? v.y : 0.0f;
                }
                // The registers are first used inside the multiply loop, which issues LDS-direct
                // loads of its own: left alone, the compiler's wait for THESE loads lands in the
                // loop and drains the ring on every pass.  Touch them here so that it waits now.
#pragma unroll
                for (int gi = 0; gi < GPW; gi++)
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        fm_u4 t = __builtin_bit_cast(fm_u4, A[gi][k]);
                        asm volatile("" : "+v"(t));
                        if (!on) t = fm_u4{0u, 0u, 0u, 0u};     // rows past the item's positions
                        A[gi][k] = __builtin_bit_cast(uint4, t);
                    }
                if (more) e_ahead = item_next.expert;     // the loader enters it during this item
            }
            // K slots of the bias/offset MFMAs: slot = 4*piece + group, one MFMA per term (xsum
            // for the biases, -xoff for the scales).  Rows 16..31 (lo pieces) take no part.
#pragma unroll
            for (int term = 0; term < 2; term++) {
                uint32_t pc[4][3];
#pragma unroll
                for (int gi = 0; gi < 4; gi++) pf_pieces(term ? -xo[gi] : xs[gi], pc[gi]);
                const int p0 = hh ? 2 : 0;
                sideA[term][0] = pc[0][p0] | (pc[1][p0] << 16);
                sideA[term][1] = pc[2][p0] | (pc[3][p0] << 16);
                // (hh = 1: piece 0 once more, for the tails of FP16 scales and biases; BF16 ones
                // put zeros against it)
                sideA[term][2] = hh ? pc[0][0] | (pc[1][0] << 16) : pc[0][1] | (pc[1][1] << 16);
                sideA[term][3] = hh ? pc[2][0] | (pc[3][0] << 16) : pc[2][1] | (pc[3][1] << 16);
                if (n >= 16) sideA[term][0] = sideA[term][1] = sideA[term][2] = sideA[term][3] = 0u;
            }
        }
        // output position of result register r = wave of this lane
        const int my_pos = 8 * (wave >> 2) + 4 * hh + (wave & 3);
        const bool my_on = my_pos < item.count;

        for (int s = s_begin; s < s_end; s++) {
#pragma unroll
            for (int mat = 0; mat < 2; mat++) {
                // The hardware issues the older of two waves on a SIMD first, which lets waves
                // 0-3 run ahead and wait at every barrier for waves 4-7: take turns instead.
                if (((wave >> 2) ^ mat) & 1) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
                // ---- the oldest slot of the ring
                if (issued - consumed == (uint32_t)RING) fm_dma_wait<P::LOADS *(RING - 1)>(false);
                else fm_dma_wait<0>(true);
                const uint32_t slot = ring0 + (uint32_t)c * P::SLOT;
                uint32_t cw[GPW][DW], sw[2], bw[2];
                if constexpr (BITS == 4) {
                    // a lane's half of a group is one 16-byte piece
                    const uint32_t ac = slot + (uint32_t)(n * (P::RS * 16) + 16 * hh);
                    const uint32_t as = slot + P::LDS_CODE + 8 * n;
                    fm_u4 r0, r1, r2, r3;
                    asm volatile(
                        "ds_read_b128 %0, %8\n\tds_read_b128 %1, %8 offset:32\n\t"
                        "ds_read_b128 %2, %8 offset:64\n\tds_read_b128 %3, %8 offset:96\n\t"
                        "ds_read_b32 %4, %9\n\tds_read_b32 %5, %9 offset:4\n\t"
                        "ds_read_b32 %6, %9 offset:256\n\tds_read_b32 %7, %9 offset:260\n\t"
                        "s_waitcnt lgkmcnt(0)"
                        : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(sw[0]), "=&v"(sw[1]),
                          "=&v"(bw[0]), "=&v"(bw[1])
                        : "v"(ac), "v"(as)
                        : "memory");
                    const fm_u4 rr[4] = {r0, r1, r2, r3};
#pragma unroll
                    for (int gi = 0; gi < 4; gi++) {
                        cw[gi][0] = rr[gi].x, cw[gi][1] = rr[gi].y;
                        cw[gi][DW - 2] = rr[gi].z, cw[gi][DW - 1] = rr[gi].w;
                    }
                } else {
                    // a lane's half of a group is 12 bytes, 4-byte aligned: three dword reads per
                    // group.  (Reading the row's whole 96-byte run with 128-bit reads and picking
                    // the half out of the registers costs twice the LDS bytes and a select per
                    // register: 4 us per 512-position chunk.)
                    const uint32_t ac = slot + (uint32_t)(n * (P::RS * 16) + 12 * hh);
                    const uint32_t as = slot + P::LDS_CODE + 8 * n;
                    asm volatile(
                        "ds_read_b32 %0, %16\n\tds_read_b32 %1, %16 offset:4\n\tds_read_b32 %2, %16 offset:8\n\t"
                        "ds_read_b32 %3, %16 offset:24\n\tds_read_b32 %4, %16 offset:28\n\tds_read_b32 %5, %16 offset:32\n\t"
                        "ds_read_b32 %6, %16 offset:48\n\tds_read_b32 %7, %16 offset:52\n\tds_read_b32 %8, %16 offset:56\n\t"
                        "ds_read_b32 %9, %16 offset:72\n\tds_read_b32 %10, %16 offset:76\n\tds_read_b32 %11, %16 offset:80\n\t"
                        "ds_read_b32 %12, %17\n\tds_read_b32 %13, %17 offset:4\n\t"
                        "ds_read_b32 %14, %17 offset:256\n\tds_read_b32 %15, %17 offset:260\n\t"
                        "s_waitcnt lgkmcnt(0)"
                        : "=&v"(cw[0][0]), "=&v"(cw[0][1]), "=&v"(cw[0][2]), "=&v"(cw[1][0]), "=&v"(cw[1][1]),
                          "=&v"(cw[1][2]), "=&v"(cw[2][0]), "=&v"(cw[2][1]), "=&v"(cw[2][2]), "=&v"(cw[3][0]),
                          "=&v"(cw[3][1]), "=&v"(cw[3][2]), "=&v"(sw[0]), "=&v"(sw[1]), "=&v"(bw[0]), "=&v"(bw[1])
                        : "v"(ac), "v"(as)
                        : "memory");
                }
                consumed++;
                c = c + 1 == RING ? 0 : c + 1;
                issue();

                // ---- bias and offset terms, then the groups of the slab
                f16v acc;
#pragma unroll
                for (int i = 0; i < 16; i++) acc[i] = 0.0f;
                uint2 tb, ts;
                const uint4 Bb = pf_side_b<FP16>(bw[0], bw[1], hh, tb);
                const uint4 Bs = pf_side_b<FP16>(sw[0], sw[1], hh, ts);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    __builtin_bit_cast(bf8, make_uint4(sideA[0][0], sideA[0][1], sideA[0][2], sideA[0][3])),
                    __builtin_bit_cast(bf8, Bb), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    __builtin_bit_cast(bf8, make_uint4(sideA[1][0], sideA[1][1], sideA[1][2], sideA[1][3])),
                    __builtin_bit_cast(bf8, Bs), acc, 0, 0, 0);
                if constexpr (FP16) {
                    // tails x piece 1 of both terms: K slots 0..3 biases, 4..7 scales (hh = 0 lanes)
                    const uint4 At = hh ? make_uint4(0u, 0u, 0u, 0u)
                                        : make_uint4(sideA[0][2], sideA[0][3], sideA[1][2], sideA[1][3]);
                    const uint4 Bt = hh ? make_uint4(0u, 0u, 0u, 0u) : make_uint4(tb.x, tb.y, ts.x, ts.y);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, At),
                                                                  __builtin_bit_cast(bf8, Bt), acc, 0, 0, 0);
                }
                // the groups' MFMA chains interleaved (a chain's next MFMA needs the previous
                // one's result: back to back it would idle the matrix core for most of its
                // 8 passes), the scales applied once all four are done
                {
                    uint32_t v[GPW][16];
                    f16v dg[GPW];
#pragma unroll
                    for (int gi = 0; gi < GPW; gi++) {
                        pf_unpack<BITS, 0>(cw[gi], ones, v[gi]);
#pragma unroll
                        for (int i = 0; i < 16; i++) dg[gi][i] = 0.0f;
                    }
#pragma unroll
                    for (int k = 0; k < 4; k++)
#pragma unroll
                        for (int gi = 0; gi < GPW; gi++) {
                            bf8 bop = __builtin_bit_cast(
                                bf8, make_uint4(v[gi][4 * k], v[gi][4 * k + 1], v[gi][4 * k + 2],
                                                v[gi][4 * k + 3]));
                            dg[gi] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                                __builtin_bit_cast(bf8, A[gi][k]), bop, dg[gi], 0, 0, 0);
                        }
#pragma unroll
                    for (int gi = 0; gi < GPW; gi++) {
                        const float sc = (gi & 1) ? fm_widen_hi<FP16>(sw[gi >> 1]) : fm_widen_lo<FP16>(sw[gi >> 1]);
#pragma unroll
                        for (int i = 0; i < 16; i++) acc[i] = fmaf(sc, dg[gi][i], acc[i]);
                    }
                }
                // ---- this wave's partial tile: hi + lo rows, register i of every lane
                {
                    const uint32_t aw = red0 + (uint32_t)(((buf * 2 + mat) * 8 + wave) * 2048 + 4 * lane);
                    float o[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) o[i] = acc[i] + acc[i + 8];
                    asm volatile("ds_write_b32 %0, %1\n\tds_write_b32 %0, %2 offset:256\n\t"
                                 "ds_write_b32 %0, %3 offset:512\n\tds_write_b32 %0, %4 offset:768\n\t"
                                 "ds_write_b32 %0, %5 offset:1024\n\tds_write_b32 %0, %6 offset:1280\n\t"
                                 "ds_write_b32 %0, %7 offset:1536\n\tds_write_b32 %0, %8 offset:1792"
                                 :
                                 : "v"(aw), "v"(o[0]), "v"(o[1]), "v"(o[2]), "v"(o[3]), "v"(o[4]),
                                   "v"(o[5]), "v"(o[6]), "v"(o[7])
                                 : "memory");
                }
            }
            // ---- every wave has written both partial tiles of this step
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            if constexpr (!TEAMS) {
                // wave r sums result register r (position my_pos) over the waves, in wave order
                const uint32_t ar = red0 + (uint32_t)((buf * 2 * 8) * 2048 + wave * 256 + 4 * lane);
                float p[16];
                asm volatile(
                    "ds_read_b32 %0, %16\n\tds_read_b32 %1, %16 offset:2048\n\tds_read_b32 %2, %16 offset:4096\n\t"
                    "ds_read_b32 %3, %16 offset:6144\n\tds_read_b32 %4, %16 offset:8192\n\tds_read_b32 %5, %16 offset:10240\n\t"
                    "ds_read_b32 %6, %16 offset:12288\n\tds_read_b32 %7, %16 offset:14336\n\t"
                    "ds_read_b32 %8, %16 offset:16384\n\tds_read_b32 %9, %16 offset:18432\n\tds_read_b32 %10, %16 offset:20480\n\t"
                    "ds_read_b32 %11, %16 offset:22528\n\tds_read_b32 %12, %16 offset:24576\n\tds_read_b32 %13, %16 offset:26624\n\t"
                    "ds_read_b32 %14, %16 offset:28672\n\tds_read_b32 %15, %16 offset:30720\n\t"
                    "s_waitcnt lgkmcnt(0)"
                    : "=&v"(p[0]), "=&v"(p[1]), "=&v"(p[2]), "=&v"(p[3]), "=&v"(p[4]), "=&v"(p[5]),
                      "=&v"(p[6]), "=&v"(p[7]), "=&v"(p[8]), "=&v"(p[9]), "=&v"(p[10]), "=&v"(p[11]),
                      "=&v"(p[12]), "=&v"(p[13]), "=&v"(p[14]), "=&v"(p[15])
                    : "v"(ar)
                    : "memory");
                float t0 = p[0], t1 = p[8];
#pragma unroll
                for (int w2 = 1; w2 < 8; w2++) {
                    t0 += p[w2];
                    t1 += p[8 + w2];
                }
                // the two row tiles of the step; later column passes add to the earlier ones
                if (my_on) {
                    float *o = a.d_out + (size_t)(item.start + my_pos) * a.d_rows + 64 * s + n;
                    const bool add = a.d_pass > 0 || (a.d_flags & FM_ACCUMULATE);
                    o[0] = add ? o[0] + t0 : t0;
                    o[32] = add ? o[32] + t1 : t1;
                }
            } else {
                // wave (team, j) sums tile j of its team over the team's two waves (slab 0, then
                // slab 1): all eight registers = the eight positions this lane stores
                const int j = wave & 1;
                const uint32_t ar = red0 + (uint32_t)(((buf * 2 + j) * 8 + 2 * team) * 2048 + 4 * lane);
                float p[16];
                asm volatile(
                    "ds_read_b32 %0, %16\n\tds_read_b32 %1, %16 offset:256\n\tds_read_b32 %2, %16 offset:512\n\t"
                    "ds_read_b32 %3, %16 offset:768\n\tds_read_b32 %4, %16 offset:1024\n\tds_read_b32 %5, %16 offset:1280\n\t"
                    "ds_read_b32 %6, %16 offset:1536\n\tds_read_b32 %7, %16 offset:1792\n\t"
                    "ds_read_b32 %8, %16 offset:2048\n\tds_read_b32 %9, %16 offset:2304\n\tds_read_b32 %10, %16 offset:2560\n\t"
                    "ds_read_b32 %11, %16 offset:2816\n\tds_read_b32 %12, %16 offset:3072\n\tds_read_b32 %13, %16 offset:3328\n\t"
                    "ds_read_b32 %14, %16 offset:3584\n\tds_read_b32 %15, %16 offset:3840\n\t"
                    "s_waitcnt lgkmcnt(0)"
                    : "=&v"(p[0]), "=&v"(p[1]), "=&v"(p[2]), "=&v"(p[3]), "=&v"(p[4]), "=&v"(p[5]),
                      "=&v"(p[6]), "=&v"(p[7]), "=&v"(p[8]), "=&v"(p[9]), "=&v"(p[10]), "=&v"(p[11]),
                      "=&v"(p[12]), "=&v"(p[13]), "=&v"(p[14]), "=&v"(p[15])
                    : "v"(ar)
                    : "memory");
                const int row = 256 * s + 64 * team + 32 * j + n;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const int tok = 8 * (i / 4) + 4 * hh + (i % 4);
                    if (tok < item.count) {
                        const float v = p[i] + p[8 + i];
                        float *o = a.d_out + (size_t)(item.start + tok) * a.d_rows + row;
                        *o = (a.d_flags & FM_ACCUMULATE) ? *o + v : v;
                    }
                }
            }
            buf ^= 1;
        }
    }
#else
    (void)a;
#endif
}

// out[m][j] = sum_k w[m][k] * eo[m*K + k][j] in slot order (finchmoe/shaders.metal:2764-2802)
__global__ __launch_bounds__(256) void fm_pf_combine(PfArgs a, float *out, int flags) {
    const int m = blockIdx.x, H = a.g.hidden, K = a.K;
    float wk[FM_MAX_K];
#pragma unroll
    for (int k = 0; k < FM_MAX_K; k++) {
        float w = 0.0f;
        if (k < K) {
            w = a.w[m * K + k];
            if ((unsigned)a.idx[m * K + k] >= (unsigned)a.g.n_experts) w = 0.0f;
        }
        wk[k] = w;
    }
    // four columns per thread (hidden is a multiple of 4)
    const float4 *eo = reinterpret_cast<const float4 *>(a.eo + (size_t)m * K * H);
    float4 *o4 = reinterpret_cast<float4 *>(out + (size_t)m * H);
    const int H4 = H / 4;
    for (int j = blockIdx.y * blockDim.x + threadIdx.x; j < H4; j += gridDim.y * blockDim.x) {
        float4 v[FM_MAX_K];
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            if (k < K && wk[k] != 0.0f) v[k] = eo[(size_t)k * H4 + j];
        float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            if (k < K && wk[k] != 0.0f) {
                acc.x += wk[k] * v[k].x;
                acc.y += wk[k] * v[k].y;
                acc.z += wk[k] * v[k].z;
                acc.w += wk[k] * v[k].w;
            }
        if (flags & FM_ACCUMULATE) {
            const float4 p = o4[j];
            acc.x += p.x, acc.y += p.y, acc.z += p.z, acc.w += p.w;
        }
        o4[j] = acc;
    }
}

// dense product: workgroup 0 cuts the M positions into items of PF_TM, the others prepare X
template <int BITS>
__global__ __launch_bounds__(1024) void fm_pf_dense_prep(PfArgs a) {
    if (blockIdx.x > 0) {
        pf_prepare<BITS>(a.X, a.M, a.d_cols, a.xop, a.xsums, (int)((blockIdx.x - 1) * blockDim.x + threadIdx.x));
        return;
    }
    const int n = (a.M + PF_TM - 1) / PF_TM;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        PfItem it;
        it.expert = 0;
        it.start = i * PF_TM;
        it.count = a.M - i * PF_TM < PF_TM ? a.M - i * PF_TM : PF_TM;
        it.pad = 0;
        a.items[i] = it;
    }
    if (threadIdx.x == 0) *a.n_items = n;
}

// ======================================================================
// Row-tile kernels (fm_pf_rows): the expert products of a chunk.
//
// A wave owns 32 weight rows over the WHOLE K dimension, so a row tile is summed
// inside one accumulator and nothing is exchanged between waves: no partial tiles
// in LDS, no barrier per step.  What the waves of a workgroup share instead is the
// activation operand of the current item, kept in LDS in MFMA register form (the
// "image"), staged once per item.
//
//   item       (expert, up to 16 of its positions; 8 when the gate/up activations
//              arrive as fp32: two bf16 pieces per value, in two M rows)
//   task       32 weight rows of an item against all its positions: gate/up = 16
//              gate rows + the same 16 up rows (SwiGLU needs both, and they meet in
//              one lane), down = 32 rows
//   slab       256 columns (four quantization groups) of a task's rows = one ring
//              slot of 32 x 96 (128) code bytes, copied with LDS-direct loads; a task
//              is 8 (gate/up) or 2 (down) slabs
//   round      8 consecutive tasks of an item, one per wave; a workgroup takes a
//              contiguous run of rounds of the chunk (every workgroup the same number
//              within one), so every wave streams the same number of bytes and the
//              waves meet again exactly where the item — the image — changes
//
// MFMA geometry.  V_MFMA_F32_16X16X32_BF16: positions on M (16), weight rows on N
// (16: the task's rows are two N tiles), one product covers half a quantization
// group (32 columns).  Lane (n, kb) holds, of weight row n, the 16 codes 16 kb ..
// 16 kb + 15 of each group — 6 bytes (8 for 4-bit codes) — and supplies k slots
// 8 kb .. 8 kb + 7 of both products of the group; codes c and c + 4 share a register
// as bf16 values 1 + q * 2^t / 128 (fm_mfma.h; 3-bit: t = 4 and 0, one mask for all
// pairs).  Each (tile, group) has its own accumulator of four registers and gets its
// scale in fp32.  fp32 activations are two bf16 pieces: along K (two products on one
// accumulator: the down product), or in M rows p and p + 8 (gate/up on fp32 X; the two
// halves of the result are added at the end).  Bias and offset terms of a slab's four
// groups are one more product per tile whose 32 k slots are (term, piece, group).
//
// What bounds these kernels is the number of cache-line requests of the LDS-direct
// loads, not their bytes: a slab is 32 runs of 96 bytes, 768 bytes apart.  Measured on
// the 512-position benchmark chunk (gate/up kernel): 101 us with the slab's scales and
// biases fetched per slot (8 bytes per row, 64 bytes apart: as many line requests as
// the codes), 82 us without them, 73 us with no loads at all — while taking out the
// unpack arithmetic, the products or the image reads changes nothing.  Hence gate/up
// keeps a task's scales and biases in registers, fetched as four contiguous KB.
// ======================================================================
enum { PFR_GATE_UP = 0, PFR_DOWN = 1 };

template <int MODE, int BITS, int QK>
struct PfRows {
    static constexpr int S = MODE == PFR_GATE_UP ? 8 : 2;          // slabs of a task (K / 256)
    static constexpr int CB = 8 * BITS * 4;                        // code bytes of a row inside a slab
    static constexpr int RP = CB / 16;                             // 16-byte pieces per row
    static constexpr int NQ = 32 * RP / 64;                        // LDS-direct loads for the codes
    static constexpr int CODE = 32 * CB;
    // gate/up keeps the scales and biases of a task in registers (SREG): its rows have 32
    // groups, so a slab's 8 bytes per row are 64 bytes apart; a task's 16 rows x 64 bytes are
    // one contiguous KB instead.  down (8 groups per row) fetches them with every slot.
    static constexpr bool SREG = MODE == PFR_GATE_UP;
    static constexpr int SLOT = CODE + (SREG ? 0 : 512);           // + scales 256 + biases 256
    static constexpr int LOADS = NQ + (SREG ? 0 : 2);
    static constexpr int OPB = 1024;                               // one operand of the image: 64 lanes x 16 B
    static constexpr int SLAB_IMG = 4 * 2 * QK * OPB;              // [group][k step][piece]
    static constexpr int IMG = S * SLAB_IMG;
    static constexpr int SIDE = S * OPB;
    static constexpr int RING_ROOM = (160 * 1024 - 2048 - IMG - SIDE) / (8 * SLOT);
    static constexpr int RING = RING_ROOM > 4 ? 4 : RING_ROOM;
    static constexpr int LDS_BYTES = 8 * RING * SLOT + IMG + SIDE;
    static_assert(RING >= 2, "a ring needs a slot in flight beside the one being multiplied");
    static_assert(IMG <= 65536, "image offsets are 16-bit immediates");
};

// mantissa positions of the two codes of a pair (low / high half of the register) and the
// power of two each position costs the activation
template <int BITS> struct PfrPair;
template <> struct PfrPair<3> {
    static constexpr uint32_t MASK = (7u << 4) | (7u << 16);
    static constexpr float FL = 8.0f, FH = 128.0f;
};
template <> struct PfrPair<4> {
    static constexpr uint32_t MASK = 0x000F000Fu;
    static constexpr float FL = 128.0f, FH = 128.0f;
};

// One k step of a group of 64 activations as operand registers: register i holds columns
// c0 + i (low half) and c0 + i + 4 (high half), scaled; hi (and, TWO, lo) bf16 piece.
// xs / xo collect what the bias and offset terms multiply.
template <int BITS, bool TWO>
__device__ __forceinline__ void pfr_stage_op(const float *x, int c0, uint4 &hi, uint4 &lo, float &xs, float &xo) {
    uint32_t h[4], l[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        constexpr float cl = PfrPair<BITS>::FL, ch = PfrPair<BITS>::FH;
        const float vl = x[c0 + i] * cl, vh = x[c0 + i + 4] * ch;
        const uint32_t l0 = __float_as_uint(vl) & 0xFFFF0000u, h0 = __float_as_uint(vh) & 0xFFFF0000u;
        h[i] = (l0 >> 16) | h0;
        float tl = __uint_as_float(l0), th = __uint_as_float(h0);
        l[i] = 0u;
        if constexpr (TWO) {
            const float rl = vl - tl, rh = vh - th;
            const uint32_t l1 = __float_as_uint(rl) & 0xFFFF0000u, h1 = __float_as_uint(rh) & 0xFFFF0000u;
            l[i] = (l1 >> 16) | h1;
            tl += __uint_as_float(l1);
            th += __uint_as_float(h1);
        }
        xo += tl + th;
        xs += tl * (1.0f / cl) + th * (1.0f / ch);
    }
    hi = make_uint4(h[0], h[1], h[2], h[3]);
    lo = make_uint4(l[0], l[1], l[2], l[3]);
}

// 64 consecutive activations of one position as floats: bf16 bits or fp32
template <bool XBF16>
__device__ __forceinline__ void pfr_load64(const void *row, int col0, bool on, float *x) {
    if constexpr (XBF16) {
        const uint4 *p = reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(row) + col0);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint4 v = on ? p[i] : make_uint4(0u, 0u, 0u, 0u);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                x[8 * i + 2 * k] = __uint_as_float(w[k] << 16);
                x[8 * i + 2 * k + 1] = __uint_as_float(w[k] & 0xFFFF0000u);
            }
        }
    } else {
        const float4 *p = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(row) + col0);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float4 v = on ? p[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
        }
    }
}

// a dword of two 16-bit scales (biases) as MFMA operand halves: BF16 bits are operands as
// they are; an FP16 value (11 significant bits) is split exactly into a bf16 head and tail
template <bool FP16>
__device__ __forceinline__ void pfr_head_tail(uint32_t w, uint32_t &head, uint32_t &tail) {
    if constexpr (!FP16) {
        head = w;
        tail = 0u;
    } else {
        const float f0 = fm_fp16_bits(w & 0xFFFFu), f1 = fm_fp16_bits(w >> 16);
        const uint32_t h0 = __float_as_uint(f0) & 0xFFFF0000u, h1 = __float_as_uint(f1) & 0xFFFF0000u;
        const uint32_t t0 = __float_as_uint(f0 - __uint_as_float(h0)), t1 = __float_as_uint(f1 - __uint_as_float(h1));
        head = (h0 >> 16) | h1;
        tail = (t0 >> 16) | (t1 & 0xFFFF0000u);
    }
}

typedef uint32_t pfr_u4 __attribute__((ext_vector_type(4)));
typedef float pfr_f4 __attribute__((ext_vector_type(4)));

// XBF16: gate/up reads X as bf16 bits; otherwise fp32 activations: gate/up puts their two
// pieces in M rows p / p + 8 (8 positions per item), down along K (QK = 2)
template <int MODE, int BITS, bool FP16, bool XBF16>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void fm_pf_rows(PfArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr bool GU = MODE == PFR_GATE_UP;
    constexpr int QK = GU ? 1 : 2;
    constexpr bool ROWP = GU && !XBF16;                 // the two pieces in M rows
    constexpr int TM = ROWP ? 8 : 16;
    using P = PfRows<MODE, BITS, QK>;
    constexpr int S = P::S, RING = P::RING;
    extern __shared__ __attribute__((aligned(16))) uint8_t pfr_smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = lane & 15, kb = lane >> 4;
    const uint32_t lds0 = fm_lds_addr(pfr_smem);
    const uint32_t ring0 = lds0 + (uint32_t)wave * (RING * P::SLOT);
    uint8_t *img_mem = pfr_smem + 8 * RING * P::SLOT;
    uint8_t *side_mem = img_mem + P::IMG;
    const uint32_t img0 = lds0 + 8 * RING * P::SLOT, side0 = img0 + P::IMG;
    const int in_dim = GU ? a.g.hidden : a.g.inter, out_rows = GU ? a.g.inter : a.g.hidden;
    const int row_bytes = in_dim * BITS / 8, sb_bytes = (in_dim / 64) * 2;
    const PfItem *items = GU ? a.items_up : a.items_dn;
    const int n_items = *(GU ? a.n_items_up : a.n_items_dn);
    const int RPI = out_rows / (GU ? 16 : 32) / 8;      // rounds per item
    const uint32_t ones = fm_opaque(0x3F803F80u);

    // ---- this workgroup's rounds [R0, R1).  Workgroups are dealt out to the eight XCDs in
    // turn and every XCD has an L2 of its own: workgroup b takes share (b % 8) * (grid / 8) +
    // b / 8, so that neighbouring shares — the rounds of one expert — run behind one L2.
    const long RT = (long)n_items * RPI;
    const FmRange rounds = fm_pfr_rounds(RT, blockIdx.x, gridDim.x);
    const int R0 = (int)rounds.lo, R1 = (int)rounds.hi;
    if (R0 >= R1) return;
    const int it0 = R0 / RPI;
    // the items the share touches, one per lane (the launcher sizes the grid so that a share
    // spans at most 64 items): expert, first sorted position, number of positions
    const int it_last = (R1 - 1) / RPI;
    int ev = 0, ev_start = 0, ev_count = 0;
    if (it0 + lane <= it_last) {
        const PfItem d = items[it0 + lane];
        ev = d.expert, ev_start = d.start, ev_count = d.count;
    }
    // What staging an item needs from memory besides the activations themselves is fetched one
    // item ahead: this thread's staging task is (group st_g, position st_pos), and st_pair is
    // the pair id of that position (gate/up: its row of X is st_pair / K; down: threads 0-15
    // publish the ids for the output addresses).
    constexpr int NG = S * 4;
    const int st_pos = threadIdx.x % TM, st_g = threadIdx.x / TM;
    const bool st_has = threadIdx.x < TM * NG;
    __shared__ int pairs_tab[16];
    int st_pair = 0;
    if (st_has && st_pos < __builtin_amdgcn_readlane(ev_count, 0))
        st_pair = a.sorted[__builtin_amdgcn_readlane(ev_start, 0) + st_pos];

    // ---- this lane's pieces of a slot copy
    // codes: piece q = 64 j + lane of the slot = 16 bytes of row q / RP (the slot keeps the
    // rows back to back).  gate/up: slot rows 0-15 = gate rows, 16-31 = the same rows of up
    uint32_t coff[P::NQ];
#pragma unroll
    for (int j = 0; j < P::NQ; j++)
        coff[j] = fm_pfr_piece_off(GU, BITS, 64 * j + lane, GU ? a.g.gate_w : a.g.down_w, a.g.up_w, row_bytes);
    // scales / biases fetched with the slot (down): 8 bytes per row and slab, one dword per lane
    const uint32_t soff = fm_pfr_sb_off(GU, lane, GU ? a.g.gate_s : a.g.down_s, a.g.up_s, sb_bytes);
    const uint32_t boff = fm_pfr_sb_off(GU, lane, GU ? a.g.gate_b : a.g.down_b, a.g.up_b, sb_bytes);

    // ---- loader: the slabs of this wave's tasks, in order
    int l_r = R0, l_s = 0, wpos = 0;
    uint32_t issued = 0, consumed = 0;
    const uint8_t *l_w = nullptr, *l_sb = nullptr;
    // SREG: scales and biases of the task the loader has entered, requested with four loads of
    // one contiguous KB each — lane (n, kb) gets the 16 bytes (eight groups) 16 kb of its rows —
    // in front of the task's first slot: once that slot has landed, so have they.  They land in
    // v[240:255], which the statements name themselves: a value that is still in flight must
    // never sit in a register the compiler allocates, because the compiler may move such a
    // value to another register (at a loop's back edge, say) before the wait that makes it
    // valid.  The kernel's own values stay far below v240 (the allocator fills registers from
    // v0 upwards; a host test reads the compiled kernel and checks that nothing else names
    // these sixteen).  csc: the landed copy of the task being multiplied, [tile 0 s, tile 0 b,
    // tile 1 s, tile 1 b], taken behind that wait.
    pfr_u4 csc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) csc[i] = pfr_u4{0u, 0u, 0u, 0u};
    const uint32_t sc_lane = (uint32_t)(n * sb_bytes + 16 * kb);
    int sc_round = R0;            // the round whose scales were requested last
    auto loader_enter = [&]() __attribute__((always_inline)) {
        const int it = l_r / RPI, t = (l_r - it * RPI) * 8 + wave;
        const int e = __builtin_amdgcn_readlane(ev, it - it0);
        const uint8_t *blob = a.layer + (size_t)e * a.g.expert_size;
        const size_t r0 = (size_t)t * (GU ? 16 : 32);
        l_w = fm_uniform(blob + r0 * row_bytes);
        l_sb = fm_uniform(blob + r0 * sb_bytes);
        if constexpr (P::SREG) {
            const uint8_t *p0 = l_sb + a.g.gate_s, *p1 = l_sb + a.g.gate_b, *p2 = l_sb + a.g.up_s, *p3 = l_sb + a.g.up_b;
            asm volatile("global_load_dwordx4 v[240:243], %0, %1\n\tglobal_load_dwordx4 v[244:247], %0, %2\n\t"
                         "global_load_dwordx4 v[248:251], %0, %3\n\tglobal_load_dwordx4 v[252:255], %0, %4"
                         :
                         : "v"(sc_lane), "s"(p0), "s"(p1), "s"(p2), "s"(p3)
                         : "memory", "v240", "v241", "v242", "v243", "v244", "v245", "v246", "v247", "v248", "v249",
                           "v250", "v251", "v252", "v253", "v254", "v255");
            sc_round = l_r;
        }
    };
    loader_enter();
    auto issue = [&]() __attribute__((always_inline)) {
        if (l_r >= R1) return;
        const uint32_t slot = ring0 + (uint32_t)wpos * P::SLOT;
        const uint8_t *wb = l_w + (size_t)l_s * P::CB, *sb = l_sb + (size_t)l_s * 8;
#pragma unroll
        for (int j = 0; j < P::NQ; j++)
            __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(wb + coff[j]),
                                             (fm_lptr)(uintptr_t)(slot + 1024 * j), 16, 0, 0);
        if constexpr (!P::SREG) {
            __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(sb + soff),
                                             (fm_lptr)(uintptr_t)(slot + P::CODE), 4, 0, 0);
            __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(sb + boff),
                                             (fm_lptr)(uintptr_t)(slot + P::CODE + 256), 4, 0, 0);
        }
        wpos = wpos + 1 == RING ? 0 : wpos + 1;
        issued++;
        if (++l_s == S) {
            l_s = 0;
            if (++l_r < R1) loader_enter();
        }
    };
#pragma unroll
    for (int k = 0; k < RING; k++) issue();

    // ---- addresses of this lane inside a slot, the image and the side operands
    // 3-bit: its 6 bytes of a (row, group) are read as the two aligned dwords around them
    // and shifted down by 16 bits in the odd lanes
    const uint32_t code_lane = BITS == 3 ? (uint32_t)(n * P::CB + 12 * (kb >> 1) + 4 * (kb & 1))
                                         : (uint32_t)(n * P::CB + 8 * kb);
    const uint32_t sh3 = 16u * (uint32_t)(kb & 1);
    const uint32_t img_lane = img0 + 16u * (uint32_t)lane, side_lane = side0 + 16u * (uint32_t)lane;
    // rows 8-15 of the side operands stay zero when the pieces sit in M rows
    if constexpr (ROWP)
        for (int i = threadIdx.x; i < P::SIDE / 16; i += blockDim.x)
            reinterpret_cast<uint4 *>(side_mem)[i] = make_uint4(0u, 0u, 0u, 0u);

    // block BLK of a slab's image operands (eight of them, in [group][k step][piece] order)
    auto img_read = [&](uint32_t addr, pfr_u4 *buf, auto blk) __attribute__((always_inline)) {
        constexpr int O = decltype(blk)::value * 8 * P::OPB;
        asm volatile(
            "ds_read_b128 %0, %8 offset:%9\n\tds_read_b128 %1, %8 offset:%10\n\t"
            "ds_read_b128 %2, %8 offset:%11\n\tds_read_b128 %3, %8 offset:%12\n\t"
            "ds_read_b128 %4, %8 offset:%13\n\tds_read_b128 %5, %8 offset:%14\n\t"
            "ds_read_b128 %6, %8 offset:%15\n\tds_read_b128 %7, %8 offset:%16"
            : "=&v"(buf[0]), "=&v"(buf[1]), "=&v"(buf[2]), "=&v"(buf[3]), "=&v"(buf[4]), "=&v"(buf[5]),
              "=&v"(buf[6]), "=&v"(buf[7])
            : "v"(addr), "n"(O), "n"(O + P::OPB), "n"(O + 2 * P::OPB), "n"(O + 3 * P::OPB),
              "n"(O + 4 * P::OPB), "n"(O + 5 * P::OPB), "n"(O + 6 * P::OPB), "n"(O + 7 * P::OPB)
            : "memory");
    };
    auto lgkm_wait = [&](pfr_u4 *buf) __attribute__((always_inline)) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(buf[0]), "+v"(buf[1]), "+v"(buf[2]), "+v"(buf[3]), "+v"(buf[4]), "+v"(buf[5]),
                       "+v"(buf[6]), "+v"(buf[7])
                     :
                     : "memory");
    };

    int c = 0, cur_item = -1;
    PfItem item = PfItem{0, 0, 0, 0};
    uint32_t oidx[4];                  // output element offset of result register i, ~0u = no store
#pragma unroll
    for (int i = 0; i < 4; i++) oidx[i] = ~0u;

    for (int r = R0; r < R1; r++) {
        const int it = r / RPI;
        if (it != cur_item) {
            // ---- the workgroup moves to another item: stage its activations
            cur_item = it;
            item.expert = __builtin_amdgcn_readlane(ev, it - it0);
            item.start = __builtin_amdgcn_readlane(ev_start, it - it0);
            item.count = __builtin_amdgcn_readlane(ev_count, it - it0);
            // the activations are requested before the barrier: their addresses are known
            const bool on = st_has && st_pos < item.count;
            const size_t m = !on ? 0 : GU ? (size_t)(st_pair / a.K) : (size_t)(item.start + st_pos);
            float x[64];
            if constexpr (GU && XBF16) pfr_load64<true>(a.Xbf + m * in_dim, 64 * st_g, on, x);
            else pfr_load64<false>((GU ? a.X : a.act) + m * in_dim, 64 * st_g, on, x);
            const int my_pair = st_pair;
            // (and the next item's pair ids behind them)
            st_pair = 0;
            if (it < it_last && st_has && st_pos < __builtin_amdgcn_readlane(ev_count, it + 1 - it0))
                st_pair = a.sorted[__builtin_amdgcn_readlane(ev_start, it + 1 - it0) + st_pos];
            __syncthreads();                                   // every wave is done with the old image
            if (st_has) {
                // task = (group, position), positions fastest: a wave covers whole slabs
                const int sl = st_g >> 2, gi = st_g & 3;
                uint8_t *dst = img_mem + (size_t)sl * P::SLAB_IMG + (size_t)gi * 2 * QK * P::OPB + 16 * st_pos;
                float xs = 0.0f, xo = 0.0f;
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        uint4 hi, lo;
                        pfr_stage_op<BITS, !XBF16 || !GU>(x, 16 * k + 8 * j, hi, lo, xs, xo);
                        uint8_t *d = dst + (size_t)j * QK * P::OPB + 256 * k;       // lane 16 k + position
                        *reinterpret_cast<uint4 *>(d) = hi;
                        if constexpr (QK == 2) *reinterpret_cast<uint4 *>(d + P::OPB) = lo;
                        if constexpr (ROWP) *reinterpret_cast<uint4 *>(d + 16 * 8) = lo;       // M row 8 + position
                    }
                // bias / offset operands of (slab, position): the four groups' sums sit in the
                // lanes TM apart; the lane of group gi builds the operand of k block gi: piece gi
                // (k block 3: piece 0 once more, against the tails of FP16 scales) of
                // (xsum g0 g1, xsum g2 g3, -xoff g0 g1, -xoff g2 g3)
                uint32_t pc[8][3];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int from = lane + (k - gi) * TM;
                    pf_pieces(__shfl(xs, from), pc[k]);
                    pf_pieces(-__shfl(xo, from), pc[4 + k]);
                }
                const int pi = gi < 3 ? gi : 0;
                uint32_t sel[8];
#pragma unroll
                for (int k = 0; k < 8; k++) sel[k] = pi == 0 ? pc[k][0] : pi == 1 ? pc[k][1] : pc[k][2];
                const uint4 sv = make_uint4(sel[0] | (sel[1] << 16), sel[2] | (sel[3] << 16),
                                            sel[4] | (sel[5] << 16), sel[6] | (sel[7] << 16));
                *reinterpret_cast<uint4 *>(side_mem + (size_t)sl * P::OPB + 16 * (16 * gi + st_pos)) = sv;
                if (!GU && st_g == 0) pairs_tab[st_pos] = my_pair;
            }
            __syncthreads();                                   // the image is complete
            // where this lane's results go: register i = position 4 * (lane / 16) + i
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int tok = (ROWP ? 4 * (kb & 1) : 4 * kb) + i;
                oidx[i] = ~0u;
                if (tok < item.count)
                    oidx[i] = GU ? (uint32_t)(item.start + tok) * (uint32_t)a.g.inter
                                 : (uint32_t)pairs_tab[tok] * (uint32_t)a.g.hidden;
            }
        }
        const int t = (r - it * RPI) * 8 + wave;               // this wave's task of the round

        pfr_f4 acc[2], side[2];
#pragma unroll
        for (int T = 0; T < 2; T++) acc[T] = pfr_f4{0.0f, 0.0f, 0.0f, 0.0f}, side[T] = pfr_f4{0.0f, 0.0f, 0.0f, 0.0f};

        for (int s = 0; s < S; s++) {
            const uint32_t ia = img_lane + (uint32_t)s * P::SLAB_IMG;
            // image operands and the bias/offset operand: they depend on nothing
            pfr_u4 abuf[QK][8], sA;
            img_read(ia, abuf[0], std::integral_constant<int, 0>());
            {
                const uint32_t sa = side_lane + (uint32_t)s * P::OPB;
                asm volatile("ds_read_b128 %0, %1" : "=&v"(sA) : "v"(sa) : "memory");
            }
            if constexpr (QK == 2) img_read(ia, abuf[1], std::integral_constant<int, 1>());
            // ---- the oldest slot of the ring.  SREG: once the loader has entered the next task,
            // that task's four scale loads are in flight too, behind every slot of this one
            if (issued - consumed != (uint32_t)RING) fm_dma_wait<0>(true);
            else if (P::SREG && sc_round > r) fm_dma_wait<P::LOADS *(RING - 1) + 4>(false);
            else fm_dma_wait<P::LOADS *(RING - 1)>(false);
            const uint32_t slot = ring0 + (uint32_t)c * P::SLOT;
            uint32_t d0[2][4], d1[2][4], sw[2][2], bw[2][2];     // [tile][group] codes, [tile][dword] scales
            const uint32_t a0 = slot + code_lane, a1 = a0 + 16 * P::CB;
            uint2 q[2][4];
            if constexpr (P::SREG) {
                if (s == 0) {          // the task's first slot is there, and so are its scales
                    uint32_t t[16];
                    asm volatile("v_mov_b32 %0, v240\n\tv_mov_b32 %1, v241\n\t"
                                 "v_mov_b32 %2, v242\n\tv_mov_b32 %3, v243\n\t"
                                 "v_mov_b32 %4, v244\n\tv_mov_b32 %5, v245\n\t"
                                 "v_mov_b32 %6, v246\n\tv_mov_b32 %7, v247\n\t"
                                 "v_mov_b32 %8, v248\n\tv_mov_b32 %9, v249\n\t"
                                 "v_mov_b32 %10, v250\n\tv_mov_b32 %11, v251\n\t"
                                 "v_mov_b32 %12, v252\n\tv_mov_b32 %13, v253\n\t"
                                 "v_mov_b32 %14, v254\n\tv_mov_b32 %15, v255"
                                 : "=v"(t[0]), "=v"(t[1]), "=v"(t[2]), "=v"(t[3]), "=v"(t[4]), "=v"(t[5]), "=v"(t[6]),
                                   "=v"(t[7]), "=v"(t[8]), "=v"(t[9]), "=v"(t[10]), "=v"(t[11]), "=v"(t[12]),
                                   "=v"(t[13]), "=v"(t[14]), "=v"(t[15])
                                 :
                                 : "memory");
#pragma unroll
                    for (int i = 0; i < 4; i++) csc[i] = pfr_u4{t[4 * i], t[4 * i + 1], t[4 * i + 2], t[4 * i + 3]};
                }
                // the slab's four groups are one dword pair of the lanes kb = s / 2
                const uint32_t src = 4u * (uint32_t)(n + 16 * (s >> 1));
                const bool hi = s & 1;
                uint32_t v[8], o[8];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    v[2 * i] = hi ? csc[i][2] : csc[i][0];
                    v[2 * i + 1] = hi ? csc[i][3] : csc[i][1];
                }
                asm volatile("ds_bpermute_b32 %0, %8, %9\n\tds_bpermute_b32 %1, %8, %10\n\t"
                             "ds_bpermute_b32 %2, %8, %11\n\tds_bpermute_b32 %3, %8, %12\n\t"
                             "ds_bpermute_b32 %4, %8, %13\n\tds_bpermute_b32 %5, %8, %14\n\t"
                             "ds_bpermute_b32 %6, %8, %15\n\tds_bpermute_b32 %7, %8, %16"
                             : "=&v"(o[0]), "=&v"(o[1]), "=&v"(o[2]), "=&v"(o[3]), "=&v"(o[4]), "=&v"(o[5]),
                               "=&v"(o[6]), "=&v"(o[7])
                             : "v"(src), "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]),
                               "v"(v[7])
                             : "memory");
                if constexpr (BITS == 3) {
                    asm volatile(
                        "ds_read2_b32 %0, %8 offset0:0 offset1:1\n\tds_read2_b32 %1, %8 offset0:6 offset1:7\n\t"
                        "ds_read2_b32 %2, %8 offset0:12 offset1:13\n\tds_read2_b32 %3, %8 offset0:18 offset1:19\n\t"
                        "ds_read2_b32 %4, %9 offset0:0 offset1:1\n\tds_read2_b32 %5, %9 offset0:6 offset1:7\n\t"
                        "ds_read2_b32 %6, %9 offset0:12 offset1:13\n\tds_read2_b32 %7, %9 offset0:18 offset1:19\n\t"
                        "s_waitcnt lgkmcnt(0)"
                        : "=&v"(q[0][0]), "=&v"(q[0][1]), "=&v"(q[0][2]), "=&v"(q[0][3]), "=&v"(q[1][0]), "=&v"(q[1][1]),
                          "=&v"(q[1][2]), "=&v"(q[1][3])
                        : "v"(a0), "v"(a1)
                        : "memory");
                } else {
                    asm volatile(
                        "ds_read_b64 %0, %8\n\tds_read_b64 %1, %8 offset:32\n\t"
                        "ds_read_b64 %2, %8 offset:64\n\tds_read_b64 %3, %8 offset:96\n\t"
                        "ds_read_b64 %4, %9\n\tds_read_b64 %5, %9 offset:32\n\t"
                        "ds_read_b64 %6, %9 offset:64\n\tds_read_b64 %7, %9 offset:96\n\t"
                        "s_waitcnt lgkmcnt(0)"
                        : "=&v"(q[0][0]), "=&v"(q[0][1]), "=&v"(q[0][2]), "=&v"(q[0][3]), "=&v"(q[1][0]), "=&v"(q[1][1]),
                          "=&v"(q[1][2]), "=&v"(q[1][3])
                        : "v"(a0), "v"(a1)
                        : "memory");
                }
                asm volatile("" : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]), "+v"(o[4]), "+v"(o[5]), "+v"(o[6]),
                             "+v"(o[7]));
#pragma unroll
                for (int T = 0; T < 2; T++)
                    sw[T][0] = o[4 * T], sw[T][1] = o[4 * T + 1], bw[T][0] = o[4 * T + 2], bw[T][1] = o[4 * T + 3];
            } else {
                const uint32_t as = slot + P::CODE + 8 * n;
                uint2 sq[2], bq[2];
                if constexpr (BITS == 3) {
                    asm volatile(
                        "ds_read2_b32 %0, %12 offset0:0 offset1:1\n\tds_read2_b32 %1, %12 offset0:6 offset1:7\n\t"
                        "ds_read2_b32 %2, %12 offset0:12 offset1:13\n\tds_read2_b32 %3, %12 offset0:18 offset1:19\n\t"
                        "ds_read2_b32 %4, %13 offset0:0 offset1:1\n\tds_read2_b32 %5, %13 offset0:6 offset1:7\n\t"
                        "ds_read2_b32 %6, %13 offset0:12 offset1:13\n\tds_read2_b32 %7, %13 offset0:18 offset1:19\n\t"
                        "ds_read_b64 %8, %14\n\tds_read_b64 %9, %14 offset:128\n\t"
                        "ds_read_b64 %10, %14 offset:256\n\tds_read_b64 %11, %14 offset:384\n\t"
                        "s_waitcnt lgkmcnt(0)"
                        : "=&v"(q[0][0]), "=&v"(q[0][1]), "=&v"(q[0][2]), "=&v"(q[0][3]), "=&v"(q[1][0]), "=&v"(q[1][1]),
                          "=&v"(q[1][2]), "=&v"(q[1][3]), "=&v"(sq[0]), "=&v"(sq[1]), "=&v"(bq[0]), "=&v"(bq[1])
                        : "v"(a0), "v"(a1), "v"(as)
                        : "memory");
                } else {
                    asm volatile(
                        "ds_read_b64 %0, %12\n\tds_read_b64 %1, %12 offset:32\n\t"
                        "ds_read_b64 %2, %12 offset:64\n\tds_read_b64 %3, %12 offset:96\n\t"
                        "ds_read_b64 %4, %13\n\tds_read_b64 %5, %13 offset:32\n\t"
                        "ds_read_b64 %6, %13 offset:64\n\tds_read_b64 %7, %13 offset:96\n\t"
                        "ds_read_b64 %8, %14\n\tds_read_b64 %9, %14 offset:128\n\t"
                        "ds_read_b64 %10, %14 offset:256\n\tds_read_b64 %11, %14 offset:384\n\t"
                        "s_waitcnt lgkmcnt(0)"
                        : "=&v"(q[0][0]), "=&v"(q[0][1]), "=&v"(q[0][2]), "=&v"(q[0][3]), "=&v"(q[1][0]), "=&v"(q[1][1]),
                          "=&v"(q[1][2]), "=&v"(q[1][3]), "=&v"(sq[0]), "=&v"(sq[1]), "=&v"(bq[0]), "=&v"(bq[1])
                        : "v"(a0), "v"(a1), "v"(as)
                        : "memory");
                }
#pragma unroll
                for (int T = 0; T < 2; T++)
                    sw[T][0] = sq[T].x, sw[T][1] = sq[T].y, bw[T][0] = bq[T].x, bw[T][1] = bq[T].y;
            }
#pragma unroll
            for (int T = 0; T < 2; T++)
#pragma unroll
                for (int g = 0; g < 4; g++) d0[T][g] = q[T][g].x, d1[T][g] = q[T][g].y;
            consumed++;
            c = c + 1 == RING ? 0 : c + 1;
            issue();
            // (that wait covered the image reads above as well)
            lgkm_wait(abuf[0]);
            if constexpr (QK == 2) lgkm_wait(abuf[1]);
            asm volatile("" : "+v"(sA));

            // ---- bias and offset terms of the slab's four groups, one product per tile
#pragma unroll
            for (int T = 0; T < 2; T++) {
                uint32_t hb0, hb1, hs0, hs1, tb0, tb1, ts0, ts1;
                pfr_head_tail<FP16>(bw[T][0], hb0, tb0);
                pfr_head_tail<FP16>(bw[T][1], hb1, tb1);
                pfr_head_tail<FP16>(sw[T][0], hs0, ts0);
                pfr_head_tail<FP16>(sw[T][1], hs1, ts1);
                const bool last = kb == 3;
                const uint4 Bs = last ? make_uint4(tb0, tb1, ts0, ts1) : make_uint4(hb0, hb1, hs0, hs1);
                side[T] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, sA), __builtin_bit_cast(bf8, Bs),
                                                                  side[T], 0, 0, 0);
                if constexpr (FP16) {
                    // tails x piece 1 of both terms (k block 1 holds piece 1)
                    const bool one = kb == 1;
                    const uint4 A2 = one ? __builtin_bit_cast(uint4, sA) : make_uint4(0u, 0u, 0u, 0u);
                    const uint4 B2 = one ? make_uint4(tb0, tb1, ts0, ts1) : make_uint4(0u, 0u, 0u, 0u);
                    side[T] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, A2),
                                                                      __builtin_bit_cast(bf8, B2), side[T], 0, 0, 0);
                }
            }

            // ---- (tile, group): unpack this lane's 16 codes, two products per piece, scale
#pragma unroll
            for (int g = 0; g < 4; g++) {
                pfr_f4 D[2];
#pragma unroll
                for (int T = 0; T < 2; T++) {
                    uint32_t op[8];
                    if constexpr (BITS == 3) {
                        const uint32_t q0 = __builtin_amdgcn_alignbit(d1[T][g], d0[T][g], sh3), q1 = d1[T][g] >> sh3;
                        op[0] = ((q0 << 4) & PfrPair<3>::MASK) | ones;
                        op[1] = ((q0 << 1) & PfrPair<3>::MASK) | ones;
                        op[2] = ((q0 >> 2) & PfrPair<3>::MASK) | ones;
                        op[3] = ((q0 >> 5) & PfrPair<3>::MASK) | ones;
                        op[4] = (__builtin_amdgcn_alignbit(q1, q0, 20) & PfrPair<3>::MASK) | ones;
                        op[5] = (__builtin_amdgcn_alignbit(q1, q0, 23) & PfrPair<3>::MASK) | ones;
                        op[6] = (__builtin_amdgcn_alignbit(q1, q0, 26) & PfrPair<3>::MASK) | ones;
                        op[7] = (__builtin_amdgcn_alignbit(q1, q0, 29) & PfrPair<3>::MASK) | ones;
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            op[i] = ((d0[T][g] >> (4 * i)) & PfrPair<4>::MASK) | ones;
                            op[4 + i] = ((d1[T][g] >> (4 * i)) & PfrPair<4>::MASK) | ones;
                        }
                    }
                    D[T] = pfr_f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int j = 0; j < 2; j++) {
                        const bf8 b = __builtin_bit_cast(bf8, make_uint4(op[4 * j], op[4 * j + 1], op[4 * j + 2], op[4 * j + 3]));
#pragma unroll
                        for (int qq = 0; qq < QK; qq++) {
                            const int k = (g * 2 + j) * QK + qq;         // operand of the slab
                            D[T] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, abuf[k / 8][k % 8]), b,
                                                                           D[T], 0, 0, 0);
                        }
                    }
                }
#pragma unroll
                for (int T = 0; T < 2; T++) {
                    const uint32_t w = sw[T][g >> 1];
                    const float sc = (g & 1) ? fm_widen_hi<FP16>(w) : fm_widen_lo<FP16>(w);
#pragma unroll
                    for (int i = 0; i < 4; i++) acc[T][i] = fmaf(sc, D[T][i], acc[T][i]);
                }
            }
        }

        // ---- the task's 32 rows x positions
        const int r0 = t * (GU ? 16 : 32);
        float val[2][4];
#pragma unroll
        for (int T = 0; T < 2; T++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                val[T][i] = acc[T][i] + side[T][i];
                if constexpr (ROWP) {
                    // M rows p (lanes 0-31) and p + 8 (lanes 32-63) hold the two pieces' results
                    const uint32_t v = __float_as_uint(val[T][i]);
                    const auto hl = __builtin_amdgcn_permlane32_swap(v, v, false, false);
                    val[T][i] = __uint_as_float(hl[0]) + __uint_as_float(hl[1]);
                }
            }
        if constexpr (GU) {
            // tile 0 = gate rows, tile 1 = the same rows of up, both in this lane
            float *act = a.act + r0 + n;
            const bool mine = !ROWP || kb < 2;
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (mine && oidx[i] != ~0u) act[oidx[i]] = fm_silu_mul(val[0][i], val[1][i]);
        } else {
            float *eo = a.eo + r0 + n;
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (oidx[i] != ~0u) {
                    eo[oidx[i]] = val[0][i];
                    eo[oidx[i] + 16] = val[1][i];
                }
        }
    }
#else
    (void)a;
#endif
}

// Pairs grouped by expert and cut into items, twice: items of tm_up positions for the gate/up
// product and of tm_dn positions for the down product (the same grouping, `sorted`).  One
// workgroup of 1024 threads, one expert per thread for the prefix sums.
__global__ __launch_bounds__(1024) void fm_pf_group(PfArgs a) {
    __shared__ int hist[PF_MAX_EXPERTS], cursor[PF_MAX_EXPERTS], scan_a[16], scan_b[16], scan_c[16];
    const int E = a.g.n_experts, n = a.M * a.K, e = threadIdx.x;
    hist[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n; p += blockDim.x) {
        int x = a.idx[p];
        if ((unsigned)x < (unsigned)E) atomicAdd(&hist[x], 1);
    }
    __syncthreads();
    const int cnt = e < E ? hist[e] : 0;
    const int nu = (cnt + a.tm_up - 1) / a.tm_up, nd = (cnt + a.tm_dn - 1) / a.tm_dn;
    // inclusive scans of the pair counts and of both item counts: inside each wave by lane
    // shifts, the 16 wave totals by wave 0
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    int sa = cnt, sb = nu, sc = nd;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int va = __shfl_up(sa, d), vb = __shfl_up(sb, d), vc = __shfl_up(sc, d);
        if (lane >= d) sa += va, sb += vb, sc += vc;
    }
    if (lane == 63) scan_a[wv] = sa, scan_b[wv] = sb, scan_c[wv] = sc;
    __syncthreads();
    if (wv == 0) {
        int ta = lane < 16 ? scan_a[lane] : 0, tb = lane < 16 ? scan_b[lane] : 0, tc = lane < 16 ? scan_c[lane] : 0;
#pragma unroll
        for (int d = 1; d < 16; d <<= 1) {
            const int va = __shfl_up(ta, d), vb = __shfl_up(tb, d), vc = __shfl_up(tc, d);
            if (lane >= d) ta += va, tb += vb, tc += vc;
        }
        if (lane < 16) scan_a[lane] = ta, scan_b[lane] = tb, scan_c[lane] = tc;
    }
    __syncthreads();
    if (wv > 0) sa += scan_a[wv - 1], sb += scan_b[wv - 1], sc += scan_c[wv - 1];
    const int off = sa - cnt;
    cursor[e] = off;
    for (int s = 0; s < nu; s++) {
        const int left = cnt - s * a.tm_up;
        a.items_up[sb - nu + s] = PfItem{e, off + s * a.tm_up, left < a.tm_up ? left : a.tm_up, 0};
    }
    for (int s = 0; s < nd; s++) {
        const int left = cnt - s * a.tm_dn;
        a.items_dn[sc - nd + s] = PfItem{e, off + s * a.tm_dn, left < a.tm_dn ? left : a.tm_dn, 0};
    }
    if (e == 1023) *a.n_items_up = sb, *a.n_items_dn = sc;
    __syncthreads();
    for (int p = threadIdx.x; p < n; p += blockDim.x) {
        int x = a.idx[p];
        if ((unsigned)x < (unsigned)E) a.sorted[atomicAdd(&cursor[x], 1)] = p;
    }
}

// bf16 bits -> fp32 (chunks that take the per-position path)
__global__ __launch_bounds__(256) void fm_pf_widen(const uint16_t *src, float *dst, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = __uint_as_float((uint32_t)src[i] << 16);
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

bool pf_supported(const FmExpertGeom *g) {
    // 3- or 4-bit codes at the benchmark's widths (eight and two slabs of four groups)
    return (g->bits == 3 || g->bits == 4) && g->n_experts <= PF_MAX_EXPERTS && g->hidden == 2048 &&
           g->inter == 512;
}

template <int BITS, bool FP16>
int pf_launch(const PfArgs &a, const FmExpertGeom *g, int M, float *d_out, int flags, int n_cu,
              hipStream_t st) {
    const size_t n = (size_t)M * a.K;
    hipLaunchKernelGGL(fm_pf_group, dim3(1), dim3(1024), 0, st, a);
    const int grid_up = fm_pfr_grid(g->n_experts + (int)(n / a.tm_up), n_cu);
    const int grid_dn = fm_pfr_grid(g->n_experts + (int)(n / a.tm_dn), n_cu);
#define PFR_LAUNCH(MODE, XB, GRID)                                                               \
    do {                                                                                         \
        auto kfn = fm_pf_rows<MODE, BITS, FP16, XB>;                                             \
        constexpr int LDS = PfRows<MODE, BITS, MODE == PFR_GATE_UP ? 1 : 2>::LDS_BYTES;          \
        static FmLdsAttr attr;                                                                   \
        if (!fm_dyn_lds_ready(attr, (const void *)kfn, LDS)) return FM_ERR_HIP;                  \
        hipLaunchKernelGGL(kfn, dim3(GRID), dim3(512), LDS, st, a);                              \
    } while (0)
    if (a.Xbf) PFR_LAUNCH(PFR_GATE_UP, true, grid_up);
    else PFR_LAUNCH(PFR_GATE_UP, false, grid_up);
    PFR_LAUNCH(PFR_DOWN, false, grid_dn);
#undef PFR_LAUNCH
    hipLaunchKernelGGL(fm_pf_combine, dim3(M, (g->hidden + 1023) / 1024), dim3(256), 0, st, a, d_out, flags);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

template <int BITS, bool FP16>
int pf_launch_dense(PfArgs a, int n_cu, bool prepare, hipStream_t st) {
    const int prep_tasks = a.M * (a.d_cols / 64) * 2;
    if (prepare)
        hipLaunchKernelGGL(fm_pf_dense_prep<BITS>, dim3(1 + (prep_tasks + 1023) / 1024), dim3(1024), 0, st, a);
    const int grid = fm_pf_dense_grid(a.M, a.d_rows, 0, n_cu).grid;
    constexpr int LDS = PfSlab<BITS>::LDS_BYTES;
    static FmLdsAttr attr;
    if (!fm_dyn_lds_ready(attr, (const void *)fm_pf_gemm<PF_DENSE, BITS, FP16>, LDS)) return FM_ERR_HIP;
    if (a.d_cols == 512) {       // two slabs: the teams of the down product, 256 rows per step
        const int tgrid = fm_pf_dense_grid(a.M, a.d_rows, 1, n_cu).grid;
        static FmLdsAttr attr_t;
        if (!fm_dyn_lds_ready(attr_t, (const void *)fm_pf_gemm<PF_DENSE_TEAMS, BITS, FP16>, LDS)) return FM_ERR_HIP;
        hipLaunchKernelGGL((fm_pf_gemm<PF_DENSE_TEAMS, BITS, FP16>), dim3(tgrid), dim3(512), LDS, st, a);
        return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
    }
    for (int pass = 0; pass < a.d_cols / 2048; pass++) {
        a.d_pass = pass;
        hipLaunchKernelGGL((fm_pf_gemm<PF_DENSE, BITS, FP16>), dim3(grid), dim3(512), LDS, st, a);
    }
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

bool pf_dense_supported(int out_dim, int in_dim, int group_size, int bits) {
    if (!(bits == 3 || bits == 4) || group_size != 64) return false;
    // 512 columns: two slabs, four teams on 64 rows each
    if (in_dim == 512) return out_dim >= 256 && out_dim % 256 == 0;
    // eight slabs of four groups per column pass, two 32-row tiles per step
    return in_dim >= 2048 && in_dim % 2048 == 0 && in_dim <= 16384 && out_dim >= 64 && out_dim % 64 == 0;
}

// ======================================================================
// GGUF experts (Q4_K gate/up, Q6_K down), chunks of many positions: grouped products.
// Replaces the per-position pool kernels of prefill_chunk_cmd3_batch_general
// (finchmoe/infer.m:10958-11059; finchmoe/shaders.metal:3460-3517, 3641-3712), which stream
// every routed expert once per position, by one pass per (expert, group of its positions).
//
// One workgroup (8 waves) takes one item of fm_pf_group's lists — an expert and up to 8
// (gate/up) or 16 (down) of its positions — stages the positions' activations in LDS in MFMA
// operand form and walks the expert's rows, a wave per tile of 16 rows, codes straight from
// memory into registers (a lane's bytes of a block are used by no other lane).
//
// Arithmetic.  A block format is affine per sub-block: Q4_K y = (d sc_j) q - dmin m_j over 32
// values, Q6_K y = (d sc_g)(q - 32) over 16 (finchmoe/infer.m:1604-1657).  The codes go into
// bf16 mantissas as 1 + q/128 (fm_mfma.h) — one V_AND_OR per two codes — so a product over a
// sub-block is D' = sum x + sum q x / 128, exact products, fp32 sum; with xs = sum x from the
// staging pass, sum y x = (128 d sc) D' - (128 d sc + dmin m) xs for Q4_K and
// (128 d sc) D' - (160 d sc) xs for Q6_K, in fp32 on the accumulator registers.  fp32
// activations are two bf16 pieces (16 significant bits): gate/up puts them in M rows p and
// p + 8 of a 16x16x32 product, down runs two 16x16x16 products on one accumulator.
// ======================================================================
typedef short gq_s4 __attribute__((ext_vector_type(4)));
constexpr int GQ_TM_DN = 16;
// positions of a gate/up item: 16 where the two images of 16 positions fit in LDS, else 8
static inline int gq_tm_up(const FmGgufGeom *g) { return g->hidden <= 2048 ? 16 : 8; }

__device__ __forceinline__ uint32_t gq_hi(float v) { return __float_as_uint(v) >> 16; }
__device__ __forceinline__ uint32_t gq_lo(float v) {
    return __float_as_uint(v - __uint_as_float(__float_as_uint(v) & 0xFFFF0000u)) >> 16;
}
// what the two pieces of v add up to (what the products really multiply)
__device__ __forceinline__ float gq_both(float v) {
    const float h = __uint_as_float(__float_as_uint(v) & 0xFFFF0000u);
    return h + __uint_as_float(__float_as_uint(v - h) & 0xFFFF0000u);
}

// (scale, min) pair j of a Q4_K block's 12 scale bytes s0 s1 s2 (finchmoe/infer.m:1595-1603)
__device__ __forceinline__ void gq_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int j, float &sc, float &mn) {
    uint32_t a, b;
    if (j < 4) {
        a = (s0 >> (8 * j)) & 63u;
        b = (s1 >> (8 * j)) & 63u;
    } else {
        const int i = j - 4;
        const uint32_t hi = (s2 >> (8 * i)) & 0xFFu;
        a = (hi & 0xFu) | (((s0 >> (8 * i + 6)) & 3u) << 4);
        b = (hi >> 4) | (((s1 >> (8 * i + 6)) & 3u) << 4);
    }
    sc = (float)a;
    mn = (float)b;
}

// gate/up: Q4_K rows [inter][hidden/256 blocks of 144 B]; item = (expert, <= TM positions).
// TM = 8: the two bf16 pieces of position p in M rows p and p + 8 of one product.  TM = 16 (rows
// of at most 2048 values: the two images are 128 KB): a product per piece on one accumulator —
// twice the matrix instructions per item, but an expert with many positions is streamed and
// unpacked half as often.  A lane's bytes of the next block are requested before the block in
// hand is multiplied.
struct GqUpBlock {
    uint4 hdr[2];
    uint2 qs[2][4];
};
__device__ __forceinline__ void gq_up_load(GqUpBlock &k, const uint8_t *const rp[2], int b, int kb) {
#pragma unroll
    for (int T = 0; T < 2; T++) {
        const uint8_t *blk = rp[T] + (size_t)b * 144;
        k.hdr[T] = *reinterpret_cast<const uint4 *>(blk);
#pragma unroll
        for (int c = 0; c < 4; c++) k.qs[T][c] = *reinterpret_cast<const uint2 *>(blk + 16 + 32 * c + 8 * kb);
    }
}
// A workgroup's share of the launch: units u0 .. u1 of n_items * per_item, a unit = (item, group of
// eight 16-row tiles, one per wave).  Contiguous shares: a workgroup stages an item's positions
// when its units change item — once or twice more than its share of the items.
struct GqShare {
    int u0, u1;
};
__device__ __forceinline__ GqShare gq_share(int n_items, int per_item) {
    const FmRange r = fm_share((long)n_items * per_item, blockIdx.x, gridDim.x);
    GqShare s;
    s.u0 = (int)r.lo, s.u1 = (int)r.hi;
    return s;
}

template <int TM>
__global__ __launch_bounds__(512) void fm_gq_gate_up(PfArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
    extern __shared__ __attribute__((aligned(16))) uint8_t gq_smem[];
    constexpr bool TWO = TM == 16;
    const int H = a.g.hidden, I = a.g.inter, NKS = H / 32, NB = H / 256;
    const int tiles = I / 16, per_item = (tiles + 7) / 8;
    const GqShare sh_ = gq_share(*a.n_items_up, per_item);
    uint4 *img = reinterpret_cast<uint4 *>(gq_smem);                       // [NKS][64 lanes] (TWO: the hi pieces)
    uint4 *img_lo = img + (size_t)NKS * 64;                                // TWO only
    float *xs = reinterpret_cast<float *>(gq_smem + (size_t)NKS * 1024 * (TWO ? 2 : 1));   // [NKS][16 M rows]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const size_t row_bytes = (size_t)NB * 144;
    const uint32_t ones = fm_opaque(0x3F803F80u);
    int cur_item = -1;
    const int n_items = *a.n_items_up;
    PfItem item{0, 0, 0, 0}, item_next{0, 0, 0, 0};
    GqUpBlock pre;                           // the first block of this wave's next tile, requested a tile ahead
    bool pre_ok = false;
    for (int u = sh_.u0; u < sh_.u1; u++) {
        const int it = u / per_item, part = u - it * per_item;
        if (it != cur_item) {
            cur_item = it;
            item = a.items_up[it];
            item_next = a.items_up[it + 1 < n_items ? it + 1 : it];
            __syncthreads();                 // every wave is done with the images of the item before
            // ---- stage: thread (position p, k steps ks, ks + 512 / TM, ...)
            const int p = threadIdx.x & (TM - 1);
            const bool on = p < item.count;
            const size_t m = on ? (size_t)(a.sorted[item.start + p] / a.K) : 0;
            for (int ks = threadIdx.x / TM; ks < NKS; ks += 512 / TM) {
                float x[32];
                const float4 *src = reinterpret_cast<const float4 *>(a.X + m * H + 32 * ks);
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float4 v = on ? src[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    x[4 * i] = v.x, x[4 * i + 1] = v.y, x[4 * i + 2] = v.z, x[4 * i + 3] = v.w;
                }
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 32; i++) sum += gq_both(x[i]);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    // k slots of lane group q: bytes 0 2 | 1 3 | 4 6 | 5 7 of its eight values
                    const float *v = x + 8 * q;
                    const uint4 hi = make_uint4(gq_hi(v[0]) | (gq_hi(v[2]) << 16), gq_hi(v[1]) | (gq_hi(v[3]) << 16),
                                                gq_hi(v[4]) | (gq_hi(v[6]) << 16), gq_hi(v[5]) | (gq_hi(v[7]) << 16));
                    const uint4 lo = make_uint4(gq_lo(v[0]) | (gq_lo(v[2]) << 16), gq_lo(v[1]) | (gq_lo(v[3]) << 16),
                                                gq_lo(v[4]) | (gq_lo(v[6]) << 16), gq_lo(v[5]) | (gq_lo(v[7]) << 16));
                    img[(size_t)ks * 64 + 16 * q + p] = hi;
                    if constexpr (TWO) img_lo[(size_t)ks * 64 + 16 * q + p] = lo;
                    else img[(size_t)ks * 64 + 16 * q + p + 8] = lo;
                }
                xs[ks * 16 + p] = sum;
                if constexpr (!TWO) xs[ks * 16 + p + 8] = 0.0f;
            }
            __syncthreads();
        }
        const int tile = part * 8 + wave;
        if (tile >= tiles) continue;
        const uint8_t *gbase = a.gq_gate + (size_t)item.expert * I * row_bytes;
        const uint8_t *ubase = a.gq_up + (size_t)item.expert * I * row_bytes;
        const int row = tile * 16 + n;
        const uint8_t *const rp[2] = {gbase + (size_t)row * row_bytes, ubase + (size_t)row * row_bytes};
        pfr_f4 acc[2] = {pfr_f4{0.0f, 0.0f, 0.0f, 0.0f}, pfr_f4{0.0f, 0.0f, 0.0f, 0.0f}};
        GqUpBlock cur;
        if (pre_ok) cur = pre;
        else gq_up_load(cur, rp, 0, kb);
        pre_ok = false;
        for (int b = 0; b < NB; b++) {
            GqUpBlock nxt = cur;
            if (b + 1 < NB) {
                gq_up_load(nxt, rp, b + 1, kb);
            } else if (u + 1 < sh_.u1) {
                const int it2 = (u + 1) / per_item, tile2 = (u + 1 - it2 * per_item) * 8 + wave;
                if (tile2 < tiles) {
                    const int e2 = it2 == cur_item ? item.expert : item_next.expert;
                    const size_t r2 = ((size_t)e2 * I + (size_t)tile2 * 16 + n) * row_bytes;
                    const uint8_t *const rp2[2] = {a.gq_gate + r2, a.gq_up + r2};
                    gq_up_load(nxt, rp2, 0, kb);
                    pre_ok = true;
                }
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const int ks = b * 8 + j;
                const uint4 av = img[(size_t)ks * 64 + lane];
                uint4 al = av;
                if constexpr (TWO) al = img_lo[(size_t)ks * 64 + lane];
                const float4 xv = *reinterpret_cast<const float4 *>(xs + ks * 16 + 4 * kb);
#pragma unroll
                for (int T = 0; T < 2; T++) {
                    const float d = fm_fp16_bits(cur.hdr[T].x & 0xFFFFu), dmin = fm_fp16_bits(cur.hdr[T].x >> 16);
                    float sc, mn;
                    gq_scale_min(cur.hdr[T].y, cur.hdr[T].z, cur.hdr[T].w, j, sc, mn);
                    const float c1 = 128.0f * (d * sc), c2 = c1 + dmin * mn;
                    const uint2 w = cur.qs[T][j >> 1];
                    const int sh = (j & 1) * 4;
                    const pfr_u4 bq = {((w.x >> sh) & 0x000F000Fu) | ones, ((w.x >> (sh + 8)) & 0x000F000Fu) | ones,
                                       ((w.y >> sh) & 0x000F000Fu) | ones, ((w.y >> (sh + 8)) & 0x000F000Fu) | ones};
                    pfr_f4 D = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf8, av), __builtin_bit_cast(bf8, bq), pfr_f4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                    if constexpr (TWO)
                        D = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, al), __builtin_bit_cast(bf8, bq), D, 0, 0, 0);
                    acc[T][0] = fmaf(c1, D[0], fmaf(-c2, xv.x, acc[T][0]));
                    acc[T][1] = fmaf(c1, D[1], fmaf(-c2, xv.y, acc[T][1]));
                    acc[T][2] = fmaf(c1, D[2], fmaf(-c2, xv.z, acc[T][2]));
                    acc[T][3] = fmaf(c1, D[3], fmaf(-c2, xv.w, acc[T][3]));
                }
            }
            cur = nxt;
        }
        pre = cur;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int pos = 4 * kb + i;
            if constexpr (TWO) {
                if (pos < item.count) a.act[(size_t)(item.start + pos) * I + row] = fm_silu_mul(acc[0][i], acc[1][i]);
            } else {
                // M rows p and p + 8 (lanes kb and kb + 2) are the two pieces of position p
                const float g = acc[0][i] + __shfl_xor(acc[0][i], 32);
                const float u_ = acc[1][i] + __shfl_xor(acc[1][i], 32);
                if (kb < 2 && pos < item.count) a.act[(size_t)(item.start + pos) * I + row] = fm_silu_mul(g, u_);
            }
        }
    }
#else
    (void)a;
#endif
}

// down: Q6_K rows [hidden][inter/256 blocks of 210 B]; item = (expert, <= 16 positions);
// input a.act by sorted position, output a.eo by pair id.  Shares of units as in gate/up; a
// lane's words of the next block are requested before the block in hand is multiplied.
struct GqDnBlock {
    uint32_t ql[8], qh[4], scw[4], d;      // ql[4 h + 2 (qt & 1) + (g & 1)], qh[2 h + (g & 1)]
};
__device__ __forceinline__ void gq_dn_load(GqDnBlock &k, const uint8_t *blk, int kb) {
    struct __attribute__((packed, aligned(2))) U32a2 { uint32_t v; };
    struct __attribute__((packed, aligned(2))) U16a2 { uint16_t v; };
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int o = 0; o < 2; o++) {
            const int l = 16 * o + 4 * kb;
#pragma unroll
            for (int q1 = 0; q1 < 2; q1++) k.ql[4 * h + 2 * q1 + o] = reinterpret_cast<const U32a2 *>(blk + 64 * h + 32 * q1 + l)->v;
            k.qh[2 * h + o] = reinterpret_cast<const U32a2 *>(blk + 128 + 32 * h + l)->v;
        }
#pragma unroll
    for (int i = 0; i < 4; i++) k.scw[i] = reinterpret_cast<const U32a2 *>(blk + 192 + 4 * i)->v;
    k.d = reinterpret_cast<const U16a2 *>(blk + 208)->v;
}
// one block of one 16-row tile: the lane's words in `cur`, acc += its share of sum y x
__device__ __forceinline__ void gq_dn_block(const GqDnBlock &cur, int b, int lane, int kb, uint32_t ones,
                                            const uint2 *img_hi, const uint2 *img_lo, const uint2 *xsi, pfr_f4 &acc) {
    const float d = fm_fp16_bits(cur.d);
    {   // - 160 d sum_g sc_g xs_g: the block's 16 scales (exact in bf16) times the groups' sums of x,
        // this lane's k slots = groups 4 kb .. 4 kb + 3 = the bytes of scw[kb]
        const uint32_t w = kb == 0 ? cur.scw[0] : kb == 1 ? cur.scw[1] : kb == 2 ? cur.scw[2] : cur.scw[3];
        const uint32_t b0 = __float_as_uint((float)(int)(int8_t)(w & 0xFFu)) >> 16;
        const uint32_t b1 = __float_as_uint((float)(int)(int8_t)((w >> 8) & 0xFFu)) & 0xFFFF0000u;
        const uint32_t b2 = __float_as_uint((float)(int)(int8_t)((w >> 16) & 0xFFu)) >> 16;
        const uint32_t b3 = __float_as_uint((float)(int)(int8_t)(w >> 24)) & 0xFFFF0000u;
        const uint2 bs = make_uint2(b0 | b1, b2 | b3);
        const uint2 *xp = xsi + (size_t)b * 3 * 64 + lane;
        pfr_f4 E = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(gq_s4, xp[0]), __builtin_bit_cast(gq_s4, bs),
                                                            pfr_f4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        E = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(gq_s4, xp[64]), __builtin_bit_cast(gq_s4, bs), E, 0, 0, 0);
        E = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(gq_s4, xp[128]), __builtin_bit_cast(gq_s4, bs), E, 0, 0, 0);
        const float c2 = -160.0f * d;
        acc[0] = fmaf(c2, E[0], acc[0]);
        acc[1] = fmaf(c2, E[1], acc[1]);
        acc[2] = fmaf(c2, E[2], acc[2]);
        acc[3] = fmaf(c2, E[3], acc[3]);
    }
#pragma unroll
    for (int g = 0; g < 16; g++) {
        // group g: half h, quarter qt of the half (which nibble / which two qh bits),
        // l = 16 (g & 1) + 4 kb .. + 3 (finchmoe/infer.m:1636-1657)
        const int h = g >> 3, qt = (g >> 1) & 3;
        const uint32_t wql = cur.ql[4 * h + 2 * (qt & 1) + (g & 1)];
        const uint32_t wqh = cur.qh[2 * h + (g & 1)];
        const uint32_t code = ((wql >> (4 * (qt >> 1))) & 0x0F0F0F0Fu) | (((wqh >> (2 * qt)) & 0x03030303u) << 4);
        const uint2 bq = make_uint2((code & 0x00FF00FFu) | ones, ((code >> 8) & 0x00FF00FFu) | ones);
        const int ks = b * 16 + g;
        const uint2 ah = img_hi[(size_t)ks * 64 + lane], al = img_lo[(size_t)ks * 64 + lane];
        pfr_f4 D = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(gq_s4, ah), __builtin_bit_cast(gq_s4, bq),
                                                            pfr_f4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
        D = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(gq_s4, al), __builtin_bit_cast(gq_s4, bq), D, 0, 0, 0);
        const float sc = (float)(int)(int8_t)((cur.scw[g >> 2] >> (8 * (g & 3))) & 0xFFu);
        const float c1 = 128.0f * (d * sc);
        acc[0] = fmaf(c1, D[0], acc[0]);
        acc[1] = fmaf(c1, D[1], acc[1]);
        acc[2] = fmaf(c1, D[2], acc[2]);
        acc[3] = fmaf(c1, D[3], acc[3]);
    }
}

// (A form that copied a tile's 16 whole rows — one contiguous run — into a per-wave LDS buffer with
// 16-byte loads and picked the words out of LDS was slower, 146 against 124 us: the loads are not
// what bounds this kernel.)
__global__ __launch_bounds__(512) void fm_gq_down(PfArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
    extern __shared__ __attribute__((aligned(16))) uint8_t gq_smem[];
    __shared__ int pairs[GQ_TM_DN];
    constexpr int NW = 8, NT = NW * 64;
    const int H = a.g.hidden, I = a.g.inter, NKS = I / 16, NB = I / 256;
    const int tiles = H / 16, per_item = (tiles + NW - 1) / NW;
    const GqShare sh_ = gq_share(*a.n_items_dn, per_item);
    uint2 *img_hi = reinterpret_cast<uint2 *>(gq_smem);                    // [NKS][64 lanes]
    uint2 *img_lo = img_hi + (size_t)NKS * 64;
    // the sums of x over each scale group, as three bf16 pieces (exactly the fp32 sum) in the
    // operand form of a 16x16x16 product over a block's 16 groups: [NB][3 pieces][64 lanes]
    uint2 *xsi = img_lo + (size_t)NKS * 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, kb = lane >> 4;
    const size_t row_bytes = (size_t)NB * 210;
    const uint32_t ones = fm_opaque(0x3F803F80u);
    int cur_item = -1;
    const int n_items = *a.n_items_dn;
    PfItem item{0, 0, 0, 0}, item_next{0, 0, 0, 0};
    GqDnBlock pre;                           // the first block of this wave's next tile, requested a tile ahead
    bool pre_ok = false;
    for (int u = sh_.u0; u < sh_.u1; u++) {
        const int it = u / per_item, part = u - it * per_item;
        if (it != cur_item) {
            cur_item = it;
            item = a.items_dn[it];
            item_next = a.items_dn[it + 1 < n_items ? it + 1 : it];
            __syncthreads();                 // every wave is done with the images and pair ids of the item before
            const int p = threadIdx.x & 15;
            const bool on = p < item.count;
            if (threadIdx.x < GQ_TM_DN) pairs[p] = on ? a.sorted[item.start + p] : 0;
            const float *arow = a.act + (size_t)(item.start + (on ? p : 0)) * I;
            for (int ks = threadIdx.x >> 4; ks < NKS; ks += NT / 16) {
                float x[16];
                const float4 *src = reinterpret_cast<const float4 *>(arow + 16 * ks);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float4 v = on ? src[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    x[4 * i] = v.x, x[4 * i + 1] = v.y, x[4 * i + 2] = v.z, x[4 * i + 3] = v.w;
                }
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; i++) sum += gq_both(x[i]);
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float *v = x + 4 * q;        // k slots: values 0 2 | 1 3 of the lane group's four
                    img_hi[(size_t)ks * 64 + 16 * q + p] = make_uint2(gq_hi(v[0]) | (gq_hi(v[2]) << 16), gq_hi(v[1]) | (gq_hi(v[3]) << 16));
                    img_lo[(size_t)ks * 64 + 16 * q + p] = make_uint2(gq_lo(v[0]) | (gq_lo(v[2]) << 16), gq_lo(v[1]) | (gq_lo(v[3]) << 16));
                }
                // group ks = 16 b + 4 kq + i: k slot i of lane (p, kq) of block b
                const uint32_t s0 = __float_as_uint(sum) & 0xFFFF0000u;
                const float r1 = sum - __uint_as_float(s0);
                const uint32_t s1 = __float_as_uint(r1) & 0xFFFF0000u;
                const uint32_t s2 = __float_as_uint(r1 - __uint_as_float(s1));
                uint16_t *dst = reinterpret_cast<uint16_t *>(xsi + ((size_t)(ks >> 4) * 3) * 64 + 16 * ((ks >> 2) & 3) + p) + (ks & 3);
                dst[0] = (uint16_t)(s0 >> 16);
                dst[64 * 4] = (uint16_t)(s1 >> 16);
                dst[2 * 64 * 4] = (uint16_t)(s2 >> 16);
            }
            __syncthreads();
        }
        const int tile = part * NW + wave;
        if (tile >= tiles) continue;
        const int row = tile * 16 + n;
        // the wave's tile of the next unit, if it has one
        const uint8_t *next_src = nullptr;
        if (u + 1 < sh_.u1) {
            const int it2 = (u + 1) / per_item, tile2 = (u + 1 - it2 * per_item) * NW + wave;
            if (tile2 < tiles) {
                const int e2 = it2 == cur_item ? item.expert : item_next.expert;
                next_src = a.gq_down + ((size_t)e2 * H + (size_t)tile2 * 16) * row_bytes;
            }
        }
        pfr_f4 acc = pfr_f4{0.0f, 0.0f, 0.0f, 0.0f};
        {
            const uint8_t *rp = a.gq_down + ((size_t)item.expert * H + row) * row_bytes;
            GqDnBlock cur;
            if (pre_ok) cur = pre;
            else gq_dn_load(cur, rp, kb);
            pre_ok = false;
            for (int b = 0; b < NB; b++) {
                GqDnBlock nxt = cur;
                if (b + 1 < NB) {
                    gq_dn_load(nxt, rp + (size_t)(b + 1) * 210, kb);
                } else if (next_src) {
                    gq_dn_load(nxt, next_src + (size_t)n * row_bytes, kb);
                    pre_ok = true;
                }
                gq_dn_block(cur, b, lane, kb, ones, img_hi, img_lo, xsi, acc);
                cur = nxt;
            }
            pre = cur;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int pos = 4 * kb + i;
            if (pos < item.count) a.eo[(size_t)pairs[pos] * H + row] = acc[i];
        }
    }
#else
    (void)a;
#endif
}

}  // namespace

// Dense tensor against M positions on the same matrix-core kernel as the expert products
// (gpu_encode_prefill_matvec, finchmoe/infer.m:3672: the reference runs M matvecs).
extern "C" size_t fm_prefill_dense_ws_bytes(int out_dim, int in_dim, int group_size, int bits, int M) {
    if (!pf_dense_supported(out_dim, in_dim, group_size, bits) || M < 1) return 0;
    static_assert(sizeof(PfItem) == 16 && sizeof(uint4) == 16 && sizeof(float2) == 8, "sizes of fm_pf_dense_ws");
    return fm_pf_dense_ws(M, in_dim).total;
}

extern "C" int fm_launch_prefill_dense(const void *d_W, const void *d_S, const void *d_B, int out_dim,
                                       int in_dim, int group_size, int bits, int scale_fp16,
                                       const float *d_X, int M, float *d_out, void *d_ws,
                                       size_t ws_bytes, int flags, int prepare, int n_cu,
                                       hipStream_t st) {
    const size_t need = fm_prefill_dense_ws_bytes(out_dim, in_dim, group_size, bits, M);
    if (need == 0) return FM_ERR_UNSUPPORTED;
    if (ws_bytes < need) return FM_ERR_ARG;
    {   // Launches in which a workgroup takes more than one step (more steps than CUs) last ran in a
        // session that ended with a GPU memory fault whose cause is not known; the host walk of
        // their addresses is clean, but until the cause is known they are not taken: the caller
        // runs one GEMV per position.
        const FmPfDenseGrid gr = fm_pf_dense_grid(M, out_dim, in_dim == 512, n_cu);
        if ((long)gr.items * gr.n_steps > (long)n_cu) return FM_ERR_UNSUPPORTED;
    }
    char *ws = (char *)d_ws;
    PfArgs a{};
    a.X = d_X;
    a.M = M;
    a.K = 1;
    const FmPfDenseWs lay = fm_pf_dense_ws(M, in_dim);
    a.items = (PfItem *)(ws + lay.items);
    a.n_items = (int *)(ws + lay.n_items);
    a.xop = (uint4 *)(ws + lay.xop);
    a.xsums = (float2 *)(ws + lay.xsums);
    a.d_w = (const uint8_t *)d_W;
    a.d_s = (const uint8_t *)d_S - (const uint8_t *)d_W;
    a.d_b = (const uint8_t *)d_B - (const uint8_t *)d_W;
    a.d_rows = out_dim;
    a.d_cols = in_dim;
    a.d_pass = 0;
    a.d_flags = flags;
    a.d_out = d_out;
    // prepare = 0: the workspace holds X's operand form from the call before (same X, M, in_dim
    // and code width: the pairing of the codes depends on the width)
    const bool prep = prepare != 0;
    if (scale_fp16)
        return bits == 3 ? pf_launch_dense<3, true>(a, n_cu, prep, st) : pf_launch_dense<4, true>(a, n_cu, prep, st);
    return bits == 3 ? pf_launch_dense<3, false>(a, n_cu, prep, st) : pf_launch_dense<4, false>(a, n_cu, prep, st);
}

// positions per item of the two products: 16, or 8 for gate/up on fp32 activations
static inline int pf_tm_up(int x_bf16) { return x_bf16 ? 16 : 8; }

extern "C" size_t fm_prefill_affine_ws_bytes(const FmExpertGeom *g, int M, int K, int x_bf16) {
    if (!pf_supported(g)) return 0;
    const size_t n = (size_t)M * K;
    return align256(n * 4) + align256((g->n_experts + n / pf_tm_up(x_bf16) + 1) * sizeof(PfItem)) +
           align256((g->n_experts + n / 16 + 1) * sizeof(PfItem)) + 256 + align256(n * g->inter * 4) +
           align256(n * g->hidden * 4);
}

// d_X: fp32 [M][hidden], or bf16 bits [M][hidden] when x_bf16 is set
extern "C" int fm_launch_prefill_affine(const uint8_t *d_layer, const FmExpertGeom *g,
                                        const void *d_X, int x_bf16, const int32_t *d_idx,
                                        const float *d_w, int M, int K, float *d_out, void *d_ws,
                                        size_t ws_bytes, int flags, int n_cu, hipStream_t st) {
    if (!pf_supported(g)) return FM_ERR_UNSUPPORTED;
    if (ws_bytes < fm_prefill_affine_ws_bytes(g, M, K, x_bf16)) return FM_ERR_ARG;
    const size_t n = (size_t)M * K;
    char *ws = (char *)d_ws;
    PfArgs a{};
    a.layer = d_layer;
    a.g = *g;
    a.X = x_bf16 ? nullptr : (const float *)d_X;
    a.Xbf = x_bf16 ? (const uint16_t *)d_X : nullptr;
    a.idx = d_idx;
    a.w = d_w;
    a.M = M;
    a.K = K;
    a.tm_up = pf_tm_up(x_bf16);
    a.tm_dn = 16;
    a.sorted = (int *)ws;                 ws += align256(n * 4);
    a.items_up = (PfItem *)ws;            ws += align256((g->n_experts + n / a.tm_up + 1) * sizeof(PfItem));
    a.items_dn = (PfItem *)ws;            ws += align256((g->n_experts + n / a.tm_dn + 1) * sizeof(PfItem));
    a.n_items_up = (int *)ws;
    a.n_items_dn = (int *)ws + 1;         ws += 256;
    a.act = (float *)ws;                  ws += align256(n * g->inter * 4);
    a.eo = (float *)ws;
    if (g->scale_fp16)
        return g->bits == 3 ? pf_launch<3, true>(a, g, M, d_out, flags, n_cu, st)
                            : pf_launch<4, true>(a, g, M, d_out, flags, n_cu, st);
    return g->bits == 3 ? pf_launch<3, false>(a, g, M, d_out, flags, n_cu, st)
                        : pf_launch<4, false>(a, g, M, d_out, flags, n_cu, st);
}

// ---- GGUF experts: grouped products of a chunk ----------------------------------------------
static bool gq_supported(const FmGgufGeom *g) {
    return g->gate_type == FM_GGML_Q4_K && g->up_type == FM_GGML_Q4_K && g->down_type == FM_GGML_Q6_K &&
           g->n_experts <= PF_MAX_EXPERTS && g->hidden % 256 == 0 && g->inter % 256 == 0 &&
           g->hidden <= 4096 && g->inter <= 4096;
}

extern "C" size_t fm_prefill_gguf_ws_bytes(const FmGgufGeom *g, int M, int K) {
    if (!gq_supported(g) || M < 1 || K < 1) return 0;
    const size_t n = (size_t)M * K;
    return align256(n * 4) + align256((g->n_experts + n / gq_tm_up(g) + 1) * sizeof(PfItem)) +
           align256((g->n_experts + n / GQ_TM_DN + 1) * sizeof(PfItem)) + 256 +
           align256(n * g->inter * 4) + align256(n * g->hidden * 4);
}

// d_gate / d_up / d_down: the layer's slabs.  FM_ERR_UNSUPPORTED: the caller runs the chunk
// position by position.
extern "C" int fm_launch_prefill_gguf(const uint8_t *d_gate, const uint8_t *d_up, const uint8_t *d_down,
                                      const FmGgufGeom *g, const float *d_X, const int32_t *d_idx,
                                      const float *d_w, int M, int K, float *d_out, void *d_ws,
                                      size_t ws_bytes, int flags, int n_cu, hipStream_t st) {
    if (!gq_supported(g)) return FM_ERR_UNSUPPORTED;
    if (ws_bytes < fm_prefill_gguf_ws_bytes(g, M, K)) return FM_ERR_ARG;
    const size_t n = (size_t)M * K;
    char *ws = (char *)d_ws;
    PfArgs a{};
    a.g.hidden = g->hidden;
    a.g.inter = g->inter;
    a.g.n_experts = g->n_experts;
    a.X = d_X;
    a.idx = d_idx;
    a.w = d_w;
    a.M = M;
    a.K = K;
    a.tm_up = gq_tm_up(g);
    a.tm_dn = GQ_TM_DN;
    a.gq_gate = d_gate;
    a.gq_up = d_up;
    a.gq_down = d_down;
    a.sorted = (int *)ws;                 ws += align256(n * 4);
    a.items_up = (PfItem *)ws;            ws += align256((g->n_experts + n / a.tm_up + 1) * sizeof(PfItem));
    a.items_dn = (PfItem *)ws;            ws += align256((g->n_experts + n / GQ_TM_DN + 1) * sizeof(PfItem));
    a.n_items_up = (int *)ws;
    a.n_items_dn = (int *)ws + 1;         ws += 256;
    a.act = (float *)ws;                  ws += align256(n * g->inter * 4);
    a.eo = (float *)ws;
    const bool two = a.tm_up == 16;
    const size_t lds_up = (size_t)(g->hidden / 32) * ((two ? 2048 : 1024) + 64), lds_dn = (size_t)(g->inter / 16) * 1024 + (size_t)(g->inter / 256) * 1536;
    if (lds_up > 160 * 1024 - 1024 || lds_dn > 160 * 1024 - 1024) return FM_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(fm_pf_group, dim3(1), dim3(1024), 0, st, a);
    static FmLdsAttr attr_up8, attr_up16, attr_dn;
    if (!fm_dyn_lds_ready(attr_up8, (const void *)fm_gq_gate_up<8>, 160 * 1024 - 1024)) return FM_ERR_HIP;
    if (!fm_dyn_lds_ready(attr_up16, (const void *)fm_gq_gate_up<16>, 160 * 1024 - 1024)) return FM_ERR_HIP;
    if (!fm_dyn_lds_ready(attr_dn, (const void *)fm_gq_down, 160 * 1024 - 1024)) return FM_ERR_HIP;
    // persistent grids: one workgroup per CU for gate/up (its images fill most of the LDS), two for down
    const dim3 grid_up((unsigned)(n_cu > 0 ? n_cu : 256)), grid_dn((unsigned)(2 * (n_cu > 0 ? n_cu : 256)));
    if (two) hipLaunchKernelGGL(fm_gq_gate_up<16>, grid_up, dim3(512), lds_up, st, a);
    else hipLaunchKernelGGL(fm_gq_gate_up<8>, grid_up, dim3(512), lds_up, st, a);
    hipLaunchKernelGGL(fm_gq_down, grid_dn, dim3(512), lds_dn, st, a);
    hipLaunchKernelGGL(fm_pf_combine, dim3(M, (g->hidden + 1023) / 1024), dim3(256), 0, st, a, d_out, flags);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

extern "C" int fm_launch_widen_bf16(const uint16_t *d_src, float *d_dst, size_t n, hipStream_t st) {
    hipLaunchKernelGGL(fm_pf_widen, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, d_src, d_dst, n);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}
