// fm_prefill.hip — grouped chunked-prefill expert product on bf16 MFMA.
//
// The reference has no GEMM here: prefill_chunk_cmd3_encode (finchmoe/infer.m:
// 10704-10765) runs the per-position GEMV chain for each of the M positions, so two
// positions routed to the same expert read its weights twice.  This file groups
// the M*K (position, slot) pairs by expert and multiplies each expert's weights
// once against all of its positions.  Numerical contract: the per-position
// result (fm_decode.hip) within the parity bar.
//
// Why not "dequantize to bf16 and multiply": rounding (q*s + b) to bf16 misses
// the bar (max relative error 1.8e-3 on the benchmark's weight distribution).
// Instead
//   * the CODES are the MFMA operand, as exact bf16 numbers 1 + q*2^t/128 (the
//     mantissa trick of fm_mfma.h: one V_AND_OR_B32 per two codes; 4-bit codes: t = 0);
//   * each quantization group (64 columns) is accumulated by its own MFMA chain
//     and its scale is applied to the result in fp32: acc += s[row][g] * D_g;
//   * activations are split hi + lo (two bf16 pieces, 16 significant bits); the
//     pieces are extra M rows: M row j = hi piece of position j, row j+16 = lo piece,
//     which land in registers i and i+8 of the same lane;
//   * the bias term sum_g b[row][g] * xsum[pos][g] and the offset the "1 +" adds,
//     sum_g s[row][g] * xoff[pos][g], are two small products over the group index,
//     also on MFMA: the bf16 bits of b and s are operands as they are (FP16 ones are
//     split into a bf16 head and tail first, pf_side_b).
//
// V_MFMA_F32_32X32X16_BF16 with positions on M and weight rows on N: lane
// (n = lane%32, h = lane/32) supplies 8 consecutive k of weight row n and holds
// 16 results, all of weight row n — so a lane needs ONE scale per group.
// A lane's codes for one group are half a group: 32 codes = 12 bytes (3-bit) or 16 bytes
// (4-bit).  The kernels are instantiated for both widths.
//
// Work item = (expert, up to 16 of its positions).  Four kinds of kernel per chunk:
//   fm_pf_sort         workgroup 0 groups the pairs by expert and cuts them into items; the
//                      others turn X into MFMA operand registers (pf_prepare)
//   fm_pf_gemm<false>  gate/up + SwiGLU for every item -> act (by sorted position)
//   fm_pf_prepare_act  act -> operand registers
//   fm_pf_gemm<true>   down for every item -> expert_out (by pair)
//   fm_pf_combine      weighted sum in slot order
#include "fm_mfma.h"
#include "fm_ring.h"

namespace {

typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef const __attribute__((address_space(1))) uint8_t *gptr;

#define PF_TM 16          // positions per item
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
    uint4 *aop;        // [M*K][inter/64][4][2][2]: act (by sorted position) in the same form
    float2 *asums;     // [M*K][inter/64]
    // dense tensor (PF_DENSE): out[M][d_rows] = X[M][d_cols] * W^T, scales / biases d_sb bytes
    // behind / before W; one launch covers the 2048 columns of pass d_pass
    const uint8_t *d_w;
    ptrdiff_t d_s, d_b;
    int d_rows, d_cols, d_pass, d_flags;
    float *d_out;
};

enum { PF_GATE_UP = 0, PF_DOWN = 1, PF_DENSE = 2, PF_DENSE_TEAMS = 3 };

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
// pairs -> grouped by expert, cut into items of <= PF_TM positions.  One workgroup of
// 1024 threads, one expert per thread for the two prefix sums.
// X in the form the gate/up kernel multiplies with: per position, group, k step and column
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
    const int h = task & 1, g = (task >> 1) % NG, m = task / (2 * NG);
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
        uint4 *dst = dst_op + ((size_t)m * NG + g) * 16;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            dst[4 * k + 2 * h] = regs[4 * k];
            dst[4 * k + 2 * h + 1] = regs[4 * k + 1];
        }
        if (h == 0) dst_sums[(size_t)m * NG + g] = make_float2(xs, xo);
    }
}

// the SwiGLU outputs (by sorted position) as operand registers for the down product
template <int BITS>
__global__ __launch_bounds__(256) void fm_pf_prepare_act(PfArgs a) {
    pf_prepare<BITS>(a.act, a.M * a.K, a.g.inter, a.aop, a.asums, (int)(blockIdx.x * blockDim.x + threadIdx.x));
}

// workgroup 0 sorts, the others prepare X
template <int BITS>
__global__ __launch_bounds__(1024) void fm_pf_sort(PfArgs a) {
    __shared__ int hist[PF_MAX_EXPERTS], cursor[PF_MAX_EXPERTS], scan_a[PF_MAX_EXPERTS],
        scan_b[PF_MAX_EXPERTS];
    if (blockIdx.x > 0) {
        pf_prepare<BITS>(a.X, a.M, a.g.hidden, a.xop, a.xsums, (int)((blockIdx.x - 1) * blockDim.x + threadIdx.x));
        return;
    }
    const int E = a.g.n_experts, n = a.M * a.K, e = threadIdx.x;
    hist[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n; p += blockDim.x) {
        int x = a.idx[p];
        if ((unsigned)x < (unsigned)E) atomicAdd(&hist[x], 1);
    }
    __syncthreads();
    const int cnt = e < E ? hist[e] : 0, nit = (cnt + PF_TM - 1) / PF_TM;
    // inclusive scans of the pair counts and the item counts: inside each wave by lane
    // shifts, the 16 wave totals by wave 0, two barriers in all
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    int sa = cnt, sb = nit;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int va = __shfl_up(sa, d), vb = __shfl_up(sb, d);
        if (lane >= d) sa += va, sb += vb;
    }
    if (lane == 63) scan_a[wv] = sa, scan_b[wv] = sb;
    __syncthreads();
    if (wv == 0) {
        int ta = lane < 16 ? scan_a[lane] : 0, tb = lane < 16 ? scan_b[lane] : 0;
#pragma unroll
        for (int d = 1; d < 16; d <<= 1) {
            const int va = __shfl_up(ta, d), vb = __shfl_up(tb, d);
            if (lane >= d) ta += va, tb += vb;
        }
        if (lane < 16) scan_a[lane] = ta, scan_b[lane] = tb;     // inclusive totals of waves 0..lane
    }
    __syncthreads();
    if (wv > 0) sa += scan_a[wv - 1], sb += scan_b[wv - 1];
    const int off = sa - cnt, ioff = sb - nit;
    cursor[e] = off;
    for (int s = 0; s < nit; s++) {
        PfItem it;
        it.expert = e;
        it.start = off + s * PF_TM;
        it.count = cnt - s * PF_TM < PF_TM ? cnt - s * PF_TM : PF_TM;
        it.pad = 0;
        a.items[ioff + s] = it;
    }
    if (e == 1023) *a.n_items = sb;
    __syncthreads();
    for (int p = threadIdx.x; p < n; p += blockDim.x) {
        int x = a.idx[p];
        if ((unsigned)x < (unsigned)E) a.sorted[atomicAdd(&cursor[x], 1)] = p;
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
    static constexpr int GPW = 4;                       // groups per wave
    static constexpr int CB = 8 * BITS * GPW;           // code bytes of a row inside the slab: 96 / 128
    static constexpr int PS = 16;                       // bytes a lane copies per load
    static constexpr int RP = CB / PS;                  // pieces per row: 6 / 8
    // a row takes one piece slot more in LDS (it stays empty): with 96- or 128-byte rows the
    // 128-bit reads of neighbouring rows would hit the same banks
    static constexpr int RS = RP + 1;                   // piece slots per row in LDS: 7 / 9
    static constexpr int PIECES = 32 * RS;              // piece slots of a tile-matrix: 224 / 288
    static constexpr int NQ = (PIECES + 63) / 64;       // LDS-direct loads for the codes
    static constexpr int LDS_CODE = PIECES * PS;        // 3584 / 4608
    static constexpr int SLOT = LDS_CODE + 512;         // + scales 256 + biases 256
    static constexpr int LOADS = NQ + 2;
    static constexpr int RED_BYTES = 2 * 2 * 8 * 8 * 64 * 4;   // [buffer][matrix][wave][reg][lane]
    // what is left of the 160 KB for the eight waves' rings: 3 slots of 4096 B / 2 of 5120 B
    static constexpr int RING = (160 * 1024 - RED_BYTES) / (8 * SLOT);
    static constexpr int LDS_BYTES = 8 * RING * SLOT + RED_BYTES;
    static_assert(RING >= 2, "a ring needs a slot in flight beside the one being multiplied");
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

// MODE PF_GATE_UP (DOWN = false): K = hidden is eight slabs, wave w owns slab w, all waves work on the
//   same 32 rows; a step = the gate tile and the up tile of those rows; sum over eight waves,
//   SwiGLU, act.
// MODE PF_DOWN: K = inter is two slabs: the workgroup is four teams of two waves (slab = wave & 1),
//   every team on its own 64 rows of a step's 256; a step = two row tiles per team; sum over
//   the team's two waves, expert_out.  The activation operand comes from aop / asums
//   (fm_pf_prepare_act), indexed by sorted position.
// MODE PF_DENSE: one dense tensor against M positions, 2048 of its columns per launch (eight slabs
//   as in gate/up; column pass d_pass adds to what the passes before it stored); an item is a
//   block of 16 positions, a step = two row tiles (64 rows), the operand comes from xop.
// MODE PF_DENSE_TEAMS: a dense tensor of 512 columns: the slabs and teams of PF_DOWN (a step =
//   256 rows), operand and output as in PF_DENSE.
template <int MODE, int BITS, bool FP16>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void fm_pf_gemm(PfArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)   // (the host pass cannot allocate the registers of the asm blocks)
    using P = PfSlab<BITS>;
    constexpr int DW = PfCode<BITS>::DW;
    // TEAMS: geometry of the down product; DTENSOR: operands of a dense tensor; DENSE / DOWN: the
    // two pure forms
    constexpr bool TEAMS = MODE == PF_DOWN || MODE == PF_DENSE_TEAMS;
    constexpr bool DTENSOR = MODE == PF_DENSE || MODE == PF_DENSE_TEAMS;
    constexpr bool DOWN = MODE == PF_DOWN, DENSE = MODE == PF_DENSE;
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
    const int in_dim = DTENSOR ? a.d_cols : DOWN ? a.g.inter : a.g.hidden;
    const int row_bytes = in_dim * BITS / 8, sb_bytes = (in_dim / 64) * 2;
    const int slab = DENSE ? wave + 8 * a.d_pass : TEAMS ? (wave & 1) : wave, team = TEAMS ? (wave >> 1) : 0;
    const int n_steps = DENSE ? a.d_rows / 64 : DTENSOR ? a.d_rows / 256 : DOWN ? a.g.hidden / 256 : a.g.inter / 32;
    const uint32_t ones = fm_opaque(0x3F803F80u);
    // region offsets of the first tile-matrix of a step (this team's), the distance to the
    // second one, rows per step
    // (byte offsets from the blob's — the dense tensor's W — first byte, modulo 2^64)
    const size_t team_w = 64u * team * row_bytes, team_sb = 64u * team * sb_bytes;
    const size_t w_off0 = DTENSOR ? team_w : DOWN ? a.g.down_w + team_w : a.g.gate_w;
    const size_t s_off0 = DTENSOR ? (size_t)a.d_s + team_sb : DOWN ? a.g.down_s + team_sb : a.g.gate_s;
    const size_t b_off0 = DTENSOR ? (size_t)a.d_b + team_sb : DOWN ? a.g.down_b + team_sb : a.g.gate_b;
    const uint32_t w_d = TEAMS || DENSE ? 32u * row_bytes : a.g.up_w - a.g.gate_w;
    const uint32_t s_d = TEAMS || DENSE ? 32u * sb_bytes : a.g.up_s - a.g.gate_s;
    const uint32_t b_d = TEAMS || DENSE ? 32u * sb_bytes : a.g.up_b - a.g.gate_b;
    const uint32_t step_rows = DENSE ? 64u : TEAMS ? 256u : 32u;
    const uint8_t *store = DTENSOR ? a.d_w : a.layer;        // what an item's "expert" indexes into
    const size_t expert_size = DTENSOR ? 0 : a.g.expert_size;
    // this lane's pieces of a slot copy
    uint32_t coff[P::NQ];
    bool cvalid[P::NQ];
#pragma unroll
    for (int j = 0; j < P::NQ; j++) {
        const int q = 64 * j + lane;
        const int row = q / P::RS, piece = q - row * P::RS;
        cvalid[j] = q < P::PIECES && piece < P::RP;
        coff[j] = (uint32_t)(row * row_bytes + P::CB * slab + P::PS * piece);
    }
    // scales / biases of the slab: 2*GPW bytes per row, fetched as whole dwords
    const int sb_slab = (2 * GPW * slab) & ~3;
    const uint32_t soff = (uint32_t)((lane >> 1) * sb_bytes + sb_slab + 4 * (lane & 1));

    // ---- this workgroup's share of the launch: steps [t0, t1) of the sequence
    // (item, step), items in order — every workgroup gets the same number of steps
    // (within one) whatever the number of items, at the price of building the
    // activation operand of an item in two workgroups when a share ends inside it
    // Workgroups are dealt out to the eight XCDs in turn and every XCD has an L2 of its own:
    // workgroup b takes share (b % 8) * (grid / 8) + b / 8, so that neighbouring shares — the
    // items of one expert — run behind the same L2 and its weights come from HBM once.
    const long T = (long)n_items * n_steps;
    const unsigned int share = gridDim.x % 8u == 0u ? (blockIdx.x % 8u) * (gridDim.x / 8u) + blockIdx.x / 8u
                                                    : blockIdx.x;
    const int t0 = (int)(T * share / gridDim.x), t1 = (int)(T * (share + 1) / gridDim.x);

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
        const size_t row0 = (size_t)l_s * step_rows;
        const uint8_t *wb = l_blob + (w_off0 + (l_mat ? w_d : 0u) + row0 * row_bytes);
        const uint8_t *sb = l_blob + (s_off0 + (l_mat ? s_d : 0u) + row0 * sb_bytes);
        const uint8_t *bb = l_blob + (b_off0 + (l_mat ? b_d : 0u) + row0 * sb_bytes);
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
    int pair_next = 0;              // pair id of this lane's position (divided by K when used)
    int out_pairs_next[8];          // DOWN: pair ids of the eight positions this lane stores
#pragma unroll
    for (int i = 0; i < 8; i++) out_pairs_next[i] = 0;
    if (t0 < t1) {
        item_next = a.items[t0 / n_steps];
        if constexpr (DOWN) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int tok = 8 * (i / 4) + 4 * hh + (i % 4);
                if (tok < item_next.count) out_pairs_next[i] = a.sorted[item_next.start + tok];
            }
        } else if constexpr (!DTENSOR) {
            if ((n & 15) < item_next.count) pair_next = a.sorted[item_next.start + (n & 15)];
        }
    }
    for (int t = t0; t < t1;) {
        const int it = t / n_steps, s_begin = t - it * n_steps;
        const int s_end = t1 - t < n_steps - s_begin ? s_begin + (t1 - t) : n_steps;
        t += s_end - s_begin;
        const PfItem item = item_next;
        int out_pairs[8];
#pragma unroll
        for (int i = 0; i < 8; i++) out_pairs[i] = out_pairs_next[i];
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
                const size_t m = !on ? 0 : DOWN || DTENSOR ? (size_t)(item.start + pos) : (size_t)(pair_next / a.K);
                const int ng = in_dim / 64;
                const uint4 *src = (DOWN ? a.aop : a.xop) + (m * ng + GPW * slab) * 16 + 2 * hh + piece;
                const float2 *sm = (DOWN ? a.asums : a.xsums) + m * ng + GPW * slab;
#pragma unroll
                for (int gi = 0; gi < GPW; gi++) {
#pragma unroll
                    for (int k = 0; k < 4; k++) A[gi][k] = src[16 * gi + 4 * k];
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
                // the next item has arrived with them: its position row, used at its start
                // (no arithmetic on it here: that would wait for the load now)
                if constexpr (DOWN) {
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const int tok = 8 * (i / 4) + 4 * hh + (i % 4);
                        out_pairs_next[i] = 0;
                        if (more && tok < item_next.count) out_pairs_next[i] = a.sorted[item_next.start + tok];
                    }
                } else if constexpr (!DTENSOR) {
                    pair_next = 0;
                    if (more && pos < item_next.count) pair_next = a.sorted[item_next.start + pos];
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
                if constexpr (DENSE) {
                    // the two row tiles of the step; later column passes add to the earlier ones
                    if (my_on) {
                        float *o = a.d_out + (size_t)(item.start + my_pos) * a.d_rows + 64 * s + n;
                        const bool add = a.d_pass > 0 || (a.d_flags & FM_ACCUMULATE);
                        o[0] = add ? o[0] + t0 : t0;
                        o[32] = add ? o[32] + t1 : t1;
                    }
                } else if (my_on) {
                    a.act[(size_t)(item.start + my_pos) * a.g.inter + 32 * s + n] = fm_silu_mul(t0, t1);
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
                        if constexpr (DTENSOR) {
                            float *o = a.d_out + (size_t)(item.start + tok) * a.d_rows + row;
                            *o = (a.d_flags & FM_ACCUMULATE) ? *o + v : v;
                        } else {
                            a.eo[(size_t)out_pairs[i] * a.g.hidden + row] = v;
                        }
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
    // workgroup 0 sorts, the rest turn X into operand registers (one thread per position,
    // group and half)
    const int prep_tasks = M * (g->hidden / 64) * 2;
    hipLaunchKernelGGL(fm_pf_sort<BITS>, dim3(1 + (prep_tasks + 1023) / 1024), dim3(1024), 0, st, a);
    const int max_items = g->n_experts + (int)(n / PF_TM);
    // one 8-wave workgroup per CU (LDS: the ring and the partial tiles take all 160 KB; ~220-245
    // registers per lane cap a SIMD at two waves)
    const int grid = max_items < n_cu ? max_items : n_cu;
    constexpr int LDS = PfSlab<BITS>::LDS_BYTES;
    static FmLdsAttr attr_up, attr_down;
    if (!fm_dyn_lds_ready(attr_up, (const void *)fm_pf_gemm<PF_GATE_UP, BITS, FP16>, LDS)) return FM_ERR_HIP;
    if (!fm_dyn_lds_ready(attr_down, (const void *)fm_pf_gemm<PF_DOWN, BITS, FP16>, LDS)) return FM_ERR_HIP;
    hipLaunchKernelGGL((fm_pf_gemm<PF_GATE_UP, BITS, FP16>), dim3(grid), dim3(512), LDS, st, a);
    const int act_tasks = (int)n * (g->inter / 64) * 2;
    hipLaunchKernelGGL(fm_pf_prepare_act<BITS>, dim3((act_tasks + 255) / 256), dim3(256), 0, st, a);
    hipLaunchKernelGGL((fm_pf_gemm<PF_DOWN, BITS, FP16>), dim3(grid), dim3(512), LDS, st, a);
    hipLaunchKernelGGL(fm_pf_combine, dim3(M, (g->hidden + 1023) / 1024), dim3(256), 0, st, a, d_out, flags);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

template <int BITS, bool FP16>
int pf_launch_dense(PfArgs a, int n_cu, bool prepare, hipStream_t st) {
    const int prep_tasks = a.M * (a.d_cols / 64) * 2;
    if (prepare)
        hipLaunchKernelGGL(fm_pf_dense_prep<BITS>, dim3(1 + (prep_tasks + 1023) / 1024), dim3(1024), 0, st, a);
    const long steps = (long)((a.M + PF_TM - 1) / PF_TM) * (a.d_rows / 64);
    const int grid = steps < n_cu ? (int)steps : n_cu;
    constexpr int LDS = PfSlab<BITS>::LDS_BYTES;
    static FmLdsAttr attr;
    if (!fm_dyn_lds_ready(attr, (const void *)fm_pf_gemm<PF_DENSE, BITS, FP16>, LDS)) return FM_ERR_HIP;
    if (a.d_cols == 512) {       // two slabs: the teams of the down product, 256 rows per step
        const long tsteps = (long)((a.M + PF_TM - 1) / PF_TM) * (a.d_rows / 256);
        const int tgrid = tsteps < n_cu ? (int)tsteps : n_cu;
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

}  // namespace

// Dense tensor against M positions on the same matrix-core kernel as the expert products
// (gpu_encode_prefill_matvec, finchmoe/infer.m:3672: the reference runs M matvecs).
extern "C" size_t fm_prefill_dense_ws_bytes(int out_dim, int in_dim, int group_size, int bits, int M) {
    if (!pf_dense_supported(out_dim, in_dim, group_size, bits) || M < 1) return 0;
    return align256(((size_t)M / PF_TM + 1) * sizeof(PfItem)) + 256 +
           align256((size_t)M * (in_dim / 64) * 16 * sizeof(uint4)) +
           align256((size_t)M * (in_dim / 64) * sizeof(float2));
}

extern "C" int fm_launch_prefill_dense(const void *d_W, const void *d_S, const void *d_B, int out_dim,
                                       int in_dim, int group_size, int bits, int scale_fp16,
                                       const float *d_X, int M, float *d_out, void *d_ws,
                                       size_t ws_bytes, int flags, int prepare, int n_cu,
                                       hipStream_t st) {
    const size_t need = fm_prefill_dense_ws_bytes(out_dim, in_dim, group_size, bits, M);
    if (need == 0) return FM_ERR_UNSUPPORTED;
    if (ws_bytes < need) return FM_ERR_ARG;
    char *ws = (char *)d_ws;
    PfArgs a{};
    a.X = d_X;
    a.M = M;
    a.K = 1;
    a.items = (PfItem *)ws;               ws += align256(((size_t)M / PF_TM + 1) * sizeof(PfItem));
    a.n_items = (int *)ws;                ws += 256;
    a.xop = (uint4 *)ws;                  ws += align256((size_t)M * (in_dim / 64) * 16 * sizeof(uint4));
    a.xsums = (float2 *)ws;
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

extern "C" size_t fm_prefill_affine_ws_bytes(const FmExpertGeom *g, int M, int K) {
    if (!pf_supported(g)) return 0;
    size_t n = (size_t)M * K;
    return align256(n * 4) + align256((g->n_experts + n / PF_TM + 1) * sizeof(PfItem)) + 256 +
           align256(n * g->inter * 4) + align256(n * g->hidden * 4) +
           align256((size_t)M * (g->hidden / 64) * 16 * sizeof(uint4)) +
           align256((size_t)M * (g->hidden / 64) * sizeof(float2)) +
           align256(n * (g->inter / 64) * 16 * sizeof(uint4)) +
           align256(n * (g->inter / 64) * sizeof(float2));
}

extern "C" int fm_launch_prefill_affine(const uint8_t *d_layer, const FmExpertGeom *g,
                                        const float *d_X, const int32_t *d_idx, const float *d_w,
                                        int M, int K, float *d_out, void *d_ws, size_t ws_bytes,
                                        int flags, int n_cu, hipStream_t st) {
    if (!pf_supported(g)) return FM_ERR_UNSUPPORTED;
    if (ws_bytes < fm_prefill_affine_ws_bytes(g, M, K)) return FM_ERR_ARG;
    const size_t n = (size_t)M * K;
    char *ws = (char *)d_ws;
    PfArgs a;
    a.layer = d_layer;
    a.g = *g;
    a.X = d_X;
    a.idx = d_idx;
    a.w = d_w;
    a.M = M;
    a.K = K;
    a.sorted = (int *)ws;                 ws += align256(n * 4);
    a.items = (PfItem *)ws;               ws += align256((g->n_experts + n / PF_TM + 1) * sizeof(PfItem));
    a.n_items = (int *)ws;                ws += 256;
    a.act = (float *)ws;                  ws += align256(n * g->inter * 4);
    a.eo = (float *)ws;                   ws += align256(n * g->hidden * 4);
    a.xop = (uint4 *)ws;                  ws += align256((size_t)M * (g->hidden / 64) * 16 * sizeof(uint4));
    a.xsums = (float2 *)ws;               ws += align256((size_t)M * (g->hidden / 64) * sizeof(float2));
    a.aop = (uint4 *)ws;                  ws += align256(n * (g->inter / 64) * 16 * sizeof(uint4));
    a.asums = (float2 *)ws;
    if (g->scale_fp16)
        return g->bits == 3 ? pf_launch<3, true>(a, g, M, d_out, flags, n_cu, st)
                            : pf_launch<4, true>(a, g, M, d_out, flags, n_cu, st);
    return g->bits == 3 ? pf_launch<3, false>(a, g, M, d_out, flags, n_cu, st)
                        : pf_launch<4, false>(a, g, M, d_out, flags, n_cu, st);
}

