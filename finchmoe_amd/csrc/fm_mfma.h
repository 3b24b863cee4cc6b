// fm_mfma.h — GEMV inner product on the matrix cores.
//
// Why MFMA for a matrix-VECTOR product: at HBM speed a CU has to consume ~35
// three-bit codes per clock, which leaves the vector ALU under two
// instructions per code — less than extract + convert + FMA.  The matrix core
// takes the multiply-accumulate off the vector ALU, and the unpack that remains
// is one instruction per code:
//
//   * a code q (0..7, or 0..15) placed in the mantissa of a bf16 whose exponent
//     field is that of 1.0 reads as 1 + q * 2^t / 128 — exact, no int->float
//     conversion.  One V_AND_OR_B32 on a suitably aligned 32-bit window of the
//     packed stream yields TWO such bf16 values (low and high half), one
//     V_ALIGNBIT_B32 aligns the window: 2 instructions per 2 codes.
//   * the activation is the other MFMA operand.  To lose nothing against the
//     fp32 reference, x is split into three bf16 pieces x = p0 + p1 + p2
//     (8 + 8 + 8 significant bits, exact); the pieces ride in the otherwise
//     idle M dimension of V_MFMA_F32_4X4X4_16B_BF16, products are exact and the
//     accumulate is fp32.  The power of two a code carries from its mantissa
//     position and the "1 +" are undone exactly: x is pre-multiplied by
//     128 / 2^t and the accumulator starts at -sum(128/2^t * x).
//
// V_MFMA_F32_4X4X4_16B_BF16 computes 16 independent 4x4x4 products, one per
// group of 4 adjacent lanes ("block").  In block b, lane 4b+i supplies
// A[i][0..3], lane 4b+j supplies B[0..3][j] and receives D[0..3][j] in its four
// result registers (verified on gfx950).  Here B = codes: lane j of a block
// owns weight row j of the current 4-row step; A = activation pieces: lane i
// holds piece i (i = 3 is zero); all four lanes of a block cover the same 128
// columns.  So result register i of a lane is the dot product of ITS row with
// piece i, and the row's value is the sum of registers 0..2 — no cross-lane
// traffic until the final sum over the column chunks.
//
// Lane map of a wave step over an [rows, in_dim] matrix, LPR = in_dim/128:
//   j  = lane % 4            row inside a quad
//   ch = (lane / 4) % LPR    128-column chunk
//   rq = lane / (4 * LPR)    row quad; a step covers 64/LPR consecutive rows
// The rows of a step are contiguous in memory, so the wave still reads one
// contiguous run per step.
#pragma once

#include "fm_unpack.h"

#if defined(__HIPCC__)

typedef short fm_s4 __attribute__((ext_vector_type(4)));
typedef float fm_f4 __attribute__((ext_vector_type(4)));

// ---- pairing tables --------------------------------------------------------
// A group of 64 codes becomes 32 bf16 pairs; pair p takes code lo(p) into the low
// half and code hi(p) into the high half of one register.  The two codes must
// sit 16 + (th - tl) bits apart in the packed stream, tl/th in 0..4 being their
// offsets inside the 7-bit mantissas.
//   3-bit: codes 5 apart (15 bits: tl=4, th=3) or 6 apart (18 bits: tl=2, th=4);
//          64 = 4 blocks of 10 (distance 5) + 2 blocks of 12 (distance 6)
//   4-bit: codes 4 apart (16 bits: tl=th=3)
template <int BITS> struct FmPairs;

template <> struct FmPairs<3> {
    static constexpr int GROUP_DWORDS = 6;
    __host__ __device__ static constexpr bool far(int p) { return p >= 20; }
    __host__ __device__ static constexpr int lo(int p) {
        return far(p) ? 40 + 12 * ((p - 20) / 6) + (p - 20) % 6 : 10 * (p / 5) + p % 5;
    }
    __host__ __device__ static constexpr int hi(int p) { return lo(p) + (far(p) ? 6 : 5); }
    __host__ __device__ static constexpr int tl(int p) { return far(p) ? 2 : 4; }
    __host__ __device__ static constexpr int th(int p) { return far(p) ? 4 : 3; }
    // first stream bit of the 32-bit window (may be negative: zeros below bit 0)
    __host__ __device__ static constexpr int start(int p) { return 3 * lo(p) - tl(p); }
    __host__ __device__ static constexpr uint32_t mask(int p) {
        return (7u << tl(p)) | (7u << (16 + th(p)));
    }
};

template <> struct FmPairs<4> {
    static constexpr int GROUP_DWORDS = 8;
    __host__ __device__ static constexpr int lo(int p) { return 8 * (p / 4) + p % 4; }
    __host__ __device__ static constexpr int hi(int p) { return lo(p) + 4; }
    __host__ __device__ static constexpr int tl(int) { return 3; }
    __host__ __device__ static constexpr int th(int) { return 3; }
    __host__ __device__ static constexpr int start(int p) { return 4 * lo(p) - 3; }
    __host__ __device__ static constexpr uint32_t mask(int) { return 0x00780078u; }
};

// factor folded into x for the code in the low / high half of pair p
template <int BITS>
__host__ __device__ constexpr float fm_pair_scale_lo(int p) {
    return (float)(128 >> FmPairs<BITS>::tl(p));
}
template <int BITS>
__host__ __device__ constexpr float fm_pair_scale_hi(int p) {
    return (float)(128 >> FmPairs<BITS>::th(p));
}

// 32-bit window of a group's packed words starting at stream bit S
template <int S, int ND>
__device__ __forceinline__ uint32_t fm_window(const uint32_t *g) {
    if constexpr (S < 0) {
        return g[0] << (-S);
    } else {
        constexpr int wd = S >> 5, sh = S & 31;
        if constexpr (sh == 0) return g[wd];
        else if constexpr (wd + 1 >= ND) return g[wd] >> sh;
        else return __builtin_amdgcn_alignbit(g[wd + 1], g[wd], sh);
    }
}

// pair P of a group as two bf16 values 1 + q * 2^t / 128
// `ones` = 0x3F803F80 held in a vector register: V_AND_OR_B32 has no room for
// two literals, with the constant in a register the mask can come from an SGPR
template <int BITS, int P>
__device__ __forceinline__ uint32_t fm_pair(const uint32_t *g, uint32_t ones) {
    using T = FmPairs<BITS>;
    uint32_t w = fm_window<T::start(P), T::GROUP_DWORDS>(g);
    return (w & T::mask(P)) | ones;   // v_and_or_b32
}

// One group (64 codes) of one row against the lane's activation registers:
// 16 MFMAs, each taking two pairs.  acc register i accumulates piece i.
template <int BITS, int M>
__device__ __forceinline__ void fm_group_mfma_steps(const uint32_t *g, const uint32_t *a,
                                                    uint32_t ones, fm_f4 &acc) {
    if constexpr (M < 16) {
        uint32_t b0 = fm_pair<BITS, 2 * M>(g, ones), b1 = fm_pair<BITS, 2 * M + 1>(g, ones);
        fm_s4 bv = __builtin_bit_cast(fm_s4, make_uint2(b0, b1));
        fm_s4 av = __builtin_bit_cast(fm_s4, make_uint2(a[2 * M], a[2 * M + 1]));
        acc = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av, bv, acc, 0, 0, 0);
        fm_group_mfma_steps<BITS, M + 1>(g, a, ones, acc);
    }
}

// Per-lane activation state for one 128-column chunk.
struct FmActRegs {
    uint32_t a[64];   // [32 * group + pair]: bf16 pairs of this lane's piece
    float xsum[2];    // plain sum of x over each group
    float xoff[2];    // sum of scale_k * x_k over each group (what the "1 +" adds)
    uint32_t ones;    // bf16 pair (1.0, 1.0), kept in a register for V_AND_OR_B32
};

// bf16 piece `piece` (0, 1, 2; 3 -> zero) of v: truncations of the running remainder
__device__ __forceinline__ uint32_t fm_bf16_piece(float v, int piece) {
    float r = v;
    float t0 = __uint_as_float(__float_as_uint(r) & 0xFFFF0000u);
    if (piece >= 1) r -= t0;
    float t1 = __uint_as_float(__float_as_uint(r) & 0xFFFF0000u);
    if (piece >= 2) r -= t1;
    uint32_t bits = __float_as_uint(r) >> 16;
    return piece >= 3 ? 0u : bits;
}

// LDS image of the activation registers of every (chunk, piece) of one input
// vector, built once per workgroup and read by all its waves.
//   a   [16][4*LPR] uint4 : register quad q of entry e = 4*chunk + piece (lane-major,
//                           so a wave's read of one quad is conflict free)
//   sum [LPR] float4      : xsum0, xsum1, xoff0, xoff1 of each chunk
template <int LPR>
struct FmActLds {
    uint4 a[16][4 * LPR];
    float4 sum[LPR];
};

// What one thread contributes to the image: register slot w = tid % 64 (group
// w/32, pair w%32) of chunks tid/64, tid/64 + 4, ...  The slot's two columns
// and their scales depend on w only, so they are computed once per kernel.
template <int BITS>
struct FmBuildSlot {
    int lo, hi;          // column offsets inside the 128-column chunk
    float slo, shi;      // 128 / 2^t of the two codes
    __device__ __forceinline__ void init() {
        using T = FmPairs<BITS>;
        const int w = threadIdx.x & 63, G = w >> 5, P = w & 31;
        lo = 64 * G + T::lo(P);
        hi = 64 * G + T::hi(P);
        slo = fm_pair_scale_lo<BITS>(P);
        shi = fm_pair_scale_hi<BITS>(P);
    }
};

// The image is built by the first 256 threads of the workgroup in two steps, so
// that the loads can be issued long before the values are needed:
//   fm_act_load : this thread's activations -> registers (x = the 128*LPR
//                 activations in global memory)
//   fm_act_build: registers -> image.  The caller puts a barrier before the
//                 image's previous readers are done and after (image complete).
// SHARED: x was written earlier in this launch or by another CU's kernel and is
// read with device-scope loads.
template <int LPR>
struct FmActX {
    static constexpr int NIT = (LPR + 3) / 4;     // chunks per thread
    float xl[NIT], xh[NIT];
};

template <int BITS, int LPR, bool SHARED>
__device__ __forceinline__ void fm_act_load(const float *x, const FmBuildSlot<BITS> &bs,
                                            FmActX<LPR> &r) {
    auto ld = [](const float *p) {
        if constexpr (SHARED)
            return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else
            return *p;
    };
#pragma unroll
    for (int i = 0; i < FmActX<LPR>::NIT; i++) {
        const int ch = (threadIdx.x >> 6) + 4 * i;
        const bool on = ch < LPR;
        r.xl[i] = on ? ld(x + ch * FM_CPL + bs.lo) : 0.0f;
        r.xh[i] = on ? ld(x + ch * FM_CPL + bs.hi) : 0.0f;
    }
}

template <int BITS, int LPR>
__device__ __forceinline__ void fm_act_build(const FmActX<LPR> &r, const FmBuildSlot<BITS> &bs,
                                             FmActLds<LPR> &L) {
    constexpr int NE = 4 * LPR;
    constexpr int NIT = FmActX<LPR>::NIT;
    const int w = threadIdx.x & 63;
    const float *xl = r.xl, *xh = r.xh;
    uint32_t *flat = reinterpret_cast<uint32_t *>(L.a);
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int ch = (threadIdx.x >> 6) + 4 * i;
        // exact three-way split of scale*x into bf16 pieces (truncations of the
        // running remainder); the two columns share a register: low | high << 16
        float vl = xl[i] * bs.slo, vh = xh[i] * bs.shi;
        uint32_t l0 = __float_as_uint(vl) & 0xFFFF0000u, h0 = __float_as_uint(vh) & 0xFFFF0000u;
        float rl = vl - __uint_as_float(l0), rh = vh - __uint_as_float(h0);
        uint32_t l1 = __float_as_uint(rl) & 0xFFFF0000u, h1 = __float_as_uint(rh) & 0xFFFF0000u;
        rl -= __uint_as_float(l1);
        rh -= __uint_as_float(h1);
        uint32_t l2 = __float_as_uint(rl), h2 = __float_as_uint(rh) & 0xFFFF0000u;
        if (ch < LPR) {
            uint32_t *dst = flat + ((w >> 2) * NE + 4 * ch) * 4 + (w & 3);
            dst[0] = (l0 >> 16) | h0;
            dst[4] = (l1 >> 16) | h1;
            dst[8] = (l2 >> 16) | h2;
            dst[12] = 0u;
        }
        // sums over the 32 slots of a group: lanes 0..31 / 32..63 of the wave
        float xs = fm_group_sum<32>(xl[i] + xh[i]);
        float xo = fm_group_sum<32>(vl + vh);
        if (ch < LPR && (w & 31) == 0) {
            float *sp = reinterpret_cast<float *>(&L.sum[ch]);
            sp[w >> 5] = xs;
            sp[2 + (w >> 5)] = xo;
        }
    }
}

// lane = lane id in the wave; its entry is (lane % (4*LPR))
template <int LPR>
__device__ __forceinline__ void fm_read_act_lds(const FmActLds<LPR> &L, int lane, FmActRegs &ar) {
    constexpr int NE = 4 * LPR;
    const int e = lane % NE;
#pragma unroll
    for (int q = 0; q < 16; q++) {
        uint4 v = L.a[q][e];
        ar.a[4 * q + 0] = v.x;
        ar.a[4 * q + 1] = v.y;
        ar.a[4 * q + 2] = v.z;
        ar.a[4 * q + 3] = v.w;
    }
    float4 sm = L.sum[e >> 2];
    ar.xsum[0] = sm.x;
    ar.xsum[1] = sm.y;
    ar.xoff[0] = sm.z;
    ar.xoff[1] = sm.w;
    ar.ones = fm_opaque(0x3F803F80u);
}

// dot product of the lane's 128 codes of one row with the activation, scale and
// bias applied: s0*sum(q x) + b0*sum(x) over group 0, same for group 1
template <int BITS, bool FP16>
__device__ __forceinline__ float fm_lane_dot_mfma(const FmRowSlice<BITS> &rs,
                                                  const FmActRegs &ar) {
    constexpr int GD = FmPairs<BITS>::GROUP_DWORDS;
    const uint32_t *d = reinterpret_cast<const uint32_t *>(rs.q);
    fm_f4 acc0 = {-ar.xoff[0], 0.0f, 0.0f, 0.0f};
    fm_f4 acc1 = {-ar.xoff[1], 0.0f, 0.0f, 0.0f};
    fm_group_mfma_steps<BITS, 0>(d, ar.a, ar.ones, acc0);
    fm_group_mfma_steps<BITS, 0>(d + GD, ar.a + 32, ar.ones, acc1);
    float d0 = (acc0[0] + acc0[1]) + acc0[2];
    float d1 = (acc1[0] + acc1[1]) + acc1[2];
    float r = fm_widen_lo<FP16>(rs.s) * d0;
    r = fmaf(fm_widen_lo<FP16>(rs.b), ar.xsum[0], r);
    r = fmaf(fm_widen_hi<FP16>(rs.s), d1, r);
    r = fmaf(fm_widen_hi<FP16>(rs.b), ar.xsum[1], r);
    return r;
}

// sum over the LPR column chunks of a row: lanes 4 apart inside a row quad
template <int LPR>
__device__ __forceinline__ float fm_chunk_sum(float v) {
    // LPR == 2: only the chunk-0 lanes need the sum (they store it)
    if constexpr (LPR == 2) v += fm_dpp<0x104>(v);   // row_shl:4: lane i <- lane i+4
    if constexpr (LPR >= 4) v += fm_dpp<0x124>(v);   // row_ror:4
    if constexpr (LPR >= 4) v += fm_dpp<0x128>(v);   // row_ror:8
    if constexpr (LPR >= 8) v += __shfl_xor(v, 16);
    if constexpr (LPR >= 16) v += __shfl_xor(v, 32);
    return v;
}

#endif  // __HIPCC__
