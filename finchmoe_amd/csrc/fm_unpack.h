// fm_unpack.h — per-lane unpack + dot of affine-packed codes (3-bit triplets,
// 4-bit nibbles, 8-bit bytes) for the GEMV kernels.
//
// A lane owns FM_CPL = 128 consecutive input columns of one weight row: two
// quantization groups of 64.  That is 48 bytes of 3-bit codes or 64 bytes of
// 4-bit codes, fetched as three / four 128-bit loads.  The lane keeps the 128
// matching activations in registers for every row it visits.
//
// Arithmetic.  The reference evaluates sum_j ((float)q_j*s + b) * x_j per row
// (finchmoe/infer.m:1716-1727, 1745-1759).  Here each group contributes
// s * sum_j q_j x_j + b * sum_j x_j, with sum_j x_j computed once per lane: the
// same value up to fp32 reassociation, at one FMA per code instead of two.
//
// Unpack cost.  The VALU budget at HBM speed is about two instructions per
// code, so extract+convert must be cheaper than the usual bfe + cvt pair:
// v_cvt_f32_ubyteN converts one byte of a register to float in one
// instruction, so the codes are isolated one per byte with a handful of AND
// masks shared by many codes, and the power-of-two factor a code carries from
// its position inside the byte (q << t) is folded into the activation
// (x_j * 2^-t, exact).
//   4-bit: w & 0x0F0F0F0F holds nibbles 0,2,4,6 (t=0); w & 0xF0F0F0F0 holds
//          nibbles 1,3,5,7 (t=4).  2 ANDs per 8 codes.
//   3-bit: in a 96-bit run (32 codes, 12 bytes) code i starts at bit 3i, i.e.
//          at in-byte offset t = 3i mod 8.  t in {0,1,2} -> mask set A,
//          t in {3,4,5} -> set B (each byte holds one A and one B code);
//          t in {6,7} straddles a byte edge -> taken from the run shifted right
//          by two bits (set C, t becomes 4 or 5).  9 ANDs + 3 shifts per 32
//          codes.
#pragma once

#include "fm_common.h"

#define FM_CPL 128   // columns per lane

#if defined(__HIPCC__)

// ---- 3-bit position tables (compile-time) --------------------------------
// code i (0..31) of a 96-bit run
__host__ __device__ constexpr int fm3_set(int i) {   // 0 = A, 1 = B, 2 = C
    int t = (3 * i) & 7;
    return t <= 2 ? 0 : (t <= 5 ? 1 : 2);
}
__host__ __device__ constexpr int fm3_bit(int i) {   // start bit in the (shifted) run
    return fm3_set(i) == 2 ? 3 * i - 2 : 3 * i;
}
__host__ __device__ constexpr int fm3_word(int i) { return fm3_bit(i) >> 5; }
__host__ __device__ constexpr int fm3_byte(int i) { return (fm3_bit(i) >> 3) & 3; }
__host__ __device__ constexpr int fm3_t(int i) { return fm3_bit(i) & 7; }
__host__ __device__ constexpr uint32_t fm3_mask(int set, int word) {
    uint32_t m = 0;
    for (int i = 0; i < 32; i++)
        if (fm3_set(i) == set && fm3_word(i) == word) m |= 7u << (fm3_bit(i) & 31);
    return m;
}

// in-byte shift carried by column j of a lane's 128 columns
template <int BITS>
__host__ __device__ constexpr int fm_col_shift(int j) {
    if (BITS == 3) return fm3_t(j & 31);
    if (BITS == 8) return 0;
    return (j & 1) ? 4 : 0;
}

typedef uint32_t fm_u4 __attribute__((ext_vector_type(4)));

template <int BITS> struct FmLaneBytes;
template <> struct FmLaneBytes<3> { static constexpr int value = 48; };
template <> struct FmLaneBytes<4> { static constexpr int value = 64; };
template <> struct FmLaneBytes<8> { static constexpr int value = 128; };

// One lane's slice of one weight row: packed codes + the 16-bit scale and bias
// pairs of its two groups.
template <int BITS>
struct FmRowSlice {
    static constexpr int NQ = FmLaneBytes<BITS>::value / 16;
    fm_u4 q[NQ];
    uint32_t s, b;
};

template <int BITS>
__device__ __forceinline__ void fm_load_slice(FmRowSlice<BITS> &rs, const uint8_t *w,
                                              const uint8_t *s, const uint8_t *b) {
    // weights always live in device memory: say so, or a pointer that passed
    // through LDS is loaded with FLAT instructions, which also count as LDS
    // traffic and stall the compute on the prefetch
    typedef const __attribute__((address_space(1))) fm_u4 *gq_t;
    typedef const __attribute__((address_space(1))) uint32_t *gd_t;
    gq_t wp = (gq_t)(uintptr_t)w;
#pragma unroll
    for (int i = 0; i < FmRowSlice<BITS>::NQ; i++) rs.q[i] = wp[i];
    rs.s = *(gd_t)(uintptr_t)s;
    rs.b = *(gd_t)(uintptr_t)b;
}

// float of byte BYTE of v (v_cvt_f32_ubyteN).  The callers hide their masked
// words from the optimizer (fm_opaque): otherwise the shift below is
// re-associated with the caller's AND mask and every code costs an extra
// byte-select instruction.
__device__ __forceinline__ uint32_t fm_opaque(uint32_t v) {
    asm("" : "+v"(v));
    return v;
}
template <int BYTE>
__device__ __forceinline__ float fm_ubyte(uint32_t v) {
    return (float)((v >> (8 * BYTE)) & 0xFFu);
}

template <int I>
__device__ __forceinline__ void fm_dot32_3bit_terms(const uint32_t (&m)[3][3], const float *xs,
                                                    float &acc0, float &acc1) {
    if constexpr (I < 32) {
        float q = fm_ubyte<fm3_byte(I)>(m[fm3_set(I)][fm3_word(I)]);
        if constexpr (I & 1) acc1 = fmaf(q, xs[I], acc1);
        else acc0 = fmaf(q, xs[I], acc0);
        fm_dot32_3bit_terms<I + 1>(m, xs, acc0, acc1);
    }
}

// sum over 32 codes of (q << t) * xs, xs already scaled by 2^-t
__device__ __forceinline__ void fm_dot32_3bit(uint32_t d0, uint32_t d1, uint32_t d2,
                                              const float *xs, float &acc0, float &acc1) {
    uint32_t m[3][3];
    m[0][0] = d0 & fm3_mask(0, 0); m[0][1] = d1 & fm3_mask(0, 1); m[0][2] = d2 & fm3_mask(0, 2);
    m[1][0] = d0 & fm3_mask(1, 0); m[1][1] = d1 & fm3_mask(1, 1); m[1][2] = d2 & fm3_mask(1, 2);
    uint32_t s0 = __builtin_amdgcn_alignbit(d1, d0, 2);
    uint32_t s1 = __builtin_amdgcn_alignbit(d2, d1, 2);
    uint32_t s2 = d2 >> 2;
    m[2][0] = s0 & fm3_mask(2, 0); m[2][1] = s1 & fm3_mask(2, 1); m[2][2] = s2 & fm3_mask(2, 2);
#pragma unroll
    for (int a = 0; a < 3; a++)
#pragma unroll
        for (int b = 0; b < 3; b++) m[a][b] = fm_opaque(m[a][b]);
    fm_dot32_3bit_terms<0>(m, xs, acc0, acc1);
}

// sum over 8 codes of one 4-bit word
__device__ __forceinline__ void fm_dot8_4bit(uint32_t w, const float *xs, float &acc0,
                                             float &acc1) {
    uint32_t lo = fm_opaque(w & 0x0F0F0F0Fu), hi = fm_opaque(w & 0xF0F0F0F0u);
    acc0 = fmaf(fm_ubyte<0>(lo), xs[0], acc0);
    acc1 = fmaf(fm_ubyte<0>(hi), xs[1], acc1);
    acc0 = fmaf(fm_ubyte<1>(lo), xs[2], acc0);
    acc1 = fmaf(fm_ubyte<1>(hi), xs[3], acc1);
    acc0 = fmaf(fm_ubyte<2>(lo), xs[4], acc0);
    acc1 = fmaf(fm_ubyte<2>(hi), xs[5], acc1);
    acc0 = fmaf(fm_ubyte<3>(lo), xs[6], acc0);
    acc1 = fmaf(fm_ubyte<3>(hi), xs[7], acc1);
}

// sum_j q_j x_j over one group (64 codes); g = 0 or 1 selects the lane's group
template <int BITS, int G>
__device__ __forceinline__ float fm_group_dot(const FmRowSlice<BITS> &rs, const float *xs) {
    const uint32_t *d = reinterpret_cast<const uint32_t *>(rs.q);
    float a0 = 0.0f, a1 = 0.0f;
    if constexpr (BITS == 3) {
        fm_dot32_3bit(d[6 * G + 0], d[6 * G + 1], d[6 * G + 2], xs + 64 * G, a0, a1);
        fm_dot32_3bit(d[6 * G + 3], d[6 * G + 4], d[6 * G + 5], xs + 64 * G + 32, a0, a1);
    } else if constexpr (BITS == 4) {
#pragma unroll
        for (int k = 0; k < 8; k++) fm_dot8_4bit(d[8 * G + k], xs + 64 * G + 8 * k, a0, a1);
    } else {   // 8-bit: four codes per word, one per byte (quantize_model.py:35-43)
#pragma unroll
        for (int k = 0; k < 16; k++) {
            uint32_t w = d[16 * G + k];
            const float *xp = xs + 64 * G + 4 * k;
            a0 = fmaf(fm_ubyte<0>(w), xp[0], a0);
            a1 = fmaf(fm_ubyte<1>(w), xp[1], a1);
            a0 = fmaf(fm_ubyte<2>(w), xp[2], a0);
            a1 = fmaf(fm_ubyte<3>(w), xp[3], a1);
        }
    }
    return a0 + a1;
}

// the lane's contribution to its row: two groups, scale and bias applied
template <int BITS, bool FP16>
__device__ __forceinline__ float fm_lane_dot(const FmRowSlice<BITS> &rs, const float *xs,
                                             float xsum0, float xsum1) {
    float d0 = fm_group_dot<BITS, 0>(rs, xs);
    float d1 = fm_group_dot<BITS, 1>(rs, xs);
    float r = fm_widen_lo<FP16>(rs.s) * d0;
    r = fmaf(fm_widen_lo<FP16>(rs.b), xsum0, r);
    r = fmaf(fm_widen_hi<FP16>(rs.s), d1, r);
    r = fmaf(fm_widen_hi<FP16>(rs.b), xsum1, r);
    return r;
}

// Load the lane's 128 activations, pre-scaled per column; xsum0/1 = plain sums
// of the two groups.
template <int BITS>
__device__ __forceinline__ void fm_load_x(const float *x, float *xs, float &xsum0,
                                          float &xsum1) {
    const float4 *xp = reinterpret_cast<const float4 *>(x);
    float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
    for (int i = 0; i < FM_CPL / 4; i++) {
        float4 v = xp[i];
        float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            int j = 4 * i + k;
            if (j < 64) s0 += e[k]; else s1 += e[k];
            xs[j] = e[k] * (1.0f / (float)(1 << fm_col_shift<BITS>(j)));
        }
    }
    xsum0 = s0;
    xsum1 = s1;
}

#endif  // __HIPCC__
