// fm_gguf.hip — routed-expert decode and single matvec for GGUF Q4_K / Q6_K
// block formats.  Replaces fused_gate_up_swiglu_qk + dequant_matvec_qk as driven
// by gpu_gguf_experts_forward (finchmoe/infer.m:3153-3347; kernels
// finchmoe/shaders.metal:3216-3365) and their per-position pool variants
// (shaders.metal:3460-3517, 3641-3712).
//
// Block formats (finchmoe/infer.m:1604-1657):
//   Q4_K  144 B / 256 values: d, dmin fp16 | 12 B of 6-bit (scale, min) x 8 |
//         128 B nibbles; 64-value chunk c = 32 bytes, low nibbles are values
//         0..31 (scale pair 2c), high nibbles values 32..63 (pair 2c+1);
//         y = d*sc*q - dmin*m
//   Q6_K  210 B / 256 values: ql 128 B | qh 64 B | int8 scales x 16 | d fp16;
//         per 128-value half: q = (ql nibble | qh 2 bits << 4) - 32,
//         y = d*sc[v/16]*q
//
// Two sets of kernels.  Shapes with 4, 8 or 16 lanes per row take the streaming
// kernels further down (LDS ring + matrix cores); every other shape, and the
// single matvec, take the plain kernels described next.
//
// Lane map.  A lane owns one 128-value HALF block of one row (its 128
// activations live in registers), LPR = in_dim/128 adjacent lanes share a row,
// a wave step covers 64/LPR consecutive rows.  Per row the lane contributes
//   Q4_K: sum_j d*sc_j * (sum q x)_j - dmin*m_j * (sum x)_j   over its 4 sub-blocks
//   Q6_K: sum_g d*sc_g * ((sum q6 x)_g - 32 * (sum x)_g)      over its 8 groups
// which is the reference's sum of y*x up to fp32 reassociation.  Codes are
// converted with V_CVT_F32_UBYTEn after being isolated one per byte by AND
// masks (fm_unpack.h explains the trick); the 16x a high nibble carries is
// folded into the activation.
//
// Q6_K blocks are only 2-byte aligned (210 = 2 mod 4).  The loads below are
// plain multi-dword loads at that alignment, which gfx950 serves in its
// unaligned-access mode.
#include "fm_index.h"
#include "fm_mfma.h"
#include "fm_ring.h"

#include <stdlib.h>

namespace {

struct GgufArgs {
    const uint8_t *const *gate, *const *up, *const *down;   // [n_layers] slab base pointers
    FmGgufGeom g;
    int layer0, layer_stride, K;
    const float *x;
    const int32_t *idx;
    const float *w;
    float *act, *expert_out, *out;
    int rows_per_item, items_per_pair, flags;
    // one dense tensor instead of an expert store (fm_launch_gguf_dense): its rows start here,
    // there is one "pair", and the index and pointer tables are not read
    const uint8_t *direct;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) uint8_t *gptr;

// loads at 2-byte alignment
struct __attribute__((packed, aligned(2))) U4a2 { u32x4 v; };
struct __attribute__((packed, aligned(2))) U2a2 { u32x2 v; };
struct __attribute__((packed, aligned(2))) U1a2 { uint32_t v; };

__device__ __forceinline__ float f16bits(uint32_t h) { return fm_fp16_bits(h & 0xFFFFu); }

// ---------------------------------------------------------------- Q4_K half block
struct Q4Half {
    u32x4 hdr;      // d | dmin, scales[0..3], scales[4..7], scales[8..11]
    u32x4 q[4];     // 64 bytes of nibbles: two 64-value chunks
};

__device__ __forceinline__ void q4_load(Q4Half &t, const uint8_t *block, int half) {
    gptr p = (gptr)(uintptr_t)block;
    t.hdr = *(const __attribute__((address_space(1))) u32x4 *)p;
    const __attribute__((address_space(1))) u32x4 *q =
        (const __attribute__((address_space(1))) u32x4 *)(p + 16 + 64 * half);
#pragma unroll
    for (int i = 0; i < 4; i++) t.q[i] = q[i];
}

// (scale, min) pair j = 4*half + jj of the 12 scale bytes (finchmoe/infer.m:1595-1603)
__device__ __forceinline__ void q4_scale_min(const u32x4 &hdr, int half, int jj, float &sc,
                                             float &mn) {
    const uint32_t s0 = hdr[1], s1 = hdr[2], s2 = hdr[3];
    uint32_t a = (s0 >> (8 * jj)) & 0xFFu, b = (s1 >> (8 * jj)) & 0xFFu, c = (s2 >> (8 * jj)) & 0xFFu;
    uint32_t sc_lo = a & 63u, mn_lo = b & 63u;                       // j < 4
    uint32_t sc_hi = (c & 0xFu) | ((a >> 6) << 4), mn_hi = (c >> 4) | ((b >> 6) << 4);   // j >= 4
    sc = (float)(half ? sc_hi : sc_lo);
    mn = (float)(half ? mn_hi : mn_lo);
}

// xs: the lane's 128 activations, high-nibble positions pre-divided by 16;
// xsum[j]: plain sum of the 32 activations of sub-block j
__device__ __forceinline__ float q4_half_dot(const Q4Half &t, int half, const float *xs,
                                             const float *xsum) {
    const float d = f16bits(t.hdr[0]), dmin = f16bits(t.hdr[0] >> 16);
    const uint32_t *qd = reinterpret_cast<const uint32_t *>(t.q);
    float r = 0.0f;
#pragma unroll
    for (int c = 0; c < 2; c++) {
        float e0 = 0.0f, e1 = 0.0f, o0 = 0.0f, o1 = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            uint32_t w = qd[8 * c + k];
            uint32_t lo = fm_opaque(w & 0x0F0F0F0Fu), hi = fm_opaque(w & 0xF0F0F0F0u);
            const float *xe = xs + 64 * c + 4 * k, *xo = xe + 32;
            e0 = fmaf(fm_ubyte<0>(lo), xe[0], e0);
            e1 = fmaf(fm_ubyte<1>(lo), xe[1], e1);
            e0 = fmaf(fm_ubyte<2>(lo), xe[2], e0);
            e1 = fmaf(fm_ubyte<3>(lo), xe[3], e1);
            o0 = fmaf(fm_ubyte<0>(hi), xo[0], o0);
            o1 = fmaf(fm_ubyte<1>(hi), xo[1], o1);
            o0 = fmaf(fm_ubyte<2>(hi), xo[2], o0);
            o1 = fmaf(fm_ubyte<3>(hi), xo[3], o1);
        }
        float sc, mn;
        q4_scale_min(t.hdr, half, 2 * c, sc, mn);
        r = fmaf(d * sc, e0 + e1, r);
        r = fmaf(-(dmin * mn), xsum[2 * c], r);
        q4_scale_min(t.hdr, half, 2 * c + 1, sc, mn);
        r = fmaf(d * sc, o0 + o1, r);
        r = fmaf(-(dmin * mn), xsum[2 * c + 1], r);
    }
    return r;
}

__device__ __forceinline__ void q4_load_x(const float *x, float *xs, float *xsum) {
    const float4 *xp = reinterpret_cast<const float4 *>(x);
#pragma unroll
    for (int j = 0; j < 4; j++) xsum[j] = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        float4 v = xp[i];
        float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int col = 4 * i + k;
            xsum[col >> 5] += e[k];
            xs[col] = ((col >> 5) & 1) ? e[k] * 0.0625f : e[k];
        }
    }
}

// ---------------------------------------------------------------- Q6_K half block
struct Q6Half {
    u32x4 ql[4];    // 64 bytes
    u32x4 qh[2];    // 32 bytes
    u32x2 sc;       // 8 int8 scales
    uint32_t d;     // fp16 in the low half
};

__device__ __forceinline__ void q6_load(Q6Half &t, const uint8_t *block, int half) {
    gptr p = (gptr)(uintptr_t)block;
    const __attribute__((address_space(1))) U4a2 *ql =
        (const __attribute__((address_space(1))) U4a2 *)(p + 64 * half);
    const __attribute__((address_space(1))) U4a2 *qh =
        (const __attribute__((address_space(1))) U4a2 *)(p + 128 + 32 * half);
#pragma unroll
    for (int i = 0; i < 4; i++) t.ql[i] = ql[i].v;
    t.qh[0] = qh[0].v;
    t.qh[1] = qh[1].v;
    t.sc = ((const __attribute__((address_space(1))) U2a2 *)(p + 192 + 8 * half))->v;
    t.d = *(const __attribute__((address_space(1))) uint16_t *)(p + 208);
}

// xs: the lane's 128 activations; xsum[g]: sum over the 16 activations of group g
__device__ __forceinline__ float q6_half_dot(const Q6Half &t, const float *xs, const float *xsum) {
    const float d = f16bits(t.d);
    const uint32_t *ql = reinterpret_cast<const uint32_t *>(t.ql);
    const uint32_t *qh = reinterpret_cast<const uint32_t *>(t.qh);
    float acc[8];
#pragma unroll
    for (int g = 0; g < 8; g++) acc[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t a = ql[i], b = ql[8 + i], h = qh[i];
        // four 6-bit codes per register, one per byte (finchmoe/infer.m:1643-1646)
        uint32_t q1 = fm_opaque((a & 0x0F0F0F0Fu) | ((h & 0x03030303u) << 4));
        uint32_t q2 = fm_opaque((b & 0x0F0F0F0Fu) | ((h & 0x0C0C0C0Cu) << 2));
        uint32_t q3 = fm_opaque(((a >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u));
        uint32_t q4 = fm_opaque(((b >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u));
        const float *x1 = xs + 4 * i;
        const int g1 = i >> 2;   // values 4i..4i+3 -> scale group (4i)/16
        acc[g1] = fmaf(fm_ubyte<0>(q1), x1[0], acc[g1]);
        acc[g1] = fmaf(fm_ubyte<1>(q1), x1[1], acc[g1]);
        acc[g1] = fmaf(fm_ubyte<2>(q1), x1[2], acc[g1]);
        acc[g1] = fmaf(fm_ubyte<3>(q1), x1[3], acc[g1]);
        acc[g1 + 2] = fmaf(fm_ubyte<0>(q2), x1[32], acc[g1 + 2]);
        acc[g1 + 2] = fmaf(fm_ubyte<1>(q2), x1[33], acc[g1 + 2]);
        acc[g1 + 2] = fmaf(fm_ubyte<2>(q2), x1[34], acc[g1 + 2]);
        acc[g1 + 2] = fmaf(fm_ubyte<3>(q2), x1[35], acc[g1 + 2]);
        acc[g1 + 4] = fmaf(fm_ubyte<0>(q3), x1[64], acc[g1 + 4]);
        acc[g1 + 4] = fmaf(fm_ubyte<1>(q3), x1[65], acc[g1 + 4]);
        acc[g1 + 4] = fmaf(fm_ubyte<2>(q3), x1[66], acc[g1 + 4]);
        acc[g1 + 4] = fmaf(fm_ubyte<3>(q3), x1[67], acc[g1 + 4]);
        acc[g1 + 6] = fmaf(fm_ubyte<0>(q4), x1[96], acc[g1 + 6]);
        acc[g1 + 6] = fmaf(fm_ubyte<1>(q4), x1[97], acc[g1 + 6]);
        acc[g1 + 6] = fmaf(fm_ubyte<2>(q4), x1[98], acc[g1 + 6]);
        acc[g1 + 6] = fmaf(fm_ubyte<3>(q4), x1[99], acc[g1 + 6]);
    }
    float r = 0.0f;
#pragma unroll
    for (int g = 0; g < 8; g++) {
        uint32_t word = t.sc[g >> 2];
        int sc = (int)(int8_t)((word >> (8 * (g & 3))) & 0xFFu);
        r = fmaf(d * (float)sc, fmaf(-32.0f, xsum[g], acc[g]), r);
    }
    return r;
}

__device__ __forceinline__ void q6_load_x(const float *x, float *xs, float *xsum) {
    const float4 *xp = reinterpret_cast<const float4 *>(x);
#pragma unroll
    for (int g = 0; g < 8; g++) xsum[g] = 0.0f;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        float4 v = xp[i];
        float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            xsum[(4 * i + k) >> 4] += e[k];
            xs[4 * i + k] = e[k];
        }
    }
}

// ---------------------------------------------------------------- kernels
__device__ __forceinline__ bool gg_expert(const GgufArgs &a, int pair, int &e) {
    e = a.idx[pair];
    return (unsigned)e < (unsigned)a.g.n_experts;
}

// gate (Q4_K) + up (Q4_K) + SwiGLU
template <int LPR>
__global__ __launch_bounds__(256) void fm_gguf_gate_up(GgufArgs a) {
    constexpr int RPS = FM_WAVE / LPR;
    const int pair = blockIdx.x / a.items_per_pair;
    const int chunk = blockIdx.x - pair * a.items_per_pair;
    const int l = pair / a.K;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane % LPR, r = lane / LPR;
    const int rows_per_wave = a.rows_per_item >> 2;
    const int row0 = chunk * a.rows_per_item + wave * rows_per_wave;
    float *act = a.act + (size_t)pair * a.g.inter;
    int e;
    if (!gg_expert(a, pair, e)) {
        for (int i = lane; i < rows_per_wave; i += FM_WAVE) act[row0 + i] = 0.0f;
        return;
    }
    const int li = a.layer0 + l * a.layer_stride;
    const uint8_t *gw = a.gate[li] + (size_t)e * a.g.gate_slab;
    const uint8_t *uw = a.up[li] + (size_t)e * a.g.up_slab;
    const int half = c & 1;
    size_t off = (size_t)(row0 + r) * a.g.gu_row_bytes + (size_t)(c >> 1) * 144;
    const size_t step = (size_t)RPS * a.g.gu_row_bytes;
    Q4Half gc, uc, gn, un;
    q4_load(gc, gw + off, half);
    q4_load(uc, uw + off, half);
    float xs[128], xsum[4];
    q4_load_x(a.x + (size_t)l * a.g.hidden + c * 128, xs, xsum);
    const int steps = rows_per_wave / RPS;
    for (int it = 0; it < steps; it++) {
        if (it + 1 < steps) {
            off += step;
            q4_load(gn, gw + off, half);
            q4_load(un, uw + off, half);
        }
        float gv = fm_group_sum<LPR>(q4_half_dot(gc, half, xs, xsum));
        float uv = fm_group_sum<LPR>(q4_half_dot(uc, half, xs, xsum));
        if (c == 0) act[row0 + it * RPS + r] = fm_silu_mul(gv, uv);
        gc = gn;
        uc = un;
    }
}

// down (Q6_K or Q4_K) -> per-expert output vectors
template <int LPR, bool Q6>
__global__ __launch_bounds__(256) void fm_gguf_down(GgufArgs a) {
    constexpr int RPS = FM_WAVE / LPR;
    const int pair = blockIdx.x / a.items_per_pair;
    const int chunk = blockIdx.x - pair * a.items_per_pair;
    const int l = pair / a.K;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane % LPR, r = lane / LPR;
    const int rows_per_wave = a.rows_per_item >> 2;
    const int row0 = chunk * a.rows_per_item + wave * rows_per_wave;
    float *eo = a.expert_out + (size_t)pair * a.g.hidden;
    int e;
    if (!gg_expert(a, pair, e)) {
        for (int i = lane; i < rows_per_wave; i += FM_WAVE) eo[row0 + i] = 0.0f;
        return;
    }
    const int li = a.layer0 + l * a.layer_stride;
    const uint8_t *dw = a.down[li] + (size_t)e * a.g.down_slab;
    const int half = c & 1;
    size_t off = (size_t)(row0 + r) * a.g.down_row_bytes + (size_t)(c >> 1) * (Q6 ? 210 : 144);
    const size_t step = (size_t)RPS * a.g.down_row_bytes;
    const float *xv = a.act + (size_t)pair * a.g.inter + c * 128;
    const int steps = rows_per_wave / RPS;
    float xs[128];
    if constexpr (Q6) {
        Q6Half cur, next;
        q6_load(cur, dw + off, half);
        float xsum[8];
        q6_load_x(xv, xs, xsum);
        for (int it = 0; it < steps; it++) {
            if (it + 1 < steps) {
                off += step;
                q6_load(next, dw + off, half);
            }
            float v = fm_group_sum<LPR>(q6_half_dot(cur, xs, xsum));
            if (c == 0) eo[row0 + it * RPS + r] = v;
            cur = next;
        }
    } else {
        Q4Half cur, next;
        q4_load(cur, dw + off, half);
        float xsum[4];
        q4_load_x(xv, xs, xsum);
        for (int it = 0; it < steps; it++) {
            if (it + 1 < steps) {
                off += step;
                q4_load(next, dw + off, half);
            }
            float v = fm_group_sum<LPR>(q4_half_dot(cur, half, xs, xsum));
            if (c == 0) eo[row0 + it * RPS + r] = v;
            cur = next;
        }
    }
}

// out[l][j] = sum_k w[l][k] * expert_out[l][k][j] in slot order; GUARD = the CPU
// combine of finchmoe/infer.m:3334-3347 (finite check + renormalisation)
template <bool GUARD>
__global__ __launch_bounds__(256) void fm_gguf_combine(GgufArgs a) {
    __shared__ float red[4];
    const int l = blockIdx.x, H = a.g.hidden, K = a.K;
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
                    float v = eo[(size_t)k * H + j];
                    part = fmaf(v, v, part);
                }
                part = fm_group_sum<64>(part);
                __syncthreads();
                if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = part;
                __syncthreads();
                float er = red[0] + red[1] + red[2] + red[3];
                if (isfinite(er) && er < 1e20f) total += w; else w = 0.0f;
            }
        }
        wk[k] = w;
    }
    float rn = 1.0f;
    if constexpr (GUARD) {
        if (total > 0.0f && total < 0.99f) rn = 1.0f / total;
    }
    float *out = a.out + (size_t)l * H;
    const int j0 = GUARD ? 0 : blockIdx.y * blockDim.x;
    const int j1 = GUARD ? H : min(H, j0 + (int)blockDim.x);
    for (int j = j0 + threadIdx.x; j < j1; j += blockDim.x) {
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            if (k < K && wk[k] != 0.0f) acc += wk[k] * eo[(size_t)k * H + j];
        if constexpr (GUARD) acc *= rn;
        out[j] = (a.flags & FM_ACCUMULATE) ? out[j] + acc : acc;
    }
}

// single matvec, any out_dim, in_dim a multiple of 256: one wave per row, lanes
// stride over the half blocks (dequant_matvec_qk, finchmoe/shaders.metal:3216-3299)
template <bool Q6>
__global__ __launch_bounds__(256) void fm_gguf_matvec_k(const uint8_t *W, const float *x, float *out,
                                                        int out_dim, int in_dim) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= out_dim) return;
    const int halves = in_dim / 128;
    const size_t row_bytes = (size_t)(in_dim / 256) * (Q6 ? 210 : 144);
    float acc = 0.0f;
    for (int hb = lane; hb < halves; hb += FM_WAVE) {
        const uint8_t *blk = W + (size_t)row * row_bytes + (size_t)(hb >> 1) * (Q6 ? 210 : 144);
        float xs[128];
        if constexpr (Q6) {
            Q6Half t;
            q6_load(t, blk, hb & 1);
            float xsum[8];
            q6_load_x(x + hb * 128, xs, xsum);
            acc += q6_half_dot(t, xs, xsum);
        } else {
            Q4Half t;
            q4_load(t, blk, hb & 1);
            float xsum[4];
            q4_load_x(x + hb * 128, xs, xsum);
            acc += q4_half_dot(t, hb & 1, xs, xsum);
        }
    }
    acc = fm_group_sum<64>(acc);
    if (lane == 0) out[row] = acc;
}

// The same product for rows of HPR <= 64 half blocks (in_dim = 128 * HPR, HPR a power of two): HPR
// adjacent lanes share a row, a wave step covers 64 / HPR rows, and a lane keeps its 128
// activations in registers over the `steps` row steps of its wave — every lane works whatever the
// row length (a vocabulary projection of 2048 columns keeps a quarter of the lanes busy in the
// kernel above).  Rows past out_dim are not loaded and not stored.
template <bool Q6, int HPR>
__global__ __launch_bounds__(256) void fm_gguf_matvec_rows_k(const uint8_t *W, const float *x, float *out,
                                                             int out_dim, int steps) {
    constexpr int RPW = FM_WAVE / HPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int hb = lane % HPR, rr = lane / HPR;
    const size_t row_bytes = (size_t)(HPR / 2) * (Q6 ? 210 : 144);
    float xs[128], xsum[8];
    if constexpr (Q6) q6_load_x(x + hb * 128, xs, xsum);
    else q4_load_x(x + hb * 128, xs, xsum);
    const long row0 = ((long)blockIdx.x * 4 + wave) * RPW * steps;
    for (int s = 0; s < steps; s++) {
        const long row = row0 + (long)s * RPW + rr;
        float acc = 0.0f;
        if (row < out_dim) {
            const uint8_t *blk = W + (size_t)row * row_bytes + (size_t)(hb >> 1) * (Q6 ? 210 : 144);
            if constexpr (Q6) {
                Q6Half t;
                q6_load(t, blk, hb & 1);
                acc = q6_half_dot(t, xs, xsum);
            } else {
                Q4Half t;
                q4_load(t, blk, hb & 1);
                acc = q4_half_dot(t, hb & 1, xs, xsum);
            }
        }
        acc = fm_group_sum<HPR>(acc);
        if (hb == 0 && row < out_dim) out[row] = acc;
    }
}

// ---------------------------------------------------------------- streaming kernels
// The large launches take the form of the affine decode kernels: one workgroup of
// twelve waves per CU (FM_GG_NW), each wave keeps a ring of two slices in LDS filled by LDS-direct
// loads (a slice = the rows of one wave step exactly as they lie in memory, block
// headers included), units are claimed from a counter in LDS, and the multiply
// runs on the matrix cores with the codes placed in bf16 mantissas (fm_mfma.h).
//
// Lane map of a wave step: lane = 4*chunk + row-in-quad as in fm_mfma.h, with
//   Q4_K  chunk = one 128-value half block          (LPR = in_dim / 128)
//   Q6_K  chunk = 64 values: side sd of half hf of a block, i.e. ql bytes
//         [64 hf + 32 sd, +32) — their low nibbles are values 32 sd + v and their
//         high nibbles values 64 + 32 sd + v of the half, v < 32 — with bits
//         2 sd.. and 2 sd + 4.. of qh bytes [32 hf, +32)      (LPR = in_dim / 64)
// so a slice is 4608 B (Q4_K) or 3360 B (Q6_K) whatever the row length.
//
// Codes in mantissas.  Q4_K: (w >> 4k) & 0x000F000F, k = 0..3, is the pair of
// nibbles (k, k + 4) of a word; nibbles of equal parity belong to one sub-block,
// so pairs k = 0, 2 feed the accumulator of the even sub-block and k = 1, 3 the
// odd one.  Q6_K: the four 6-bit codes of a ql word are assembled one per byte as
// in the scalar kernel, then (q & 0x003F003F) and ((q >> 8) & 0x003F003F) are the
// pairs of bytes (0, 2) and (1, 3).  OR-ed with 0x3F803F80 each half reads as
// 1 + q / 128; the activation registers hold 128 x split into three bf16 pieces
// and the accumulator starts at -128 sum(x) (-160 sum(x) for Q6_K, whose codes
// are offset by 32), so that it ends as sum(q x) resp. sum((q - 32) x) exactly
// as in the affine kernels.
//
// Register r of a chunk (both formats) pairs local values
//   lo(r) = 32 (r / 16) + 4 ((r % 16) / 2) + r % 2   and   hi(r) = lo(r) + 2,
// accumulator group = r / 16 (Q4_K sub-block of 32) or r / 8 (Q6_K scale group of 16).
//
// Q6_K rows of 2048 values (GG_Q6W: the vocabulary projection of a 2048-wide model) have 32
// such chunks: the 16-lanes-per-row map with two chunks per lane, c and c + 16 (1024 values and
// four blocks further on), a slice of four whole rows = 6720 B, two slices per ring.
enum { GG_Q4 = 0, GG_Q6 = 1, GG_Q6W = 2 };

template <int KIND, int LPR>
struct GgLane;
template <int LPR>
struct GgLane<GG_Q4, LPR> {
    static constexpr int NREG = 64, GROUP_REGS = 16;
    static constexpr int ROW_BYTES = (LPR / 2) * 144;
    static constexpr int SLOT_DATA = (FM_WAVE / LPR) * ROW_BYTES;      // 4608
    __device__ static int col(int c, int v) { return 128 * c + v; }
};
template <int LPR>
struct GgLane<GG_Q6, LPR> {
    static constexpr int NREG = 32, GROUP_REGS = 8;
    static constexpr int ROW_BYTES = (LPR / 4) * 210;
    static constexpr int SLOT_DATA = (FM_WAVE / LPR) * ROW_BYTES;      // 3360
    __device__ static int col(int c, int v) { return 128 * (c >> 1) + 32 * (c & 1) + (v < 32 ? v : v + 32); }
};

template <>
struct GgLane<GG_Q6W, 16> {
    static constexpr int NREG = 32, GROUP_REGS = 8;
    static constexpr int ROW_BYTES = 8 * 210;
    static constexpr int SLOT_DATA = 4 * ROW_BYTES;                    // 6720
    __device__ static int col(int c, int v) { return GgLane<GG_Q6, 16>::col(c, v); }
};
// chunks an activation image holds per row (= lanes per row, except where a lane owns two)
template <int KIND, int LPR>
struct GgImgLpr {
    static constexpr int value = KIND == GG_Q6W ? 2 * LPR : LPR;
};

template <int KIND, bool GU>
struct GgRing {
    static constexpr int value = FM_GG_RING;
};

// activation image of one input vector: register quad q of entry e = 4*chunk + piece,
// and the plain sums of x over the four accumulator groups of each chunk
template <int NREG, int LPR>
struct GgImage {
    uint4 a[NREG / 4][4 * LPR];
    float4 sum[LPR];
};
template <int NREG>
struct GgAct {
    uint32_t a[NREG];
    float xsum[4];
};

// (LPR = chunks per row of the image; LL = the lane map's lanes per row, which names the format's constants)
template <int KIND, int LPR, int LL = LPR>
__device__ __forceinline__ void gg_build_image(const float *x, GgImage<GgLane<KIND, LL>::NREG, LPR> &L) {
    using G = GgLane<KIND, LL>;
    constexpr int NE = 4 * LPR;
    uint32_t *flat = reinterpret_cast<uint32_t *>(L.a);
    for (int it = threadIdx.x; it < LPR * G::NREG; it += blockDim.x) {
        const int ch = it / G::NREG, r = it % G::NREG;
        const int lo = 32 * (r >> 4) + 4 * ((r & 15) >> 1) + (r & 1);
        const float xl = x[G::col(ch, lo)], xh = x[G::col(ch, lo + 2)];
        const float vl = xl * 128.0f, vh = xh * 128.0f;
        uint32_t l0 = __float_as_uint(vl) & 0xFFFF0000u, h0 = __float_as_uint(vh) & 0xFFFF0000u;
        float rl = vl - __uint_as_float(l0), rh = vh - __uint_as_float(h0);
        uint32_t l1 = __float_as_uint(rl) & 0xFFFF0000u, h1 = __float_as_uint(rh) & 0xFFFF0000u;
        rl -= __uint_as_float(l1);
        rh -= __uint_as_float(h1);
        uint32_t l2 = __float_as_uint(rl), h2 = __float_as_uint(rh) & 0xFFFF0000u;
        uint32_t *dst = flat + ((r >> 2) * NE + 4 * ch) * 4 + (r & 3);
        dst[0] = (l0 >> 16) | h0;
        dst[4] = (l1 >> 16) | h1;
        dst[8] = (l2 >> 16) | h2;
        dst[12] = 0u;
        const float gs = fm_group_sum<G::GROUP_REGS>(xl + xh);
        if (r % G::GROUP_REGS == 0) reinterpret_cast<float *>(&L.sum[ch])[r / G::GROUP_REGS] = gs;
    }
}

// a lane's activation registers out of an image, while LDS-direct loads are in flight
// (explicit reads: see fm_ring.h)
template <int NREG>
__device__ __forceinline__ void gg_read_image(uint32_t img_addr, int n_entries, int lane, GgAct<NREG> &ar,
                                              int entry0 = 0) {
    const int e = lane % n_entries + entry0;
    uint32_t addr = img_addr + (uint32_t)e * 16u;
    const uint32_t stride = (uint32_t)n_entries * 16u;
#pragma unroll
    for (int q = 0; q < NREG / 4; q++) {
        fm_u4 v;
        asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
        ar.a[4 * q + 0] = v[0];
        ar.a[4 * q + 1] = v[1];
        ar.a[4 * q + 2] = v[2];
        ar.a[4 * q + 3] = v[3];
        addr += stride;
    }
    fm_u4 sm;
    const uint32_t sa = img_addr + (uint32_t)(NREG / 4) * stride + (uint32_t)(e >> 2) * 16u;
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=&v"(sm) : "v"(sa) : "memory");
#pragma unroll
    for (int g = 0; g < 4; g++) ar.xsum[g] = __uint_as_float(sm[g]);
}

__device__ __forceinline__ fm_f4 gg_mfma(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, fm_f4 acc) {
    fm_s4 av = __builtin_bit_cast(fm_s4, make_uint2(a0, a1));
    fm_s4 bv = __builtin_bit_cast(fm_s4, make_uint2(b0, b1));
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av, bv, acc, 0, 0, 0);
}

// ---- Q4_K lane: header + 64 bytes of nibbles out of a landed slice
struct GgQ4Lane {
    uint32_t hdr_off, q_off;
    int half;
    template <int LPR>
    __device__ __forceinline__ void init(int row_in_step, int ch) {
        hdr_off = (uint32_t)(row_in_step * GgLane<GG_Q4, LPR>::ROW_BYTES + (ch >> 1) * 144);
        half = ch & 1;
        q_off = hdr_off + 16u + 64u * (uint32_t)half;
    }
    __device__ __forceinline__ fm_u4 read(uint32_t slot, uint32_t tag_addr, Q4Half &t) const {
        const uint32_t ah = slot + hdr_off, aq = slot + q_off;
        fm_u4 tag;
        asm volatile("ds_read_b128 %0, %6\n\tds_read_b128 %1, %7\n\tds_read_b128 %2, %7 offset:16\n\t"
                     "ds_read_b128 %3, %7 offset:32\n\tds_read_b128 %4, %7 offset:48\n\t"
                     "ds_read_b128 %5, %8\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(t.hdr), "=&v"(t.q[0]), "=&v"(t.q[1]), "=&v"(t.q[2]), "=&v"(t.q[3]),
                       "=&v"(tag)
                     : "v"(ah), "v"(aq), "v"(tag_addr)
                     : "memory");
        return tag;
    }
    __device__ __forceinline__ float dot(const Q4Half &t, const GgAct<64> &ar, uint32_t ones) const {
        const float d = f16bits(t.hdr[0]), dmin = f16bits(t.hdr[0] >> 16);
        const uint32_t *qd = reinterpret_cast<const uint32_t *>(t.q);
        // the four (scale, min) pairs of this half, one per byte (finchmoe/infer.m:1595-1603)
        const uint32_t s0 = t.hdr[1], s1 = t.hdr[2], s2 = t.hdr[3];
        const uint32_t sc4 = half ? (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u) : s0 & 0x3F3F3F3Fu;
        const uint32_t mn4 = half ? ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u)
                                  : s1 & 0x3F3F3F3Fu;
        const float sc[4] = {fm_ubyte<0>(sc4), fm_ubyte<1>(sc4), fm_ubyte<2>(sc4), fm_ubyte<3>(sc4)};
        const float mn[4] = {fm_ubyte<0>(mn4), fm_ubyte<1>(mn4), fm_ubyte<2>(mn4), fm_ubyte<3>(mn4)};
        float r = 0.0f, rm = 0.0f;
#pragma unroll
        for (int c = 0; c < 2; c++) {
            fm_f4 ae = {-128.0f * ar.xsum[2 * c], 0.0f, 0.0f, 0.0f};
            fm_f4 ao = {-128.0f * ar.xsum[2 * c + 1], 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const uint32_t w = qd[8 * c + k];
                const uint32_t p0 = (w & 0x000F000Fu) | ones, p1 = ((w >> 4) & 0x000F000Fu) | ones;
                const uint32_t p2 = ((w >> 8) & 0x000F000Fu) | ones, p3 = ((w >> 12) & 0x000F000Fu) | ones;
                const uint32_t *ap = ar.a + 32 * c + 2 * k;
                ae = gg_mfma(ap[0], ap[1], p0, p2, ae);
                ao = gg_mfma(ap[16], ap[17], p1, p3, ao);
            }
            r = fmaf(sc[2 * c], (ae[0] + ae[1]) + ae[2], r);
            rm = fmaf(mn[2 * c], ar.xsum[2 * c], rm);
            r = fmaf(sc[2 * c + 1], (ao[0] + ao[1]) + ao[2], r);
            rm = fmaf(mn[2 * c + 1], ar.xsum[2 * c + 1], rm);
        }
        return d * r - dmin * rm;
    }
};

// ---- Q6_K lane: 32 ql bytes, 32 qh bytes, four scales and d.  Blocks are only 2-byte
// aligned, so the words are read at the 4-byte boundary below and funnel-shifted; the
// same shift drops the lane's side bits of qh.
struct GgQ6Data {
    uint32_t ql[9], qh[9], sc_a, sc_b, d;
};
struct GgQ6Lane {
    uint32_t ql_off, qh_off, sc_off, d_off, sh_l, sh_h;
    template <int LPR>
    __device__ __forceinline__ void init(int row_in_step, int ch) {
        init_rows(row_in_step, ch, GgLane<GG_Q6, LPR>::ROW_BYTES);
    }
    __device__ __forceinline__ void init_rows(int row_in_step, int ch, int row_bytes) {
        const int hf = (ch >> 1) & 1, sd = ch & 1;
        const uint32_t blk = (uint32_t)(row_in_step * row_bytes + (ch >> 2) * 210);
        const uint32_t ql = blk + 64u * hf + 32u * sd, qh = blk + 128u + 32u * hf;
        ql_off = ql & ~3u;
        qh_off = qh & ~3u;
        sh_l = (ql & 3u) * 8u;
        sh_h = (qh & 3u) * 8u + 2u * sd;
        sc_off = blk + 192u + 8u * hf + 2u * sd;
        d_off = blk + 208u;
    }
    __device__ __forceinline__ fm_u4 read(uint32_t slot, uint32_t tag_addr, GgQ6Data &t) const {
        const uint32_t al = slot + ql_off, ah = slot + qh_off, as = slot + sc_off, ad = slot + d_off;
        u32x2 l0, l1, l2, l3, h0, h1, h2, h3;
        fm_u4 tag;
        asm volatile("ds_read2_b32 %0, %14 offset1:1\n\tds_read2_b32 %1, %14 offset0:2 offset1:3\n\t"
                     "ds_read2_b32 %2, %14 offset0:4 offset1:5\n\tds_read2_b32 %3, %14 offset0:6 offset1:7\n\t"
                     "ds_read_b32 %4, %14 offset:32\n\t"
                     "ds_read2_b32 %5, %15 offset1:1\n\tds_read2_b32 %6, %15 offset0:2 offset1:3\n\t"
                     "ds_read2_b32 %7, %15 offset0:4 offset1:5\n\tds_read2_b32 %8, %15 offset0:6 offset1:7\n\t"
                     "ds_read_b32 %9, %15 offset:32\n\t"
                     "ds_read_u16 %10, %16\n\tds_read_u16 %11, %16 offset:4\n\tds_read_u16 %12, %17\n\t"
                     "ds_read_b128 %13, %18\n\ts_waitcnt lgkmcnt(0)"
                     : "=&v"(l0), "=&v"(l1), "=&v"(l2), "=&v"(l3), "=&v"(t.ql[8]), "=&v"(h0), "=&v"(h1),
                       "=&v"(h2), "=&v"(h3), "=&v"(t.qh[8]), "=&v"(t.sc_a), "=&v"(t.sc_b), "=&v"(t.d),
                       "=&v"(tag)
                     : "v"(al), "v"(ah), "v"(as), "v"(ad), "v"(tag_addr)
                     : "memory");
        t.ql[0] = l0[0], t.ql[1] = l0[1], t.ql[2] = l1[0], t.ql[3] = l1[1];
        t.ql[4] = l2[0], t.ql[5] = l2[1], t.ql[6] = l3[0], t.ql[7] = l3[1];
        t.qh[0] = h0[0], t.qh[1] = h0[1], t.qh[2] = h1[0], t.qh[3] = h1[1];
        t.qh[4] = h2[0], t.qh[5] = h2[1], t.qh[6] = h3[0], t.qh[7] = h3[1];
        return tag;
    }
    __device__ __forceinline__ float dot(const GgQ6Data &t, const GgAct<32> &ar, uint32_t ones) const {
        fm_f4 acc[4];
#pragma unroll
        for (int g = 0; g < 4; g++) acc[g] = {-160.0f * ar.xsum[g], 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const uint32_t a = __builtin_amdgcn_alignbit(t.ql[i + 1], t.ql[i], sh_l);
            // bits 30, 31 may hold the next byte's: no mask below looks at them
            const uint32_t h = __builtin_amdgcn_alignbit(t.qh[i + 1], t.qh[i], sh_h);
            const uint32_t qa = ((h << 4) & 0x30303030u) | (a & 0x0F0F0F0Fu);
            const uint32_t qb = (h & 0x30303030u) | ((a >> 4) & 0x0F0F0F0Fu);
            const uint32_t pa0 = (qa & 0x003F003Fu) | ones, pa1 = ((qa >> 8) & 0x003F003Fu) | ones;
            const uint32_t pb0 = (qb & 0x003F003Fu) | ones, pb1 = ((qb >> 8) & 0x003F003Fu) | ones;
            acc[i >> 2] = gg_mfma(ar.a[2 * i], ar.a[2 * i + 1], pa0, pa1, acc[i >> 2]);
            acc[2 + (i >> 2)] = gg_mfma(ar.a[16 + 2 * i], ar.a[17 + 2 * i], pb0, pb1, acc[2 + (i >> 2)]);
        }
        const float s0 = (float)(int)(int8_t)(t.sc_a & 0xFFu), s1 = (float)(int)(int8_t)(t.sc_a >> 8);
        const float s2 = (float)(int)(int8_t)(t.sc_b & 0xFFu), s3 = (float)(int)(int8_t)(t.sc_b >> 8);
        float r = s0 * ((acc[0][0] + acc[0][1]) + acc[0][2]);
        r = fmaf(s1, (acc[1][0] + acc[1][1]) + acc[1][2], r);
        r = fmaf(s2, (acc[2][0] + acc[2][1]) + acc[2][2], r);
        r = fmaf(s3, (acc[3][0] + acc[3][1]) + acc[3][2], r);
        return f16bits(t.d) * r;
    }
};

// BYTES of a slice, 16 per lane and load; the last load is partial.  The
// instruction offset moves the global and the LDS address alike.
template <int BYTES, int I, int AUX = FM_AUX_KEEP>
__device__ __forceinline__ void gg_dma(uint32_t slot, const uint8_t *src, int lane) {
    if constexpr (I * 1024 < BYTES) {
        // (the offset field holds -4096..4095: from the fifth load on it starts again from
        // addresses moved by 4096)
        constexpr int BASE = (I / 4) * 4096, IMM = (I % 4) * 1024;
        if (I * 1024 + lane * 16 < BYTES)
            __builtin_amdgcn_global_load_lds((fm_gptr)(uintptr_t)(src + BASE),
                                             (fm_lptr)(uintptr_t)(slot + BASE), 16, IMM, AUX);
        gg_dma<BYTES, I + 1, AUX>(slot, src, lane);
    }
}

// ---- Q6_K lane of a 2048-value row: chunks ch and ch + 16 of the row
struct GgQ6WData {
    GgQ6Data p[2];
};
struct GgQ6WLane {
    GgQ6Lane l[2];
    template <int LPR>
    __device__ __forceinline__ void init(int row_in_step, int ch) {
        l[0].init_rows(row_in_step, ch, GgLane<GG_Q6W, 16>::ROW_BYTES);
        l[1].init_rows(row_in_step, ch + 16, GgLane<GG_Q6W, 16>::ROW_BYTES);
    }
    __device__ __forceinline__ fm_u4 read(uint32_t slot, uint32_t tag_addr, GgQ6WData &t) const {
        (void)l[0].read(slot, tag_addr, t.p[0]);
        return l[1].read(slot, tag_addr, t.p[1]);
    }
};

template <int KIND> struct GgLaneOps;
template <> struct GgLaneOps<GG_Q4> { using Lane = GgQ4Lane; using Data = Q4Half; };
template <> struct GgLaneOps<GG_Q6> { using Lane = GgQ6Lane; using Data = GgQ6Data; };
template <> struct GgLaneOps<GG_Q6W> { using Lane = GgQ6WLane; using Data = GgQ6WData; };

template <int KIND, int LPR, bool GU>
constexpr size_t gg_stream_lds() {
    using G = GgLane<KIND, LPR>;
    return (size_t)FM_GG_NW(KIND == GG_Q6W) * GgRing<KIND, GU>::value * (G::SLOT_DATA + 16) +
           (GU ? 2 : 3) * sizeof(GgImage<G::NREG, GgImgLpr<KIND, LPR>::value>);
}

extern __shared__ __attribute__((aligned(16))) uint8_t fm_gguf_lds[];

// u / d without the division sequence (fm_index.h), callable
struct GgDiv : FmDiv {
    __device__ __forceinline__ uint32_t operator()(uint32_t u) const { return fm_div(*this, u); }
};
inline GgDiv gg_div_make(uint32_t d) {
    GgDiv r;
    static_cast<FmDiv &>(r) = fm_div_make(d);
    return r;
}

// Where the rows of a pair's expert start, looked up once per workgroup: a global
// (scalar) load per claimed unit would stall its wave for a memory round trip
// behind the weight stream.
struct __attribute__((aligned(16))) GgPairEntry {
    uint64_t first;        // gate (or down) rows of the expert
    int64_t second;        // up rows - gate rows
    uint32_t invalid, pad[3];
};

// what a slice's trailer says about its unit
struct GgUnit {
    uint32_t flags, pair, step, image;     // flags bit 0: the pair's expert index is invalid
};

// GU: gate and up rows (both Q4_K) of a unit, SwiGLU -> act.  Otherwise: down rows -> expert_out.
// Units (wave steps) of the launch are numbered pair-major, by_upp divides by the units per pair,
// by_k by K.
template <int KIND, int LPR, bool GU>
__global__ __launch_bounds__(FM_GG_NW(KIND == GG_Q6W) * 64) void fm_gguf_stream(GgufArgs a, int total_units, GgDiv by_upp,
                                                      GgDiv by_k) {
#if defined(__HIP_DEVICE_COMPILE__)
    using G = GgLane<KIND, LPR>;
    using Lane = typename GgLaneOps<KIND>::Lane;
    using Data = typename GgLaneOps<KIND>::Data;
    constexpr bool WIDE = KIND == GG_Q6W;
    constexpr int ILPR = GgImgLpr<KIND, LPR>::value;
    using Image = GgImage<G::NREG, ILPR>;
    constexpr int RPS = FM_WAVE / LPR, NS = GU ? 2 : 1, NIMG = GU ? 2 : 3;
    constexpr int RING = GgRing<KIND, GU>::value;
    static_assert(!(WIDE && GU), "the two-chunk lane map is a down / dense-tensor form");
    constexpr int SLOT = G::SLOT_DATA + 16, TAG = G::SLOT_DATA, LOADS = (G::SLOT_DATA + 1023) / 1024;
    // pairs a workgroup's share can touch: it spans at most NIMG - 1 input vectors' worth
    constexpr int NPAIR = GU ? FM_MAX_K + 1 : NIMG;
    __shared__ unsigned int next_unit;
    __shared__ GgPairEntry ptab[NPAIR];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t ring0 = fm_lds_addr(fm_gguf_lds) + (uint32_t)wave * (RING * SLOT);
    Image *img = reinterpret_cast<Image *>(fm_gguf_lds + FM_GG_NW(WIDE) * RING * SLOT);
    const uint32_t img0 = fm_lds_addr(img);
    const FmRange wg = fm_share(total_units, blockIdx.x, gridDim.x);
    const long wg0 = wg.lo, wg1 = wg.hi;
    const uint32_t n_units = (uint32_t)(wg1 - wg0);
    if (n_units == 0) return;
    // a dense tensor, the layers of a step, one layer: every byte is read once (fm_ring.h,
    // FM_AUX_ONCE); the positions of a chunk share one layer's experts
    const bool once = a.direct != nullptr || a.layer_stride != 0 || total_units == (int)(by_upp.d * by_k.d);
    const int in_dim = GU ? a.g.hidden : a.g.inter;
    // input vector of a pair: its layer's x (gate/up) or its own act (down)
    auto vector_of = [&](uint32_t pair) __attribute__((always_inline)) {
        return GU ? by_k(pair) : pair;
    };
    const uint32_t pair0 = by_upp((uint32_t)wg0), pair_last = by_upp((uint32_t)wg1 - 1u);
    const uint32_t vid0 = vector_of(pair0);
    const int n_img = (int)(vector_of(pair_last) - vid0) + 1;
    const float *xbase = GU ? a.x : a.act;
    if (threadIdx.x == 0) next_unit = 0u;
    if (threadIdx.x <= pair_last - pair0 && threadIdx.x < NPAIR) {
        const uint32_t pair = pair0 + threadIdx.x;
        const bool direct = !GU && a.direct != nullptr;
        int e = direct ? 0 : a.idx[pair];
        const bool ok = (unsigned)e < (unsigned)a.g.n_experts;
        if (!ok) e = 0;                                  // stream something valid, store zeros
        const int li = a.layer0 + (int)by_k(pair) * a.layer_stride;
        GgPairEntry pe;
        if (direct) {
            pe.first = (uint64_t)(uintptr_t)a.direct;
            pe.second = 0;
        } else if constexpr (GU) {
            const uint8_t *g = a.gate[li] + (size_t)e * a.g.gate_slab;
            pe.first = (uint64_t)(uintptr_t)g;
            pe.second = (int64_t)((a.up[li] + (size_t)e * a.g.up_slab) - g);
        } else {
            pe.first = (uint64_t)(uintptr_t)(a.down[li] + (size_t)e * a.g.down_slab);
            pe.second = 0;
        }
        pe.invalid = ok ? 0u : 1u;
        pe.pad[0] = pe.pad[1] = pe.pad[2] = 0u;
        ptab[threadIdx.x] = pe;
    }
    __syncthreads();
    const uint32_t ptab0 = fm_lds_addr(ptab);

    const int j = lane & 3, ch = (lane >> 2) % LPR, ris = 4 * (lane / (4 * LPR)) + j;
    Lane ln;
    ln.template init<LPR>(ris, ch);

    // ---- loader
    int kn = 0, wpos = 0;
    uint32_t issued = 0, consumed = 0;
    GgUnit un{0u, 0u, 0u, 0u};
    const uint8_t *p0 = nullptr;
    ptrdiff_t p_second = 0;
    bool dry = false;
    auto issue = [&]() __attribute__((always_inline)) {
        if (dry) return;
        if (kn == 0) {
            const uint32_t ul = fm_claim_unit(&next_unit, lane);
            if (ul >= n_units) {
                dry = true;
                return;
            }
            const uint32_t u = (uint32_t)wg0 + ul;
            un.pair = by_upp(u);
            un.step = u - un.pair * by_upp.d;
            un.image = vector_of(un.pair) - vid0;
            fm_u4 pe;
            uint32_t inv;
            const uint32_t pa = ptab0 + (un.pair - pair0) * (uint32_t)sizeof(GgPairEntry);
            asm volatile("ds_read_b128 %0, %2\n\tds_read_b32 %1, %2 offset:16\n\ts_waitcnt lgkmcnt(0)"
                         : "=&v"(pe), "=&v"(inv)
                         : "v"(pa)
                         : "memory");
            un.flags = __builtin_amdgcn_readfirstlane(inv);
            // (readfirstlane returns int: widen as unsigned)
            const uint32_t f_lo = __builtin_amdgcn_readfirstlane(pe[0]), f_hi = __builtin_amdgcn_readfirstlane(pe[1]);
            const uint32_t s_lo = __builtin_amdgcn_readfirstlane(pe[2]), s_hi = __builtin_amdgcn_readfirstlane(pe[3]);
            p0 = (const uint8_t *)(uintptr_t)(((uint64_t)f_hi << 32) | f_lo) + (size_t)un.step * G::SLOT_DATA;
            if constexpr (GU) p_second = (ptrdiff_t)(((uint64_t)s_hi << 32) | s_lo);
        }
        const uint32_t slot = ring0 + (uint32_t)wpos * SLOT;
        {
            const uint32_t ta = slot + TAG;
            const fm_u4 tv = {un.flags, un.pair, un.step, un.image};
            asm volatile("ds_write_b128 %0, %1" ::"v"(ta), "v"(tv) : "memory");
        }
        const uint8_t *src = p0 + (ptrdiff_t)kn * p_second + lane * 16;
        if (once) gg_dma<G::SLOT_DATA, 0, FM_AUX_ONCE>(slot, src, lane);
        else gg_dma<G::SLOT_DATA, 0, FM_AUX_KEEP>(slot, src, lane);
        kn = kn + 1 == NS ? 0 : kn + 1;
        wpos = wpos + 1 == RING ? 0 : wpos + 1;
        issued++;
    };
#pragma unroll
    for (int k = 0; k < RING; k++) issue();

    // the images of every input vector this workgroup's units touch
    for (int v = 0; v < n_img && v < NIMG; v++)
        gg_build_image<KIND, ILPR, LPR>(xbase + (size_t)(vid0 + v) * in_dim, img[v]);
    __syncthreads();

    GgAct<G::NREG> ar, ar2;        // (ar2: the second chunk of a lane that owns two)
    uint32_t cur_image = ~0u;
    const uint32_t ones = fm_opaque(0x3F803F80u);
    int c = 0;
    while (consumed < issued) {
        float v[NS];
        fm_u4 tag;
#pragma unroll
        for (int k = 0; k < NS; k++) {
            Data t;
            if (issued - consumed == (uint32_t)RING) fm_dma_wait<LOADS *(RING - 1)>(false);
            else fm_dma_wait<0>(true);
            const uint32_t slot = ring0 + (uint32_t)c * SLOT;
            tag = ln.read(slot, slot + TAG, t);
            consumed++;
            c = c + 1 == RING ? 0 : c + 1;
            issue();
            if (k == 0) {
                const uint32_t image = __builtin_amdgcn_readfirstlane(tag[3]);
                if (image != cur_image) {
                    gg_read_image<G::NREG>(img0 + image * (uint32_t)sizeof(Image), 4 * ILPR, lane, ar);
                    if constexpr (WIDE)
                        gg_read_image<G::NREG>(img0 + image * (uint32_t)sizeof(Image), 4 * ILPR, lane, ar2, 4 * LPR);
                    cur_image = image;
                }
            }
            if constexpr (WIDE) v[k] = fm_chunk_sum<LPR>(ln.l[0].dot(t.p[0], ar, ones) + ln.l[1].dot(t.p[1], ar2, ones));
            else v[k] = fm_chunk_sum<LPR>(ln.dot(t, ar, ones));
        }
        const uint32_t pair = __builtin_amdgcn_readfirstlane(tag[1]);
        const uint32_t step = __builtin_amdgcn_readfirstlane(tag[2]);
        const bool ok = __builtin_amdgcn_readfirstlane(tag[0]) == 0u;
        if (ch == 0) {
            if constexpr (GU)
                a.act[(size_t)pair * a.g.inter + step * RPS + ris] = ok ? fm_silu_mul(v[0], v[NS - 1]) : 0.0f;
            else
                a.expert_out[(size_t)pair * a.g.hidden + step * RPS + ris] = ok ? v[0] : 0.0f;
        }
    }
#else
    (void)a;
    (void)total_units;
    (void)by_upp;
    (void)by_k;
#endif
}

// ======================================================================
// The operator as one launch when the caller does not want the per-expert vectors and the
// plain combine applies: the form of fm_moe_fused_rows (fm_decode.hip) for block formats.
//
// Gate/up: contiguous ranges of units (a unit = the gate slice and the up slice of a wave step),
// SwiGLU, activations stored at device scope into a set whose elements hold FM_ACT_EMPTY until
// then.  Down by row blocks: a row block is one wave step's rows of all K experts of a layer; a
// workgroup owns whole output rows of ONE layer (fm2_split), polls that layer's K activation
// vectors into K images, keeps the K partial vectors of its rows in LDS and adds them up itself,
// w_k * down_k in slot order — fm_gguf_combine<false>'s arithmetic.  No per-expert vectors, no
// combine launch, nobody waits for the slowest workgroup of the grid.  The shares are sized so
// that every workgroup streams the same number of bytes.
//
// A gate/up slice and a down slice differ in size, so the ring changes geometry between the
// phases: the loader does not run on from the last gate/up unit into the down phase; a wave
// refills its ring with down slices as soon as it has consumed its last gate/up slice, before
// the workgroup's barrier and the polls.
// ======================================================================
struct __attribute__((aligned(16))) GgSeg {
    uint64_t first[FM_MAX_K];      // gate (or down) rows of slot k's expert
    int64_t second[FM_MAX_K];      // up rows - gate rows
    float w[FM_MAX_K];             // router weight, 0 for an invalid expert index
    uint32_t valid;                // bit k: slot k has a valid expert index
    uint32_t next_unit;
    uint32_t first_unit, n;        // this workgroup's units of the segment
    int layer;                     // layer group
    int pad[3];
};
static_assert(sizeof(GgSeg) == FM_GG2_SEG_BYTES, "segment table entry");

template <int DN_KIND, int LPR_UP, int LPR_DN>
struct GgFused {
    using GU = GgLane<GG_Q4, LPR_UP>;
    using GD = GgLane<DN_KIND, LPR_DN>;
    using LaneD = typename GgLaneOps<DN_KIND>::Lane;
    using DataD = typename GgLaneOps<DN_KIND>::Data;
    using ImageU = GgImage<GU::NREG, LPR_UP>;
    using ImageD = GgImage<GD::NREG, LPR_DN>;
    static constexpr int RPS_UP = FM_WAVE / LPR_UP, RPS_DN = FM_WAVE / LPR_DN;
    static constexpr int RING_UP = FM_GG2_RING_UP, RING_DN = DN_KIND == GG_Q6 ? 4 : 3;
    static constexpr int SLOT_UP = GU::SLOT_DATA + 16, SLOT_DN = GD::SLOT_DATA + 16;
    static constexpr int LOADS_UP = (GU::SLOT_DATA + 1023) / 1024, LOADS_DN = (GD::SLOT_DATA + 1023) / 1024;
    static constexpr int RING_BYTES = RING_UP * SLOT_UP > RING_DN * SLOT_DN ? RING_UP * SLOT_UP : RING_DN * SLOT_DN;
    static constexpr int IMG_UP = (int)sizeof(ImageU), IMG_DN = (int)sizeof(ImageD);
    static constexpr int IMG_BYTES = 2 * IMG_UP > FM_MAX_K * IMG_DN ? 2 * IMG_UP : FM_MAX_K * IMG_DN;
    static constexpr int LDS_BYTES = 8 * RING_BYTES + IMG_BYTES + FM2_MAX_SEG * (int)sizeof(GgSeg) + FM2_PART_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");

    const GgufArgs &a;
    const Fm2Sync &sy;
    int lane, wave;
    uint32_t ring0, img0, part0;
    GgSeg *tab;
    FmDiv by_gu_upp, by_K;
    int n_up, n_seq;
    // loader
    bool l_gu, dry;
    bool once;              // every expert byte is read once in this launch (fm_ring.h, FM_AUX_ONCE)
    int lq, cq, hn, wpos, c;
    uint32_t l_first, l_n, l_nrb, tag_n, issued, consumed;
    float l_inv;
    const uint8_t *src_n;
    ptrdiff_t second_n;
    uint32_t ones;

    __device__ __forceinline__ GgFused(const GgufArgs &a_, const Fm2Sync &sy_) : a(a_), sy(sy_) {
        lane = threadIdx.x & 63;
        wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const uint32_t lds0 = fm_lds_addr(fm_gguf_lds);
        ring0 = lds0 + (uint32_t)wave * RING_BYTES;
        img0 = lds0 + 8u * RING_BYTES;
        tab = reinterpret_cast<GgSeg *>(fm_gguf_lds + 8 * RING_BYTES + IMG_BYTES);
        part0 = img0 + (uint32_t)IMG_BYTES + FM2_MAX_SEG * (uint32_t)sizeof(GgSeg);
        l_gu = true, dry = false;
        once = a.layer_stride != 0;
        lq = cq = hn = wpos = c = 0;
        l_first = l_n = l_nrb = tag_n = issued = consumed = 0u;
        l_inv = 0.0f;
        src_n = nullptr;
        second_n = 0;
        ones = fm_opaque(0x3F803F80u);
    }

    __device__ __forceinline__ void loader_enter(int q) {
        const uint32_t ta = fm_lds_addr(&tab[q].first_unit);
        l_first = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta));
        l_n = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + 4));
        if (!l_gu) {
            l_nrb = fm_div(by_K, l_n);
            l_first = fm_div(by_K, l_first);            // first row block of the part
            l_inv = 1.0f / (float)(l_nrb ? l_nrb : 1u);
        }
    }

    // the next slice of the loader's phase into the ring's write position
    template <bool GATE_UP>
    __device__ __forceinline__ void issue() {
        constexpr int RING = GATE_UP ? RING_UP : RING_DN, SLOT = GATE_UP ? SLOT_UP : SLOT_DN;
        constexpr int DATA = GATE_UP ? GU::SLOT_DATA : GD::SLOT_DATA;
        if (dry) return;
        if (!GATE_UP || hn == 0) {
            uint32_t ul;
            const int q_end = GATE_UP ? n_up : n_seq;
            for (;;) {
                ul = fm_claim_unit(&tab[lq].next_unit, lane);
                if (ul < l_n) break;
                if (lq + 1 < q_end && lq == cq) {       // run on into the next segment of the phase
                    lq++;
                    loader_enter(lq);
                    continue;
                }
                dry = true;
                return;
            }
            uint32_t pn, rsn;
            if (GATE_UP) fm2_gu_unit(l_first, ul, by_gu_upp, &pn, &rsn);
            else fm2_dn_unit(l_first, l_nrb, l_inv, ul, &pn, &rsn);     // expert by expert
            tag_n = ((uint32_t)(lq & 1) << 31) | (pn << 28) | ul;
            const uint32_t fa = fm_lds_addr(&tab[lq].first[pn]);
            const uint32_t lo = __builtin_amdgcn_readfirstlane(fm_lds_r32(fa));
            const uint32_t hi = __builtin_amdgcn_readfirstlane(fm_lds_r32(fa + 4));
            src_n = (const uint8_t *)(((uintptr_t)hi << 32) | lo) + (size_t)rsn * DATA;
            if (GATE_UP) {
                const uint32_t sa = fm_lds_addr(&tab[lq].second[pn]);
                const uint32_t slo = __builtin_amdgcn_readfirstlane(fm_lds_r32(sa));
                const uint32_t shi = __builtin_amdgcn_readfirstlane(fm_lds_r32(sa + 4));
                second_n = (ptrdiff_t)(((uint64_t)shi << 32) | slo);
            }
        }
        const uint32_t slot = ring0 + (uint32_t)wpos * SLOT;
        fm_slot_tag(slot + DATA, tag_n);
        const uint8_t *src = src_n + (GATE_UP ? (ptrdiff_t)hn * second_n : (ptrdiff_t)0) + lane * 16;
        if (once) gg_dma<DATA, 0, FM_AUX_ONCE>(slot, src, lane);
        else gg_dma<DATA, 0, FM_AUX_KEEP>(slot, src, lane);
        if (GATE_UP) hn ^= 1;
        wpos = wpos + 1 == RING ? 0 : wpos + 1;
        issued++;
    }

    // The next slice out of the ring into registers, its tag, and the slot handed back to the
    // loader at once.  The consumer fetches a slice before it multiplies the one fetched before,
    // so a slice that lands while the wave is busy does not keep its slot (measured: no
    // difference against fetching and multiplying in turn; the launch is bound by the stream).
    __device__ __forceinline__ uint32_t fetch_up(const GgQ4Lane &ln, Q4Half &t) {
        if (issued - consumed == (uint32_t)RING_UP) fm_dma_wait<LOADS_UP *(RING_UP - 1)>(false);
        else fm_dma_wait<0>(true);
        const uint32_t slot = ring0 + (uint32_t)c * SLOT_UP;
        const fm_u4 tag = ln.read(slot, slot + GU::SLOT_DATA, t);
        consumed++;
        c = c + 1 == RING_UP ? 0 : c + 1;
        issue<true>();
        return __builtin_amdgcn_readfirstlane(tag[0]);
    }
    __device__ __forceinline__ uint32_t fetch_dn(const LaneD &ln, DataD &t) {
        if (issued - consumed == (uint32_t)RING_DN) fm_dma_wait<LOADS_DN *(RING_DN - 1)>(false);
        else fm_dma_wait<0>(true);
        const uint32_t slot = ring0 + (uint32_t)c * SLOT_DN;
        const fm_u4 tag = ln.read(slot, slot + GD::SLOT_DATA, t);
        consumed++;
        c = c + 1 == RING_DN ? 0 : c + 1;
        issue<false>();
        return __builtin_amdgcn_readfirstlane(tag[0]);
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

    // w_k * partial_k over the part's rows, in slot order -> out
    __device__ __forceinline__ void reduce_part(int q) {
        const int K = a.K;
        const uint32_t ta = fm_lds_addr(&tab[q]);
        const uint32_t first = fm_lds_r32(ta + (uint32_t)offsetof(GgSeg, first_unit));
        const uint32_t n = fm_lds_r32(ta + (uint32_t)offsetof(GgSeg, n));
        float wk[FM_MAX_K];
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            wk[k] = k < K ? __uint_as_float(fm_lds_r32(ta + (uint32_t)offsetof(GgSeg, w) + 4u * k)) : 0.0f;
        const int rows = (int)fm_div(by_K, n) * RPS_DN;
        const int l = seg_layer(q);
        float *out = a.out + (size_t)l * a.g.hidden + (size_t)fm_div(by_K, first) * RPS_DN;
        for (int r = threadIdx.x; r < rows; r += 512) {
            const int rbi = r / RPS_DN, ris = r - rbi * RPS_DN;
            float acc = 0.0f;
#pragma unroll
            for (int k = 0; k < FM_MAX_K; k++)
                if (k < K && wk[k] != 0.0f)
                    acc += wk[k] * __uint_as_float(fm_lds_r32(part0 + 4u * (uint32_t)((rbi * K + k) * RPS_DN + ris)));
            out[r] = (a.flags & FM_ACCUMULATE) ? out[r] + acc : acc;
        }
    }

    // The K activation vectors of layer l -> K down images.  Thread t takes the (image, chunk,
    // register) combinations t, t + 512, ...: all loads first, polls where needed after.
    __device__ __forceinline__ void build_down_images(int l) {
        constexpr int NREG = GD::NREG, PER = LPR_DN * NREG, NE = 4 * LPR_DN;
        constexpr int NIT = FM_MAX_K * PER / 512;
        static_assert(FM_MAX_K * PER % 512 == 0 && PER % 64 == 0, "whole waves per image");
        const int K = a.K;
        float xl[NIT], xh[NIT];
#pragma unroll
        for (int i = 0; i < NIT; i++) {
            const int it = (int)threadIdx.x + 512 * i;
            const int k = it / PER, rem = it - k * PER, ch = rem / NREG, r = rem - ch * NREG;
            const int lo = 32 * (r >> 4) + 4 * ((r & 15) >> 1) + (r & 1);
            const float *src = a.act + ((size_t)l * K + (k < K ? k : 0)) * a.g.inter;
            xl[i] = fm_ld_shared(src + GD::col(ch, lo));
            xh[i] = fm_ld_shared(src + GD::col(ch, lo + 2));
        }
#pragma unroll
        for (int i = 0; i < NIT; i++) {
            const int it = (int)threadIdx.x + 512 * i;
            const int k = it / PER, rem = it - k * PER, ch = rem / NREG, r = rem - ch * NREG;
            const int lo = 32 * (r >> 4) + 4 * ((r & 15) >> 1) + (r & 1);
            const bool on = k < K;
            const float *src = a.act + ((size_t)l * K + (on ? k : 0)) * a.g.inter;
            if (__float_as_uint(xl[i]) == FM_ACT_EMPTY) xl[i] = act_get(src + GD::col(ch, lo));
            if (__float_as_uint(xh[i]) == FM_ACT_EMPTY) xh[i] = act_get(src + GD::col(ch, lo + 2));
            // gg_build_image's arithmetic with explicit LDS writes
            const float vl = xl[i] * 128.0f, vh = xh[i] * 128.0f;
            const uint32_t l0 = __float_as_uint(vl) & 0xFFFF0000u, h0 = __float_as_uint(vh) & 0xFFFF0000u;
            float rl = vl - __uint_as_float(l0), rh = vh - __uint_as_float(h0);
            const uint32_t l1 = __float_as_uint(rl) & 0xFFFF0000u, h1 = __float_as_uint(rh) & 0xFFFF0000u;
            rl -= __uint_as_float(l1);
            rh -= __uint_as_float(h1);
            const uint32_t l2 = __float_as_uint(rl), h2 = __float_as_uint(rh) & 0xFFFF0000u;
            const float gs = fm_group_sum<GD::GROUP_REGS>(xl[i] + xh[i]);
            if (on) {
                const uint32_t img = img0 + (uint32_t)k * IMG_DN;
                const uint32_t dst = img + (uint32_t)((((r >> 2) * NE + 4 * ch) * 4 + (r & 3)) * 4);
                fm_lds_w32(dst, (l0 >> 16) | h0);
                fm_lds_w32(dst + 16, (l1 >> 16) | h1);
                fm_lds_w32(dst + 32, (l2 >> 16) | h2);
                fm_lds_w32(dst + 48, 0u);
                if (r % GD::GROUP_REGS == 0)
                    fm_lds_w32(img + (uint32_t)((NREG / 4) * NE * 16 + ch * 16 + (r / GD::GROUP_REGS) * 4),
                               __float_as_uint(gs));
            }
        }
    }

    __device__ __forceinline__ void run(const Fm2Dims &dm) {
        const int K = a.K, G = gridDim.x, g = blockIdx.x;
        by_gu_upp = dm.by_gu_upp, by_K = dm.by_K;
        if (dm.L == 1u) once = true;
        const Fm2Split sp = fm2_split(dm, (uint32_t)g);
        const uint32_t gu_segu = dm.gu_segu;
        n_up = sp.n_up;
        n_seq = sp.n_up + sp.n_dn;
        const int qq = threadIdx.x >> 3;        // the segment this thread looks up below
        const bool mine = qq < n_seq;
        const Fm2Part mp = fm2_part(dm, sp, mine ? qq : 0);

        // the other activation set becomes empty again (plain stores, nobody reads it now)
        for (unsigned int i = blockIdx.x * blockDim.x + threadIdx.x; i < sy.clear_n; i += G * blockDim.x)
            sy.act_other[i] = __uint_as_float(FM_ACT_EMPTY);
        if (n_seq == 0) return;

        // the tables of every segment: thread 8q + k looks up slot k of segment q
        if (mine) {
            const int k = threadIdx.x & 7;
            const size_t sg = mp.seg;
            GgSeg &t = tab[qq];
            bool ok = false;
            if (k < K) {
                int e = a.idx[sg * K + k];
                const float wv = a.w[sg * K + k];
                ok = (unsigned)e < (unsigned)a.g.n_experts;
                if (!ok) e = 0;                          // stream something valid, count zeros
                const int li = a.layer0 + (int)sg * a.layer_stride;
                if (mp.gu) {
                    const uint8_t *gp = a.gate[li] + (size_t)e * a.g.gate_slab;
                    t.first[k] = (uint64_t)(uintptr_t)gp;
                    t.second[k] = (int64_t)((a.up[li] + (size_t)e * a.g.up_slab) - gp);
                } else {
                    t.first[k] = (uint64_t)(uintptr_t)(a.down[li] + (size_t)e * a.g.down_slab);
                    t.second[k] = 0;
                }
                t.w[k] = ok ? wv : 0.0f;
            }
            const uint64_t m = __ballot(ok);
            if (k == 0) {
                t.valid = (uint32_t)(m >> (threadIdx.x & 56)) & 0xFFu;
                t.next_unit = 0u;
                t.first_unit = mp.first;
                t.n = mp.n;
                t.layer = (int)sg;
            }
        }
        __syncthreads();

        const int j = lane & 3;
        // ---------------------------------------------------------- gate/up
        if (n_up > 0) {
            loader_enter(0);
#pragma nounroll
            for (int k = 0; k < RING_UP; k++) issue<true>();
            // the images of both gate/up segments; a wave then changes segment on its own
            ImageU *img = reinterpret_cast<ImageU *>(fm_gguf_lds + 8 * RING_BYTES);
            for (int v = 0; v < n_up && v < 2; v++)
                gg_build_image<GG_Q4, LPR_UP>(a.x + (size_t)(sp.gu_s0 + v) * a.g.hidden, img[v]);
            __syncthreads();

            const int ch = (lane >> 2) % LPR_UP, ris = 4 * (lane / (4 * LPR_UP)) + j;
            GgQ4Lane ln;
            ln.template init<LPR_UP>(ris, ch);
            Q4Half ta_, tb_;                  // gate slice of the unit in hand, its up slice
            uint32_t tag_a = 0u;
            bool have = false;
            for (; cq < n_up; cq++) {
                const int s = seg_layer(cq);
                GgAct<GU::NREG> ar;
                gg_read_image<GU::NREG>(img0 + (uint32_t)(cq & 1) * IMG_UP, 4 * LPR_UP, lane, ar);
                const uint32_t ta = fm_lds_addr(&tab[cq]);
                const uint32_t valid = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + (uint32_t)offsetof(GgSeg, valid)));
                const uint32_t c_first = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + (uint32_t)offsetof(GgSeg, first_unit)));
                const size_t out0 = ((size_t)s * gu_segu + c_first) * RPS_UP + ris;
                dry = false;
                while (issued - consumed < (uint32_t)RING_UP && !dry) issue<true>();
                if (!have && consumed < issued) {
                    tag_a = fetch_up(ln, ta_);
                    have = true;
                }
                while (have) {
                    if ((tag_a >> 31) != (uint32_t)(cq & 1)) break;      // the next segment's: it waits in the registers
                    const uint32_t pc = (tag_a >> 28) & 7u, ul = tag_a & 0x0FFFFFFFu;
                    (void)fetch_up(ln, tb_);                             // (the up slice follows its gate slice)
                    const float gv = fm_chunk_sum<LPR_UP>(ln.dot(ta_, ar, ones));
                    have = consumed < issued;
                    if (have) tag_a = fetch_up(ln, ta_);
                    const float uv = fm_chunk_sum<LPR_UP>(ln.dot(tb_, ar, ones));
                    float v = fm_silu_mul(gv, uv);
                    if (!((valid >> pc) & 1u)) v = 0.0f;
                    if (ch == 0) fm_st_shared(a.act + out0 + (size_t)ul * RPS_UP, v);
                }
            }
        }
        // ---------------------------------------------------------- down
        if (n_seq > n_up) {
            // the ring is empty: its geometry changes
            l_gu = false;
            dry = false;
            hn = wpos = c = 0;
            issued = consumed = 0u;
            lq = cq = n_up;
            loader_enter(lq);
#pragma nounroll
            for (int k = 0; k < RING_DN; k++) issue<false>();

            const int ch = (lane >> 2) % LPR_DN, ris = 4 * (lane / (4 * LPR_DN)) + j;
            LaneD ln;
            ln.template init<LPR_DN>(ris, ch);
            DataD td0, td1;                   // the slice in hand and the one fetched behind it
            uint32_t tag_d = 0u;
            bool have_d = false;
            for (; cq < n_seq; cq++) {
                const int l = seg_layer(cq);
                fm_wg_barrier();                       // images and partial vectors are free
                if (cq > n_up) reduce_part(cq - 1);
                build_down_images(l);
                fm_wg_barrier();
                const uint32_t ta = fm_lds_addr(&tab[cq]);
                const uint32_t valid = __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + (uint32_t)offsetof(GgSeg, valid)));
                const uint32_t c_nrb = fm_div(by_K, __builtin_amdgcn_readfirstlane(fm_lds_r32(ta + (uint32_t)offsetof(GgSeg, n))));
                GgAct<GD::NREG> ar;
                uint32_t k_cur = 0xFFFFFFFFu;
                dry = false;
                while (issued - consumed < (uint32_t)RING_DN && !dry) issue<false>();
                if (!have_d && consumed < issued) {
                    tag_d = fetch_dn(ln, td0);
                    have_d = true;
                }
                // one slice of this segment out of t (tag tg): image of its expert, product, partial vector
                auto one = [&](const DataD &t, uint32_t tg) __attribute__((always_inline)) {
                    const uint32_t pc = (tg >> 28) & 7u, ul = tg & 0x0FFFFFFFu;
                    if (pc != k_cur) {
                        gg_read_image<GD::NREG>(img0 + pc * (uint32_t)IMG_DN, 4 * LPR_DN, lane, ar);
                        k_cur = pc;
                    }
                    float v = fm_chunk_sum<LPR_DN>(ln.dot(t, ar, ones));
                    if (!((valid >> pc) & 1u)) v = 0.0f;
                    const uint32_t rbi = ul - pc * c_nrb;
                    if (ch == 0)
                        fm_lds_w32(part0 + 4u * ((rbi * (uint32_t)K + pc) * RPS_DN + (uint32_t)ris), __float_as_uint(v));
                };
                while (have_d) {
                    if ((tag_d >> 31) != (uint32_t)(cq & 1)) break;      // the next segment's: it waits in td0
                    const bool more = consumed < issued;
                    uint32_t tag_n = 0u;
                    if (more) tag_n = fetch_dn(ln, td1);
                    one(td0, tag_d);
                    if (!more) {
                        have_d = false;
                        break;
                    }
                    if ((tag_n >> 31) != (uint32_t)(cq & 1)) {           // (once per segment at most)
                        td0 = td1;
                        tag_d = tag_n;
                        break;
                    }
                    have_d = consumed < issued;
                    if (have_d) tag_d = fetch_dn(ln, td0);
                    one(td1, tag_n);
                }
            }
            fm_wg_barrier();
            reduce_part(n_seq - 1);
        }
    }
};

template <int DN_KIND, int LPR_UP, int LPR_DN>
__global__ __launch_bounds__(512) void fm_gguf_fused_rows(GgufArgs a, Fm2Dims dm, Fm2Sync sy) {
#if defined(__HIP_DEVICE_COMPILE__)
    GgFused<DN_KIND, LPR_UP, LPR_DN> st(a, sy);
    st.run(dm);
#else
    (void)a;
    (void)dm;
    (void)sy;
#endif
}

// One launch for the whole operator; FM_ERR_UNSUPPORTED when the shape has no instance or the
// grid could not be resident at once (every workgroup may wait for another's activations).
template <int DN_KIND, int LPR_UP, int LPR_DN>
int gg_launch_fused_t(const GgufArgs &a, int n_pairs, const FmGg2Plan &plan, hipStream_t st, const Fm2Sync &sy) {
    using F = GgFused<DN_KIND, LPR_UP, LPR_DN>;
    auto kfn = fm_gguf_fused_rows<DN_KIND, LPR_UP, LPR_DN>;
    if ((uint32_t)F::LDS_BYTES != plan.lds_bytes || (uint32_t)F::RING_BYTES != plan.ring_bytes ||
        (uint32_t)F::IMG_BYTES != plan.img_bytes || F::RING_DN != plan.ring_dn)
        return FM_ERR_UNSUPPORTED;                     // (the plan and the kernel disagree: never expected)
    static FmLdsAttr attr;
    static int per_cu[64] = {};
    if (!fm_dyn_lds_ready(attr, (const void *)kfn, (size_t)F::LDS_BYTES)) return FM_ERR_HIP;
    int dev = 0;
    (void)hipGetDevice(&dev);
    const bool known = dev >= 0 && dev < 64;
    int pc = known ? per_cu[dev] : 0;
    if (pc == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&pc, kfn, 512, (size_t)F::LDS_BYTES) != hipSuccess) pc = 0;
        if (pc < 1) pc = -1;
        if (known) per_cu[dev] = pc;
    }
    if (pc < 1) return FM_ERR_UNSUPPORTED;
    const Fm2Dims dm = fm2_dims_units(n_pairs, a.K, plan.wgs, plan.gu_upp, plan.dn_upp, plan.gu_wt, plan.dn_wt);
    hipLaunchKernelGGL(kfn, dim3((unsigned)plan.wgs), dim3(512), (size_t)F::LDS_BYTES, st, a, dm, sy);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

int gg_launch_fused(const GgufArgs &a, int n_pairs, int n_cu, hipStream_t st, const Fm2Sync &sy) {
    if (a.g.gate_type != FM_GGML_Q4_K || a.g.up_type != FM_GGML_Q4_K) return FM_ERR_UNSUPPORTED;
    const bool q6 = a.g.down_type == FM_GGML_Q6_K;
    if (!q6 && a.g.down_type != FM_GGML_Q4_K) return FM_ERR_UNSUPPORTED;
    const FmGg2Plan plan = fm_gg2_plan(n_pairs, a.K, a.g.hidden, a.g.inter, q6 ? 1 : 0, n_cu);
    if (!plan.ok || plan.wgs > n_cu) return FM_ERR_UNSUPPORTED;
    if (q6 && plan.lpr_up == 16 && plan.lpr_dn == 8) return gg_launch_fused_t<GG_Q6, 16, 8>(a, n_pairs, plan, st, sy);
    if (q6 && plan.lpr_up == 8 && plan.lpr_dn == 4) return gg_launch_fused_t<GG_Q6, 8, 4>(a, n_pairs, plan, st, sy);
    if (!q6 && plan.lpr_up == 8 && plan.lpr_dn == 4) return gg_launch_fused_t<GG_Q4, 8, 4>(a, n_pairs, plan, st, sy);
    return FM_ERR_UNSUPPORTED;
}

// launch of one streaming phase; FM_ERR_UNSUPPORTED when the shape has no instance
template <int KIND, bool GU>
int gg_launch_stream(const GgufArgs &a, int n_pairs, int n_cu, hipStream_t st) {
    const int in_dim = GU ? a.g.hidden : a.g.inter, rows = GU ? a.g.inter : a.g.hidden;
    // a workgroup holds the images of 2 layers (gate/up) or 3 pairs (down): the plan keeps its
    // share of the units within that span
    const FmGgPlan plan = fm_gg_plan(n_pairs, a.K, in_dim, rows, KIND == GG_Q6, GU, n_cu);
    if (!plan.ok) return FM_ERR_UNSUPPORTED;
    const int lpr = plan.lpr, upp = plan.upp;
    const long total = plan.total, wgs = plan.wgs;
#define GG_STK(KK, L)                                                                          \
    do {                                                                                       \
        auto kfn = fm_gguf_stream<KK, L, GU>;                                                  \
        const size_t sh = gg_stream_lds<KK, L, GU>();                                          \
        static FmLdsAttr attr;                                                                 \
        if (!fm_dyn_lds_ready(attr, (const void *)kfn, sh)) return FM_ERR_HIP;                 \
        hipLaunchKernelGGL(kfn, dim3((unsigned)wgs), dim3(FM_GG_NW(KK == GG_Q6W) * 64), sh, st, a, (int)total, \
                           gg_div_make((uint32_t)upp), gg_div_make((uint32_t)a.K));   \
    } while (0)
#define GG_ST(L) GG_STK(KIND, L)
    if constexpr (KIND == GG_Q6 && !GU) {
        if (plan.wide) {
            GG_STK(GG_Q6W, 16);
            return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
        }
    }
    switch (lpr) {
        case 4: GG_ST(4); break;
        case 8: GG_ST(8); break;
        default: GG_ST(16); break;
    }
#undef GG_ST
#undef GG_STK
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

int pick_rpi(int rows, int n_pairs, int min_rows, int cap, int want) {
    int rpi = min_rows;
    while (rpi * 2 <= cap && rows % (rpi * 2) == 0 && (rows / (rpi * 2)) * n_pairs >= want) rpi *= 2;
    return rpi;
}

}  // namespace

extern "C" int fm_launch_decode_gguf(const uint8_t *const *d_gate, const uint8_t *const *d_up,
                                     const uint8_t *const *d_down, const FmGgufGeom *g, int layer0,
                                     int layer_stride, int n_layers, const float *d_x,
                                     const int32_t *d_idx, const float *d_w, int K, float *d_act,
                                     float *d_expert_out, float *d_out, FmDecodeFlags *df, int flags,
                                     int n_cu, hipStream_t st, hipEvent_t *kev) {
    GgufArgs a;
    a.direct = nullptr;
    a.gate = d_gate;
    a.up = d_up;
    a.down = d_down;
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
    a.flags = flags & ~FM_INT_NO_EXPERT_OUT;
    const int n_pairs = n_layers * K;
    // Without per-expert vectors, without the finite guard and outside a graph capture: one launch
    // (the activation sets alternate between launches exactly as for the affine experts; a
    // captured launch would need the graph's set and a fill kernel in front, and takes the three
    // kernels instead).
    // (The three streaming launches, twelve waves per workgroup, are the faster form of a longer
    // call: layers of a step 116.7 / 95.5 / 75.9 / 55.7 / 50.9 us as three against 121.3 / 97.4 /
    // 77.9 / 55.8 / 51.2 us as one at 40 / 32 / 24 / 16 / 14 layers, and 46.1 / 35.5 / 19.0 against
    // 45.7 / 34.9 / 15.7 us at 12 / 8 / 1; positions of a chunk 76.0 / 48.6 / 41.3 / 38.7 / 32.9
    // against 84.0 / 51.5 / 43.1 / 39.6 / 33.2 us at 32 / 16 / 12 / 10 / 8.)
    const bool phases = (fm_kernel_forms & (FM_FORM_PLAIN_GGUF | FM_FORM_GGUF_PHASES)) != 0 ||
                        (n_layers > fm_gg_one_launch_max(layer_stride) &&
                         !(fm_kernel_forms & FM_FORM_GGUF_ONE_LAUNCH));
    const unsigned int act_need = (unsigned int)n_pairs * (unsigned int)g->inter;
    if (!phases && !kev && df && (flags & FM_INT_NO_EXPERT_OUT) && !(flags & FM_GUARD) && df->act_set[0] &&
        df->act_cap >= act_need && !df->always_graph_set) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        (void)hipStreamIsCapturing(st, &capture);
        if (capture == hipStreamCaptureStatusNone) {
            Fm2Sync sy{};
            sy.act_other = df->act_set[df->act_parity ^ 1];
            sy.clear_n = df->act_used[df->act_parity ^ 1];
            sy.err = df->err;
            sy.spin_limit = df->spin_limit;
            GgufArgs af = a;
            af.act = df->act_set[df->act_parity];
            const int rc = gg_launch_fused(af, n_pairs, n_cu, st, sy);
            if (rc == FM_OK) {     // the set just filled is in use, the other one is all markers again
                df->act_used[df->act_parity] = act_need;
                df->act_used[df->act_parity ^ 1] = 0u;
                df->act_parity ^= 1;
                return FM_OK;
            }
            if (rc != FM_ERR_UNSUPPORTED) return rc;
        }
    }
    const int lpr_up = g->hidden / 128, lpr_down = g->inter / 128;
    auto pow2 = [](int v) { return v > 0 && (v & (v - 1)) == 0; };
    if (!pow2(lpr_up) || !pow2(lpr_down) || lpr_up < 2 || lpr_up > 64 || lpr_down < 2 || lpr_down > 64)
        return FM_ERR_UNSUPPORTED;
    const int min_up = 4 * (FM_WAVE / lpr_up), min_down = 4 * (FM_WAVE / lpr_down);
    if (g->inter % min_up || g->hidden % min_down) return FM_ERR_UNSUPPORTED;
    dim3 b(256);
    GgufArgs a1 = a, a2 = a;
    a1.rows_per_item = pick_rpi(g->inter, n_pairs, min_up, 64, 4 * n_cu);
    a1.items_per_pair = g->inter / a1.rows_per_item;
    a2.rows_per_item = pick_rpi(g->hidden, n_pairs, min_down, 256, 4 * n_cu);
    a2.items_per_pair = g->hidden / a2.rows_per_item;
    if (kev) (void)hipEventRecord(kev[0], st);
    const bool no_stream = (fm_kernel_forms & FM_FORM_PLAIN_GGUF) != 0;
    int rc_up = FM_ERR_UNSUPPORTED;
    if (!no_stream) rc_up = gg_launch_stream<GG_Q4, true>(a, n_pairs, n_cu, st);
    if (rc_up != FM_OK && rc_up != FM_ERR_UNSUPPORTED) return rc_up;
#define GG_UP(L) hipLaunchKernelGGL(fm_gguf_gate_up<L>, dim3(n_pairs * a1.items_per_pair), b, 0, st, a1)
    if (rc_up == FM_ERR_UNSUPPORTED) switch (lpr_up) {
        case 2: GG_UP(2); break;
        case 4: GG_UP(4); break;
        case 8: GG_UP(8); break;
        case 16: GG_UP(16); break;
        case 32: GG_UP(32); break;
        default: GG_UP(64); break;
    }
#undef GG_UP
    if (kev) (void)hipEventRecord(kev[1], st);
    const bool q6 = g->down_type == FM_GGML_Q6_K;
#define GG_DOWN(L)                                                                                    \
    do {                                                                                              \
        if (q6) hipLaunchKernelGGL((fm_gguf_down<L, true>), dim3(n_pairs * a2.items_per_pair), b, 0, st, a2); \
        else hipLaunchKernelGGL((fm_gguf_down<L, false>), dim3(n_pairs * a2.items_per_pair), b, 0, st, a2);   \
    } while (0)
    int rc_dn = FM_ERR_UNSUPPORTED;
    if (!no_stream) rc_dn = q6 ? gg_launch_stream<GG_Q6, false>(a, n_pairs, n_cu, st)
                               : gg_launch_stream<GG_Q4, false>(a, n_pairs, n_cu, st);
    if (rc_dn != FM_OK && rc_dn != FM_ERR_UNSUPPORTED) return rc_dn;
    if (rc_dn == FM_ERR_UNSUPPORTED) switch (lpr_down) {
        case 2: GG_DOWN(2); break;
        case 4: GG_DOWN(4); break;
        case 8: GG_DOWN(8); break;
        case 16: GG_DOWN(16); break;
        case 32: GG_DOWN(32); break;
        default: GG_DOWN(64); break;
    }
#undef GG_DOWN
    if (flags & FM_GUARD)
        hipLaunchKernelGGL(fm_gguf_combine<true>, dim3(n_layers), b, 0, st, a);
    else
        hipLaunchKernelGGL(fm_gguf_combine<false>, dim3(n_layers, (g->hidden + 255) / 256), b, 0, st, a);
    if (kev) (void)hipEventRecord(kev[2], st);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

extern "C" int fm_launch_gguf_matvec(const uint8_t *d_W, int ggml_type, const float *d_x,
                                     float *d_out, int out_dim, int in_dim, int, hipStream_t st) {
    const bool q6 = ggml_type == FM_GGML_Q6_K;
    const int hpr = in_dim / 128;
    // rows of up to 64 half blocks: 64 / hpr rows per wave step, a few steps per wave
    if (in_dim % 256 == 0 && hpr >= 2 && hpr <= 64 && (hpr & (hpr - 1)) == 0 && ((uintptr_t)d_x & 15) == 0) {
        const int rpw = FM_WAVE / hpr;
        int steps = 1;
        while (steps < 8 && (long)out_dim > 4L * rpw * steps * 2048) steps *= 2;
        const dim3 grid((unsigned)((out_dim + 4 * rpw * steps - 1) / (4 * rpw * steps))), b(256);
#define GG_MV(H)                                                                                          \
    do {                                                                                                  \
        if (q6) hipLaunchKernelGGL((fm_gguf_matvec_rows_k<true, H>), grid, b, 0, st, d_W, d_x, d_out, out_dim, steps);  \
        else hipLaunchKernelGGL((fm_gguf_matvec_rows_k<false, H>), grid, b, 0, st, d_W, d_x, d_out, out_dim, steps);    \
    } while (0)
        switch (hpr) {
            case 2: GG_MV(2); break;
            case 4: GG_MV(4); break;
            case 8: GG_MV(8); break;
            case 16: GG_MV(16); break;
            case 32: GG_MV(32); break;
            default: GG_MV(64); break;
        }
#undef GG_MV
        return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
    }
    dim3 grid((out_dim + 3) / 4), b(256);
    if (q6) hipLaunchKernelGGL(fm_gguf_matvec_k<true>, grid, b, 0, st, d_W, d_x, d_out, out_dim, in_dim);
    else hipLaunchKernelGGL(fm_gguf_matvec_k<false>, grid, b, 0, st, d_W, d_x, d_out, out_dim, in_dim);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

// One dense Q4_K / Q6_K tensor [out_dim][in_dim] times x (the vocabulary projection and the
// other block-format tensors of a GGUF model: lm_head_forward's block branch,
// finchmoe/infer.m:5738-5746; cpu_dequant_matvec with bits 10 / 11, finchmoe/infer.m:1684-1688).
// Shapes the streaming kernel covers (a lane per 128 Q4_K / 64 Q6_K values, 4 to 16 lanes per
// row, rows a multiple of the wave step, 16-byte aligned rows) take it — the tensor is its one
// "expert" —, the others the plain kernel.
extern "C" int fm_launch_gguf_dense(const uint8_t *d_W, int ggml_type, const float *d_x, float *d_out,
                                    int out_dim, int in_dim, int n_cu, hipStream_t st) {
    if (ggml_type != FM_GGML_Q4_K && ggml_type != FM_GGML_Q6_K) return FM_ERR_UNSUPPORTED;
    if (out_dim < 1 || in_dim < 256 || in_dim % 256) return FM_ERR_UNSUPPORTED;
    const bool no_stream = (fm_kernel_forms & FM_FORM_PLAIN_GGUF) != 0;
    const bool q6 = ggml_type == FM_GGML_Q6_K;
    if (!no_stream && ((uintptr_t)d_W & 15) == 0) {
        GgufArgs a{};
        a.g.hidden = out_dim;          // the down phase's names: rows = hidden, columns = inter
        a.g.inter = in_dim;
        a.g.n_experts = 1;
        a.K = 1;
        a.act = const_cast<float *>(d_x);
        a.expert_out = d_out;
        a.direct = d_W;
        const int rc = q6 ? gg_launch_stream<GG_Q6, false>(a, 1, n_cu, st) : gg_launch_stream<GG_Q4, false>(a, 1, n_cu, st);
        if (rc != FM_ERR_UNSUPPORTED) return rc;
    }
    return fm_launch_gguf_matvec(d_W, ggml_type, d_x, d_out, out_dim, in_dim, n_cu, st);
}
