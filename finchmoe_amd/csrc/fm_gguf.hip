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
#include "fm_unpack.h"

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
                                     float *d_expert_out, float *d_out, unsigned int *, int flags,
                                     int n_cu, hipStream_t st, hipEvent_t *kev) {
    GgufArgs a;
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
    a.flags = flags;
    const int n_pairs = n_layers * K;
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
#define GG_UP(L) hipLaunchKernelGGL(fm_gguf_gate_up<L>, dim3(n_pairs * a1.items_per_pair), b, 0, st, a1)
    switch (lpr_up) {
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
    switch (lpr_down) {
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
    dim3 grid((out_dim + 3) / 4), b(256);
    if (ggml_type == FM_GGML_Q6_K)
        hipLaunchKernelGGL(fm_gguf_matvec_k<true>, grid, b, 0, st, d_W, d_x, d_out, out_dim, in_dim);
    else
        hipLaunchKernelGGL(fm_gguf_matvec_k<false>, grid, b, 0, st, d_W, d_x, d_out, out_dim, in_dim);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}
