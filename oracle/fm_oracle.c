/*
 * fm_oracle.c — CPU restatement of FinchMoE's quantized-expert hot path.
 * TEST INFRASTRUCTURE ONLY (see fm_oracle.h).  Plain C99, no dependencies.
 *
 * Citations are relative to /root/reference/finchmoe/.
 */
#include "fm_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* number widening                                                     */
/* ------------------------------------------------------------------ */

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* infer.m:690-695 — bf16 is the top half of the fp32 pattern */
float orc_bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* infer.m:697-702, repack_experts.py:232-234 — narrowing truncates */
uint16_t orc_f32_to_bf16_trunc(float f) { return (uint16_t)(f32_to_bits(f) >> 16); }

/* infer.m:1579-1593 restates ggml's half->float.  The reference reaches the
 * IEEE value with a multiply trick; this restatement decodes the fields
 * directly, which gives the same value for every non-NaN half (checked
 * exhaustively against numpy.float16 in tests). */
float orc_fp16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 0x1.0p-24f;
        return bits_to_f32(f32_to_bits(v) | sign);
    }
    if (exp == 31) return bits_to_f32(sign | 0x7F800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even fp32 -> fp16; the reference never materialises fp16
 * weights, so "dequantized fp16 weight" is defined as RNE(fp32 dequant). */
uint16_t orc_f32_to_fp16_rne(float f) {
    uint32_t u = f32_to_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) {                       /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((a > 0x7F800000u) ? 0x200u : 0));
    }
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);   /* >= 65520 -> inf */
    if (a < 0x33000001u) return sign;             /* <= 2^-25 -> 0 (tie to even) */
    int e = (int)(a >> 23) - 127;
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u;     /* 24-bit significand */
    int shift;                                    /* bits dropped from m */
    uint32_t base;
    if (e >= -14) { shift = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7FFFFFu; }
    else          { shift = 13 + (-14 - e); base = 0; }
    uint32_t keep = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    uint32_t r = base + keep;
    if (rem > half || (rem == half && (r & 1u))) r += 1;
    return (uint16_t)(sign | r);
}

uint16_t orc_f32_to_bf16_rne(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float widen16(uint16_t h, int scale_dtype) {
    return scale_dtype == ORC_SCALE_FP16 ? orc_fp16_to_f32(h) : orc_bf16_to_f32(h);
}

/* ------------------------------------------------------------------ */
/* layout                                                              */
/* ------------------------------------------------------------------ */

/* repack_experts.py:76-87 (4-bit), 137-151 (3-bit), 153-163 (2-bit);
 * infer.m:174-234.  gate, up: [inter, hidden]; down: [hidden, inter];
 * each followed by its scales then biases, [rows, cols/group] 16-bit. */
void orc_expert_layout_affine(int hidden, int inter, int group_size, int bits,
                              orc_expert_layout *lo) {
    size_t gu_w = (size_t)inter * hidden * bits / 8;
    size_t gu_s = (size_t)inter * (hidden / group_size) * 2;
    size_t d_w = (size_t)hidden * inter * bits / 8;
    size_t d_s = (size_t)hidden * (inter / group_size) * 2;
    size_t o = 0;
    lo->gate_w = o; o += gu_w; lo->gate_s = o; o += gu_s; lo->gate_b = o; o += gu_s;
    lo->up_w = o;   o += gu_w; lo->up_s = o;   o += gu_s; lo->up_b = o;   o += gu_s;
    lo->down_w = o; o += d_w;  lo->down_s = o; o += d_s;  lo->down_b = o; o += d_s;
    lo->expert_size = o;
}

/* ------------------------------------------------------------------ */
/* packers                                                             */
/* ------------------------------------------------------------------ */

/* repack_experts.py:242-257 — 8 codes -> one 24-bit little-endian field,
 * code j at bits 3j..3j+2 */
void orc_pack_3bit(const uint8_t *codes, size_t n, uint8_t *out) {
    for (size_t t = 0; t < n / 8; t++) {
        uint32_t v = 0;
        for (int j = 0; j < 8; j++) v |= (uint32_t)(codes[8 * t + j] & 7u) << (3 * j);
        out[3 * t + 0] = (uint8_t)(v & 0xFF);
        out[3 * t + 1] = (uint8_t)((v >> 8) & 0xFF);
        out[3 * t + 2] = (uint8_t)((v >> 16) & 0xFF);
    }
}

/* infer.m:1720-1725 */
void orc_unpack_3bit(const uint8_t *packed, size_t n, uint8_t *codes) {
    for (size_t t = 0; t < n / 8; t++) {
        uint32_t v = (uint32_t)packed[3 * t] | ((uint32_t)packed[3 * t + 1] << 8) |
                     ((uint32_t)packed[3 * t + 2] << 16);
        for (int j = 0; j < 8; j++) codes[8 * t + j] = (uint8_t)((v >> (3 * j)) & 7u);
    }
}

/* quantize_model.py:35-43, repack_experts.py:321-330 — value v of word u sits
 * at bit v*bits, LSB first */
void orc_pack_u32(const uint8_t *codes, size_t n, int bits, uint32_t *out) {
    int vpu = 32 / bits;
    uint32_t mask = bits == 32 ? 0xFFFFFFFFu : ((1u << bits) - 1u);
    for (size_t u = 0; u < n / (size_t)vpu; u++) {
        uint32_t w = 0;
        for (int v = 0; v < vpu; v++) w |= ((uint32_t)codes[u * vpu + v] & mask) << (v * bits);
        out[u] = w;
    }
}

/* infer.m:1751-1757 */
void orc_unpack_u32(const uint32_t *packed, size_t n, int bits, uint8_t *codes) {
    int vpu = 32 / bits;
    uint32_t mask = (1u << bits) - 1u;
    for (size_t u = 0; u < n / (size_t)vpu; u++)
        for (int v = 0; v < vpu; v++)
            codes[u * vpu + v] = (uint8_t)((packed[u] >> (v * bits)) & mask);
}

/* repack_experts.py:302-317 — per-group affine quantizer.  numpy evaluates
 * (w_max - w_min) / max_val, maximum(.,1e-8), (w - bias) / scale and
 * round-half-even in float32; rintf in the default rounding mode is
 * round-half-even.  Stored scale/bias are truncated to bf16 AFTER the codes
 * are computed (repack_experts.py:331-333). */
void orc_quantize_affine(const float *w, int out_dim, int in_dim, int group_size,
                         int bits, uint8_t *codes, uint16_t *scales, uint16_t *biases) {
    int ng = in_dim / group_size;
    float maxv = (float)((1 << bits) - 1);
    for (int r = 0; r < out_dim; r++) {
        for (int g = 0; g < ng; g++) {
            const float *p = w + (size_t)r * in_dim + (size_t)g * group_size;
            float lo = p[0], hi = p[0];
            for (int i = 1; i < group_size; i++) {
                if (p[i] < lo) lo = p[i];
                if (p[i] > hi) hi = p[i];
            }
            volatile float range = hi - lo;
            volatile float sc = range / maxv;
            float scale = sc > 1e-8f ? sc : 1e-8f;
            for (int i = 0; i < group_size; i++) {
                volatile float d = p[i] - lo;
                volatile float qf = d / scale;
                float q = rintf(qf);
                if (q < 0.0f) q = 0.0f;
                if (q > maxv) q = maxv;
                codes[(size_t)r * in_dim + (size_t)g * group_size + i] = (uint8_t)q;
            }
            scales[(size_t)r * ng + g] = orc_f32_to_bf16_trunc(scale);
            biases[(size_t)r * ng + g] = orc_f32_to_bf16_trunc(lo);
        }
    }
}

/* ------------------------------------------------------------------ */
/* affine dequant of a whole tensor                                    */
/* ------------------------------------------------------------------ */

/* infer.m:1716-1727 (3-bit) and 1745-1759 (u32-packed): fp32
 * (float)code * scale + bias with the group's widened scale and bias. */
void orc_dequant_affine(const void *W, const uint16_t *S, const uint16_t *B,
                        int out_dim, int in_dim, int group_size, int bits,
                        int scale_dtype, uint8_t *codes, float *w_f32) {
    int ng = in_dim / group_size;
    for (int r = 0; r < out_dim; r++) {
        for (int i = 0; i < in_dim; i++) {
            uint32_t q;
            if (bits == 3) {
                const uint8_t *row = (const uint8_t *)W + (size_t)r * (in_dim * 3 / 8);
                int t = i / 8, j = i % 8;
                uint32_t v = (uint32_t)row[3 * t] | ((uint32_t)row[3 * t + 1] << 8) |
                             ((uint32_t)row[3 * t + 2] << 16);
                q = (v >> (3 * j)) & 7u;
            } else {
                int vpu = 32 / bits;
                const uint32_t *row = (const uint32_t *)W + (size_t)r * (in_dim / vpu);
                q = (row[i / vpu] >> ((i % vpu) * bits)) & ((1u << bits) - 1u);
            }
            int g = i / group_size;
            float scale = widen16(S[(size_t)r * ng + g], scale_dtype);
            float bias = widen16(B[(size_t)r * ng + g], scale_dtype);
            if (codes) codes[(size_t)r * in_dim + i] = (uint8_t)q;
            if (w_f32) w_f32[(size_t)r * in_dim + i] = (float)q * scale + bias;
        }
    }
}

/* ------------------------------------------------------------------ */
/* GGUF block formats                                                  */
/* ------------------------------------------------------------------ */

/* infer.m:1595-1603 — 6-bit (scale, min) pair j of a Q4_K block's 12 bytes */
void orc_get_scale_min_k4(int j, const uint8_t *s, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = s[j] & 63;
        *m = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4));
        *m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

size_t orc_gguf_row_bytes(int in_dim, int ggml_type) {
    return (size_t)(in_dim / 256) * (ggml_type == ORC_GGML_Q4_K ? 144u : 210u);
}

/* infer.m:1604-1657 — row-loop dequant of Q4_K (144 B / 256) and Q6_K
 * (210 B / 256) blocks */
void orc_gguf_dequant_row(const void *row, float *y, int n, int ggml_type) {
    const uint8_t *p = (const uint8_t *)row;
    int nb = n / 256;
    if (ggml_type == ORC_GGML_Q4_K) {
        for (int b = 0; b < nb; b++, p += 144, y += 256) {
            uint16_t dh, mh;
            memcpy(&dh, p, 2);
            memcpy(&mh, p + 2, 2);
            float d = orc_fp16_to_f32(dh), dmin = orc_fp16_to_f32(mh);
            const uint8_t *sc12 = p + 4;
            const uint8_t *q = p + 16;
            for (int c = 0; c < 4; c++, q += 32) {       /* 4 chunks of 64 values */
                uint8_t s0, m0, s1, m1;
                orc_get_scale_min_k4(2 * c, sc12, &s0, &m0);
                orc_get_scale_min_k4(2 * c + 1, sc12, &s1, &m1);
                float d1 = d * s0, mm1 = dmin * m0;
                float d2 = d * s1, mm2 = dmin * m1;
                for (int l = 0; l < 32; l++) y[64 * c + l] = d1 * (q[l] & 0x0F) - mm1;
                for (int l = 0; l < 32; l++) y[64 * c + 32 + l] = d2 * (q[l] >> 4) - mm2;
            }
        }
    } else if (ggml_type == ORC_GGML_Q6_K) {
        for (int b = 0; b < nb; b++, p += 210) {
            uint16_t dh;
            memcpy(&dh, p + 208, 2);
            float d = orc_fp16_to_f32(dh);
            const uint8_t *ql = p, *qh = p + 128;
            const int8_t *sc = (const int8_t *)(p + 192);
            for (int half = 0; half < 2; half++, y += 128, ql += 64, qh += 32, sc += 8) {
                for (int l = 0; l < 32; l++) {
                    int is = l / 16;
                    int q1 = (int)((ql[l] & 0x0F) | (((qh[l] >> 0) & 3) << 4)) - 32;
                    int q2 = (int)((ql[l + 32] & 0x0F) | (((qh[l] >> 2) & 3) << 4)) - 32;
                    int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                    int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                    y[l]      = d * sc[is + 0] * (float)q1;
                    y[l + 32] = d * sc[is + 2] * (float)q2;
                    y[l + 64] = d * sc[is + 4] * (float)q3;
                    y[l + 96] = d * sc[is + 6] * (float)q4;
                }
            }
        }
    }
}

/* shaders.metal:3247-3293 — the word-indexed decode: element e belongs to the
 * 8-value word wb = e/8 of its block. */
float orc_gguf_block_value_wordform(const uint8_t *b, int e, int ggml_type) {
    int wb = e >> 3, i = e & 7;
    if (ggml_type == ORC_GGML_Q4_K) {
        uint16_t dh, mh;
        memcpy(&dh, b, 2);
        memcpy(&mh, b + 2, 2);
        float d = orc_fp16_to_f32(dh), dmin = orc_fp16_to_f32(mh);
        int j = (wb >> 3) * 2 + ((wb >> 2) & 1);
        int high = (wb >> 2) & 1;
        uint8_t sc, m;
        orc_get_scale_min_k4(j, b + 4, &sc, &m);
        float dsc = d * (float)sc, mm = dmin * (float)m;
        uint64_t qbytes;
        memcpy(&qbytes, b + 16 + 32 * (wb >> 3) + 8 * (wb & 3), 8);
        unsigned nib = (unsigned)((qbytes >> (8 * i + 4 * high)) & 0xF);
        return (float)nib * dsc - mm;
    } else {
        int chunk = wb >> 4, wbp = wb & 15;
        uint16_t dh;
        memcpy(&dh, b + 208, 2);
        float d = orc_fp16_to_f32(dh);
        int sc = (int)b[192 + chunk * 8 + (wbp >> 1)];
        if (sc >= 128) sc -= 256;
        float dsc = d * (float)sc;
        int vi = wbp * 8 + i;
        int qb = chunk * 64 + (vi & 63);
        int hb = chunk * 32 + (vi & 31);
        int sh = 2 * ((vi >> 5) & 3);
        unsigned nib = (b[qb] >> (4 * ((vi >> 6) & 1))) & 0xF;
        unsigned qraw = nib | (((b[128 + hb] >> sh) & 3u) << 4);
        return dsc * ((float)qraw - 32.0f);
    }
}

/* ------------------------------------------------------------------ */
/* matvec                                                              */
/* ------------------------------------------------------------------ */

/* infer.m:1660-1674 — dequant a row then dot.  (The reference keeps a static
 * scratch row and is not re-entrant; this one allocates per call.) */
static void gguf_matvec_rows(const uint8_t *W, const float *x, float *out,
                             int r0, int r1, int in_dim, int ggml_type) {
    size_t rb = orc_gguf_row_bytes(in_dim, ggml_type);
    float *y = (float *)malloc((size_t)in_dim * sizeof(float));
    for (int r = r0; r < r1; r++) {
        orc_gguf_dequant_row(W + (size_t)r * rb, y, in_dim, ggml_type);
        float acc = 0.0f;
        for (int i = 0; i < in_dim; i++) acc += y[i] * x[i];
        out[r] = acc;
    }
    free(y);
}

/* infer.m:1676-1763 for rows [r0, r1) */
static void matvec_rows(const void *W, const uint16_t *S, const uint16_t *B,
                        const float *x, float *out, int r0, int r1, int in_dim,
                        int group_size, int bits, int scale_dtype) {
    if (bits == 10 || bits == 11) {
        gguf_matvec_rows((const uint8_t *)W, x, out, r0, r1, in_dim,
                         bits == 10 ? ORC_GGML_Q4_K : ORC_GGML_Q6_K);
        return;
    }
    /* infer.m:1689-1701 — scales == NULL (or biases == NULL) means an unquantized BF16
     * weight [out_dim][in_dim]; checked after the GGUF types, as upstream */
    if (!S || !B) {
        const uint16_t *wb = (const uint16_t *)W;
        for (int r = r0; r < r1; r++) {
            const uint16_t *wr = wb + (size_t)r * in_dim;
            float acc = 0.0f;
            for (int i = 0; i < in_dim; i++) acc += orc_bf16_to_f32(wr[i]) * x[i];
            out[r] = acc;
        }
        return;
    }
    int ng = in_dim / group_size;
    if (bits == 3) {
        int trip = in_dim / 8, tpg = group_size / 8;
        size_t rb = (size_t)in_dim * 3 / 8;
        for (int r = r0; r < r1; r++) {
            const uint8_t *wr = (const uint8_t *)W + (size_t)r * rb;
            const uint16_t *sr = S + (size_t)r * ng, *br = B + (size_t)r * ng;
            float acc = 0.0f;
            for (int t = 0; t < trip; t++) {
                float scale = widen16(sr[t / tpg], scale_dtype);
                float bias = widen16(br[t / tpg], scale_dtype);
                uint32_t v = (uint32_t)wr[3 * t] | ((uint32_t)wr[3 * t + 1] << 8) |
                             ((uint32_t)wr[3 * t + 2] << 16);
                for (int j = 0; j < 8; j++) {
                    float w = (float)((v >> (3 * j)) & 7u) * scale + bias;
                    acc += w * x[8 * t + j];
                }
            }
            out[r] = acc;
        }
        return;
    }
    int vpu = 32 / bits, ppg = group_size / vpu, pcols = in_dim / vpu;
    uint32_t mask = (1u << bits) - 1u;
    for (int r = r0; r < r1; r++) {
        const uint32_t *wr = (const uint32_t *)W + (size_t)r * pcols;
        const uint16_t *sr = S + (size_t)r * ng, *br = B + (size_t)r * ng;
        float acc = 0.0f;
        for (int g = 0; g < ng; g++) {
            float scale = widen16(sr[g], scale_dtype);
            float bias = widen16(br[g], scale_dtype);
            for (int p = 0; p < ppg; p++) {
                uint32_t word = wr[g * ppg + p];
                const float *xp = x + g * group_size + p * vpu;
                for (int n = 0; n < vpu; n++) {
                    float w = (float)((word >> (n * bits)) & mask) * scale + bias;
                    acc += w * xp[n];
                }
            }
        }
        out[r] = acc;
    }
}

void orc_dequant_matvec(const void *W, const uint16_t *S, const uint16_t *B,
                        const float *x, float *out, int out_dim, int in_dim,
                        int group_size, int bits, int scale_dtype) {
    matvec_rows(W, S, B, x, out, 0, out_dim, in_dim, group_size, bits, scale_dtype);
}

typedef struct {
    const void *W; const uint16_t *S, *B; const float *x; float *out;
    int r0, r1, in_dim, group_size, bits, scale_dtype;
} mv_job;

static void *mv_thread(void *p) {
    mv_job *j = (mv_job *)p;
    matvec_rows(j->W, j->S, j->B, j->x, j->out, j->r0, j->r1, j->in_dim,
                j->group_size, j->bits, j->scale_dtype);
    return NULL;
}

void orc_dequant_matvec_mt(const void *W, const uint16_t *S, const uint16_t *B,
                           const float *x, float *out, int out_dim, int in_dim,
                           int group_size, int bits, int scale_dtype, int nthreads) {
    if (nthreads <= 1) {
        orc_dequant_matvec(W, S, B, x, out, out_dim, in_dim, group_size, bits, scale_dtype);
        return;
    }
    if (nthreads > 256) nthreads = 256;
    pthread_t th[256];
    mv_job jobs[256];
    int per = (out_dim + nthreads - 1) / nthreads;
    int n = 0;
    for (int t = 0; t < nthreads; t++) {
        int r0 = t * per, r1 = r0 + per > out_dim ? out_dim : r0 + per;
        if (r0 >= r1) break;
        jobs[n] = (mv_job){W, S, B, x, out, r0, r1, in_dim, group_size, bits, scale_dtype};
        pthread_create(&th[n], NULL, mv_thread, &jobs[n]);
        n++;
    }
    for (int t = 0; t < n; t++) pthread_join(th[t], NULL);
}

/* bf16-operand numerics model of the grouped prefill GEMM (no reference
 * counterpart: the reference runs per-position fp32 GEMVs,
 * infer.m:10704-10765).  fp32 dequant -> RNE bf16 weight; x -> RNE bf16;
 * exact products accumulated in double then rounded once. */
void orc_dequant_matvec_bf16model(const void *W, const uint16_t *S, const uint16_t *B,
                                  const float *x, float *out, int out_dim, int in_dim,
                                  int group_size, int bits, int scale_dtype) {
    float *w = (float *)malloc((size_t)in_dim * sizeof(float));
    float *xr = (float *)malloc((size_t)in_dim * sizeof(float));
    for (int i = 0; i < in_dim; i++) xr[i] = orc_bf16_to_f32(orc_f32_to_bf16_rne(x[i]));
    int ng = in_dim / group_size;
    for (int r = 0; r < out_dim; r++) {
        const void *wr;
        if (bits == 3) wr = (const uint8_t *)W + (size_t)r * (in_dim * 3 / 8);
        else wr = (const uint32_t *)W + (size_t)r * (in_dim / (32 / bits));
        orc_dequant_affine(wr, S + (size_t)r * ng, B + (size_t)r * ng, 1, in_dim,
                           group_size, bits, scale_dtype, NULL, w);
        double acc = 0.0;
        for (int i = 0; i < in_dim; i++)
            acc += (double)orc_bf16_to_f32(orc_f32_to_bf16_rne(w[i])) * (double)xr[i];
        out[r] = (float)acc;
    }
    free(w);
    free(xr);
}

/* ------------------------------------------------------------------ */
/* activation, routing, combine                                        */
/* ------------------------------------------------------------------ */

/* infer.m:1780-1786 */
void orc_swiglu(const float *gate, const float *up, float *out, int dim) {
    for (int i = 0; i < dim; i++) {
        float g = gate[i];
        out[i] = (g / (1.0f + expf(-g))) * up[i];
    }
}

/* infer.m:1794-1808 */
void orc_softmax(float *x, int dim) {
    float mx = x[0];
    for (int i = 1; i < dim; i++) if (x[i] > mx) mx = x[i];
    float sum = 0.0f;
    for (int i = 0; i < dim; i++) { x[i] = expf(x[i] - mx); sum += x[i]; }
    float inv = 1.0f / sum;
    for (int i = 0; i < dim; i++) x[i] *= inv;
}

/* infer.m:1811-1830 — K slots start at -1e30; each score replaces the slot
 * holding the current minimum (first such slot on ties) iff it is strictly
 * greater.  Slot order is therefore NOT sorted. */
void orc_topk(const float *scores, int dim, int K, int *indices, float *values) {
    for (int k = 0; k < K; k++) { values[k] = -1e30f; indices[k] = 0; }
    for (int i = 0; i < dim; i++) {
        int mn = 0;
        for (int k = 1; k < K; k++) if (values[k] < values[mn]) mn = k;
        if (scores[i] > values[mn]) { values[mn] = scores[i]; indices[mn] = i; }
    }
}

/* infer.m:1833-1840 */
void orc_normalize_weights(float *w, int K) {
    float sum = 0.0f;
    for (int k = 0; k < K; k++) sum += w[k];
    if (sum > 0.0f) {
        float inv = 1.0f / sum;
        for (int k = 0; k < K; k++) w[k] *= inv;
    }
}

/* infer.m:1849-1851 */
void orc_vec_madd(float *dst, const float *src, float scale, int dim) {
    for (int i = 0; i < dim; i++) dst[i] += scale * src[i];
}

/* ------------------------------------------------------------------ */
/* layer tail: shared expert, combine with residual, next layer's norm */
/* ------------------------------------------------------------------ */

/* infer.m:1766-1777 */
void orc_rms_norm(const float *x, const uint16_t *w_bf16, float *out, int dim, float eps) {
    float sum_sq = 0.0f;
    for (int i = 0; i < dim; i++) sum_sq += x[i] * x[i];
    float rms = sqrtf(sum_sq / dim + eps);
    float inv_rms = 1.0f / rms;
    for (int i = 0; i < dim; i++) out[i] = x[i] * inv_rms * orc_bf16_to_f32(w_bf16[i]);
}

/* What CMD3 appends after the routed experts (infer.m:9608-9760): SwiGLU of the
 * shared expert's gate/up outputs (1780-1786), its down projection (1676-1763),
 * hidden = h_mid + sum_k params[k] * expert_out[k] + sigmoid(params[8]) * shared_out
 * in slot order (shaders.metal:2196-2231; CPU twin infer.m:7390-7412), then the
 * next layer's input norm (1766-1777; shaders.metal:1134-1205).  next_in may be NULL. */
void orc_layer_tail(const void *sdW, const uint16_t *sdS, const uint16_t *sdB,
                    int hidden, int shared_inter, int group_size, int bits, int scale_dtype,
                    const float *h_mid, const float *expert_out, const float *params, int K,
                    const float *shared_gate, const float *shared_up,
                    const uint16_t *next_norm_w, float eps,
                    float *hidden_out, float *next_in) {
    float *act = (float *)malloc((size_t)shared_inter * sizeof(float));
    float *shared_out = (float *)malloc((size_t)hidden * sizeof(float));
    orc_swiglu(shared_gate, shared_up, act, shared_inter);
    orc_dequant_matvec(sdW, sdS, sdB, act, shared_out, hidden, shared_inter, group_size, bits,
                       scale_dtype);
    float shared_w = 1.0f / (1.0f + expf(-params[8]));
    for (int i = 0; i < hidden; i++) {
        float moe = 0.0f;
        for (int k = 0; k < K; k++) moe += params[k] * expert_out[(size_t)k * hidden + i];
        hidden_out[i] = h_mid[i] + moe + shared_w * shared_out[i];
    }
    if (next_in && next_norm_w) orc_rms_norm(hidden_out, next_norm_w, next_in, hidden, eps);
    free(act);
    free(shared_out);
}

/* ------------------------------------------------------------------ */
/* routed-expert block                                                 */
/* ------------------------------------------------------------------ */

/* combine step shared by both formats.
 * guard=1: infer.m:10190-10204 / 3334-3347; guard=0: shaders.metal:2213-2228 */
static void combine_one(float *moe_out, const float *eo, float w, int hidden,
                        int guard, float *total_w) {
    if (guard) {
        float er = 0.0f;
        for (int j = 0; j < hidden; j++) er += eo[j] * eo[j];
        if (isfinite(er) && er < 1e20f) {
            orc_vec_madd(moe_out, eo, w, hidden);
            *total_w += w;
        }
    } else {
        for (int j = 0; j < hidden; j++) moe_out[j] += w * eo[j];
    }
}

static void renorm(float *moe_out, int hidden, int guard, float total_w) {
    if (guard && total_w > 0.0f && total_w < 0.99f) {
        float inv = 1.0f / total_w;
        for (int i = 0; i < hidden; i++) moe_out[i] *= inv;
    }
}

/* infer.m:10114-10204: per expert k in slot order: gate matvec, up matvec,
 * SwiGLU, down matvec, guarded weighted accumulate. */
void orc_moe_experts_forward(const uint8_t *layer_blob, int hidden, int inter,
                             int group_size, int bits, int scale_dtype,
                             const float *x, const int *expert_idx,
                             const float *expert_w, int K, int guard,
                             float *moe_out, float *expert_out,
                             float *gate_out, float *up_out, float *act_out,
                             int nthreads) {
    orc_expert_layout lo;
    orc_expert_layout_affine(hidden, inter, group_size, bits, &lo);
    float *g = (float *)malloc((size_t)inter * sizeof(float));
    float *u = (float *)malloc((size_t)inter * sizeof(float));
    float *a = (float *)malloc((size_t)inter * sizeof(float));
    float *eo = (float *)malloc((size_t)hidden * sizeof(float));
    float total_w = 0.0f;
    for (int k = 0; k < K; k++) {
        const uint8_t *e = layer_blob + (size_t)expert_idx[k] * lo.expert_size;
        orc_dequant_matvec_mt(e + lo.gate_w, (const uint16_t *)(e + lo.gate_s),
                              (const uint16_t *)(e + lo.gate_b), x, g, inter, hidden,
                              group_size, bits, scale_dtype, nthreads);
        orc_dequant_matvec_mt(e + lo.up_w, (const uint16_t *)(e + lo.up_s),
                              (const uint16_t *)(e + lo.up_b), x, u, inter, hidden,
                              group_size, bits, scale_dtype, nthreads);
        orc_swiglu(g, u, a, inter);
        orc_dequant_matvec_mt(e + lo.down_w, (const uint16_t *)(e + lo.down_s),
                              (const uint16_t *)(e + lo.down_b), a, eo, hidden, inter,
                              group_size, bits, scale_dtype, nthreads);
        if (gate_out) memcpy(gate_out + (size_t)k * inter, g, (size_t)inter * sizeof(float));
        if (up_out) memcpy(up_out + (size_t)k * inter, u, (size_t)inter * sizeof(float));
        if (act_out) memcpy(act_out + (size_t)k * inter, a, (size_t)inter * sizeof(float));
        if (expert_out) memcpy(expert_out + (size_t)k * hidden, eo, (size_t)hidden * sizeof(float));
        combine_one(moe_out, eo, expert_w[k], hidden, guard, &total_w);
    }
    renorm(moe_out, hidden, guard, total_w);
    free(g); free(u); free(a); free(eo);
}

/* infer.m:3153-3347 (GPU form) and its CPU twin 10011-10099: Q4_K/Q6_K slabs,
 * expert e at e*slab within each stacked tensor. */
void orc_moe_gguf_forward(const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                          int gate_type, int up_type, int down_type,
                          int hidden, int inter,
                          const float *x, const int *expert_idx,
                          const float *expert_w, int K, int guard,
                          float *moe_out, float *expert_out, int nthreads) {
    size_t gslab = (size_t)inter * orc_gguf_row_bytes(hidden, gate_type);
    size_t uslab = (size_t)inter * orc_gguf_row_bytes(hidden, up_type);
    size_t dslab = (size_t)hidden * orc_gguf_row_bytes(inter, down_type);
    float *g = (float *)malloc((size_t)inter * sizeof(float));
    float *u = (float *)malloc((size_t)inter * sizeof(float));
    float *a = (float *)malloc((size_t)inter * sizeof(float));
    float *eo = (float *)malloc((size_t)hidden * sizeof(float));
    float total_w = 0.0f;
    for (int k = 0; k < K; k++) {
        size_t e = (size_t)expert_idx[k];
        orc_dequant_matvec_mt(gate + e * gslab, NULL, NULL, x, g, inter, hidden, 0,
                              gate_type == ORC_GGML_Q4_K ? 10 : 11, 0, nthreads);
        orc_dequant_matvec_mt(up + e * uslab, NULL, NULL, x, u, inter, hidden, 0,
                              up_type == ORC_GGML_Q4_K ? 10 : 11, 0, nthreads);
        orc_swiglu(g, u, a, inter);
        orc_dequant_matvec_mt(down + e * dslab, NULL, NULL, a, eo, hidden, inter, 0,
                              down_type == ORC_GGML_Q4_K ? 10 : 11, 0, nthreads);
        if (expert_out) memcpy(expert_out + (size_t)k * hidden, eo, (size_t)hidden * sizeof(float));
        combine_one(moe_out, eo, expert_w[k], hidden, guard, &total_w);
    }
    renorm(moe_out, hidden, guard, total_w);
    free(g); free(u); free(a); free(eo);
}
