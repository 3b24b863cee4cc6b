// fm_dequant.hip — materialise what the GEMV/GEMM kernels decode on the fly, for
// bit-exact checks: integer codes and fp32 weights of an affine tensor
// (finchmoe/infer.m:1720-1725, 1751-1757) or of GGUF Q4_K / Q6_K rows
// (finchmoe/infer.m:1604-1657).  One thread per weight; not a hot path.
#include "fm_common.h"

namespace {

// code and fp32 weight of element (r, col) of an affine tensor
__device__ __forceinline__ float fm_affine_elem(const uint8_t *W, const uint16_t *S, const uint16_t *B,
                                                int r, int col, int in_dim, int group_size, int bits,
                                                int scale_fp16, uint32_t &q) {
    if (bits == 3) {
        // 8 codes per 24-bit little-endian field (repack_experts.py:250-257)
        const uint8_t *p = W + (size_t)r * (in_dim * 3 / 8) + 3 * (col >> 3);
        uint32_t v = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
        q = (v >> (3 * (col & 7))) & 7u;
    } else {
        // LSB-first fields of a little-endian u32 (quantize_model.py:35-43)
        int vpu = 32 / bits;
        const uint32_t *p = reinterpret_cast<const uint32_t *>(W) + (size_t)r * (in_dim / vpu);
        q = (p[col / vpu] >> ((col % vpu) * bits)) & ((1u << bits) - 1u);
    }
    int ng = in_dim / group_size;
    uint32_t sbits = S[(size_t)r * ng + col / group_size];
    uint32_t bbits = B[(size_t)r * ng + col / group_size];
    float s = scale_fp16 ? fm_fp16_bits(sbits) : fm_bf16_lo(sbits);
    float b = scale_fp16 ? fm_fp16_bits(bbits) : fm_bf16_lo(bbits);
    // code * scale is exact in fp32 (<= 8 + 11 significant bits), so the sum
    // is rounded once whether or not the compiler contracts it into an FMA
    return (float)q * s + b;
}

__global__ void fm_dequant_affine_k(const uint8_t *W, const uint16_t *S, const uint16_t *B,
                                    int out_dim, int in_dim, int group_size, int bits,
                                    int scale_fp16, uint8_t *codes, float *w32,
                                    uint16_t *w16) {
    size_t n = (size_t)out_dim * in_dim;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (size_t)gridDim.x * blockDim.x) {
        int r = (int)(i / in_dim), col = (int)(i % in_dim);
        uint32_t q;
        float w = fm_affine_elem(W, S, B, r, col, in_dim, group_size, bits, scale_fp16, q);
        if (codes) codes[i] = (uint8_t)q;
        if (w32) w32[i] = w;
        if (w16) {
            _Float16 h = (_Float16)w;   // round-to-nearest-even
            w16[i] = __builtin_bit_cast(unsigned short, h);
        }
    }
}

// Embedding lookup: out[i] = dequantized row ids[i] of an affine tensor [rows][in_dim], one
// workgroup per id (embed_lookup, finchmoe/infer.m:5664-5722: the 4-/8-bit branch; a missing
// tensor gives zeros there, an id outside the tensor gives zeros here).
__global__ __launch_bounds__(256) void fm_embed_rows_k(const uint8_t *W, const uint16_t *S,
                                                       const uint16_t *B, int rows, int in_dim,
                                                       int group_size, int bits, int scale_fp16,
                                                       const int32_t *ids, float *out) {
    const int r = ids[blockIdx.x];
    float *o = out + (size_t)blockIdx.x * in_dim;
    for (int col = threadIdx.x; col < in_dim; col += blockDim.x) {
        uint32_t q;
        o[col] = (unsigned)r < (unsigned)rows
                     ? fm_affine_elem(W, S, B, r, col, in_dim, group_size, bits, scale_fp16, q)
                     : 0.0f;
    }
}

// finchmoe/infer.m:1595-1603
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t *s, int &sc, int &m) {
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (s[j + 4] & 0x0F) | ((s[j - 4] >> 6) << 4);
        m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

// fp32 value of element `col` of a Q4_K / Q6_K row (finchmoe/infer.m:1604-1657)
__device__ __forceinline__ float fm_gguf_elem(const uint8_t *row, int col, int ggml_type) {
    const int bsz = ggml_type == FM_GGML_Q4_K ? 144 : 210;
    const uint8_t *blk = row + (size_t)(col >> 8) * bsz;
    const int e = col & 255;
    if (ggml_type == FM_GGML_Q4_K) {
        float d = fm_fp16_bits(blk[0] | (blk[1] << 8));
        float dmin = fm_fp16_bits(blk[2] | (blk[3] << 8));
        int chunk = e >> 6, high = (e >> 5) & 1, l = e & 31;
        int sc, m;
        scale_min_k4(2 * chunk + high, blk + 4, sc, m);
        int nib = (blk[16 + 32 * chunk + l] >> (4 * high)) & 0xF;
        float d1 = d * (float)sc, m1 = dmin * (float)m;
        return d1 * (float)nib - m1;
    }
    float d = fm_fp16_bits(blk[208] | (blk[209] << 8));
    int half = e >> 7, vi = e & 127;
    int nib = (blk[64 * half + (vi & 63)] >> (4 * (vi >> 6))) & 0xF;
    int hi2 = (blk[128 + 32 * half + (vi & 31)] >> (2 * ((vi >> 5) & 3))) & 3;
    int sc = (int)(int8_t)blk[192 + 8 * half + (vi >> 4)];
    int q = (nib | (hi2 << 4)) - 32;
    return d * (float)sc * (float)q;
}

__global__ void fm_dequant_gguf_k(const uint8_t *W, int out_dim, int in_dim, int ggml_type,
                                  float *w32) {
    size_t n = (size_t)out_dim * in_dim;
    const size_t row_bytes = (size_t)(in_dim / 256) * (ggml_type == FM_GGML_Q4_K ? 144 : 210);
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (size_t)gridDim.x * blockDim.x) {
        int r = (int)(i / in_dim), col = (int)(i % in_dim);
        w32[i] = fm_gguf_elem(W + (size_t)r * row_bytes, col, ggml_type);
    }
}

// Embedding lookup in a Q4_K / Q6_K tensor: out[i] = dequantized row ids[i], one workgroup per
// id (embed_lookup's block-format branch, finchmoe/infer.m:5675-5683: gguf_dequant_row of the
// token's row); an id outside the tensor gives zeros.
__global__ __launch_bounds__(256) void fm_embed_rows_gguf_k(const uint8_t *W, int rows, int in_dim,
                                                            int ggml_type, const int32_t *ids, float *out) {
    const int r = ids[blockIdx.x];
    const size_t row_bytes = (size_t)(in_dim / 256) * (ggml_type == FM_GGML_Q4_K ? 144 : 210);
    float *o = out + (size_t)blockIdx.x * in_dim;
    for (int col = threadIdx.x; col < in_dim; col += blockDim.x)
        o[col] = (unsigned)r < (unsigned)rows ? fm_gguf_elem(W + (size_t)r * row_bytes, col, ggml_type) : 0.0f;
}

}  // namespace

extern "C" int fm_launch_dequant_affine(const void *W, const void *S, const void *B,
                                        int out_dim, int in_dim, int group_size, int bits,
                                        int scale_fp16, uint8_t *codes, float *w32,
                                        uint16_t *w16, hipStream_t st) {
    size_t n = (size_t)out_dim * in_dim;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 65535) blocks = 65535;
    hipLaunchKernelGGL(fm_dequant_affine_k, dim3(blocks), dim3(256), 0, st,
                       (const uint8_t *)W, (const uint16_t *)S, (const uint16_t *)B, out_dim,
                       in_dim, group_size, bits, scale_fp16, codes, w32, w16);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

extern "C" int fm_launch_embed_rows(const void *W, const void *S, const void *B, int rows, int in_dim,
                                    int group_size, int bits, int scale_fp16, const int32_t *d_ids,
                                    int n, float *d_out, hipStream_t st) {
    hipLaunchKernelGGL(fm_embed_rows_k, dim3(n), dim3(256), 0, st, (const uint8_t *)W,
                       (const uint16_t *)S, (const uint16_t *)B, rows, in_dim, group_size, bits,
                       scale_fp16, d_ids, d_out);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

extern "C" int fm_launch_dequant_gguf(const void *W, int out_dim, int in_dim, int ggml_type,
                                      float *w32, hipStream_t st) {
    size_t n = (size_t)out_dim * in_dim;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 65535) blocks = 65535;
    hipLaunchKernelGGL(fm_dequant_gguf_k, dim3(blocks), dim3(256), 0, st, (const uint8_t *)W,
                       out_dim, in_dim, ggml_type, w32);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

extern "C" int fm_launch_embed_rows_gguf(const void *W, int rows, int in_dim, int ggml_type,
                                         const int32_t *d_ids, int n, float *d_out, hipStream_t st) {
    hipLaunchKernelGGL(fm_embed_rows_gguf_k, dim3(n), dim3(256), 0, st, (const uint8_t *)W, rows, in_dim,
                       ggml_type, d_ids, d_out);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}
