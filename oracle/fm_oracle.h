/*
 * fm_oracle.h — CPU restatement of FinchMoE's quantized-expert hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker for the HIP path; it
 * is linked / loaded only by tests/, by __graft_entry__.smoke() and by the
 * cpu_baseline leg of bench.py.  The product library never calls into it and
 * has no CPU fallback.
 *
 * Every function names the reference lines (relative to /root/reference/) it
 * follows.  The restatement keeps the reference's evaluation order (fp32,
 * row-serial, sequential accumulate) so that it is the reference's CPU path
 * for timing purposes as well.
 *
 * Parity pins (what each function is checked against, see tests/test_oracle_*):
 *   every function below that has a twin in infer.m:686-702, 1575-1881 (widening,
 *   get_scale_min_k4, gguf_dequant_row, cpu_dequant_matvec at bits 3/4/8/10/11 and raw
 *   BF16, RMS norm, SwiGLU, softmax, top-K, normalise, vec_madd) is compared BIT FOR BIT
 *   with the reference's own C text compiled by build_ref.sh (oracle/_ref/libfm_ref.so,
 *   tests/test_oracle_ref.py).  Independently of that build:
 *   bf16/fp16 widening        exhaustive 65,536 values vs numpy
 *   3-bit / u32 packing       exhaustive 2^24 triplets pack<->unpack; closed form
 *   affine dequant            exactly-rounded closed form vs float64
 *   Q4_K / Q6_K dequant       row-loop form vs independent word-indexed form,
 *                             plus float64 closed form from the block fields.
 *                             The arithmetic originates in llama.cpp's
 *                             ggml-quants.c, which is not vendored in the
 *                             reference and has no pinned version there:
 *                             parity unpinned at the llama.cpp boundary,
 *                             pinned against the reference's two in-tree
 *                             restatements only.
 *   matvec                    float64 accumulation, scale=0 and one-hot cases
 *   softmax/top-k/normalise   brute force on small inputs, tie rule
 *   expert loop / combine     float64 recomputation, Inf-scale and w=0 injection
 *   quantizer (orc_quantize_affine)  golden vectors written by the reference's own
 *                             quantizers (tests/golden/quantizer_vectors.npz, made by
 *                             tests/golden/make_quantizer_vectors.py): codes, packed bytes,
 *                             scales and biases bit for bit, exact .5 ties and clamped
 *                             scales included.
 */
#ifndef FM_ORACLE_H
#define FM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORC_SCALE_BF16 = 0, ORC_SCALE_FP16 = 1 };
enum { ORC_GGML_Q4_K = 12, ORC_GGML_Q6_K = 14 };

/* Byte offsets of the nine components of one packed expert
 * (repack_experts.py:76-87,137-163; infer.m:174-234). */
typedef struct {
    size_t gate_w, gate_s, gate_b;
    size_t up_w, up_s, up_b;
    size_t down_w, down_s, down_b;
    size_t expert_size;
} orc_expert_layout;

void orc_expert_layout_affine(int hidden, int inter, int group_size, int bits,
                              orc_expert_layout *lo);

/* number widening (infer.m:690-702, 1579-1593) */
float    orc_bf16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16_trunc(float f);
float    orc_fp16_to_f32(uint16_t h);
uint16_t orc_f32_to_fp16_rne(float f);   /* defines "dequantized fp16 weight" */
uint16_t orc_f32_to_bf16_rne(float f);   /* activation rounding used by the prefill GEMM */

/* packers (repack_experts.py:242-257; quantize_model.py:35-43) */
void orc_pack_3bit(const uint8_t *codes, size_t n, uint8_t *out);
void orc_unpack_3bit(const uint8_t *packed, size_t n, uint8_t *codes);
void orc_pack_u32(const uint8_t *codes, size_t n, int bits, uint32_t *out);
void orc_unpack_u32(const uint32_t *packed, size_t n, int bits, uint8_t *codes);

/* quantizer (repack_experts.py:302-333) */
void orc_quantize_affine(const float *w, int out_dim, int in_dim, int group_size,
                         int bits, uint8_t *codes, uint16_t *scales, uint16_t *biases);

/* affine dequant of a whole [out_dim,in_dim] tensor (infer.m:1720-1725, 1756-1757) */
void orc_dequant_affine(const void *W, const uint16_t *S, const uint16_t *B,
                        int out_dim, int in_dim, int group_size, int bits,
                        int scale_dtype, uint8_t *codes, float *w_f32);

/* GGUF block formats (infer.m:1595-1657) */
void orc_get_scale_min_k4(int j, const uint8_t *scales, uint8_t *sc, uint8_t *m);
void orc_gguf_dequant_row(const void *row, float *y, int n, int ggml_type);
/* second, independent form: value of element e of one block, decoded the way
 * the word-indexed Metal kernels do (shaders.metal:3247-3293) */
float orc_gguf_block_value_wordform(const uint8_t *block, int e, int ggml_type);
size_t orc_gguf_row_bytes(int in_dim, int ggml_type);

/* matvec (infer.m:1660-1763).  bits in {1,2,3,4,8}: affine; 10/11: Q4_K/Q6_K;
 * S == NULL or B == NULL (and bits not 10/11): W is raw BF16 [out_dim][in_dim] */
void orc_dequant_matvec(const void *W, const uint16_t *S, const uint16_t *B,
                        const float *x, float *out, int out_dim, int in_dim,
                        int group_size, int bits, int scale_dtype);
/* same arithmetic per row, rows split over nthreads (bit-identical outputs) */
void orc_dequant_matvec_mt(const void *W, const uint16_t *S, const uint16_t *B,
                           const float *x, float *out, int out_dim, int in_dim,
                           int group_size, int bits, int scale_dtype, int nthreads);

/* activation, routing, combine (infer.m:1780-1851) */
void orc_swiglu(const float *gate, const float *up, float *out, int dim);
void orc_softmax(float *x, int dim);
void orc_topk(const float *scores, int dim, int K, int *indices, float *values);
void orc_normalize_weights(float *w, int K);
void orc_vec_madd(float *dst, const float *src, float scale, int dim);

/* routed-expert block, one position.
 *   guard = 1: CPU semantics of infer.m:10109-10204 — finite guard on each
 *              expert output, renormalise when 0 < sum(w) < 0.99.
 *   guard = 0: GPU semantics of moe_combine_residual (shaders.metal:2196-2231)
 *              — plain slot-order sum of w_k * out_k.
 * moe_out is accumulated into (+=), as the reference does; expert_out (may be
 * NULL) receives the K per-expert outputs [K][hidden]; gate_out/up_out/act_out
 * (may be NULL) the per-stage vectors [K][inter] (the --compare-experts
 * stages, infer.m:9767-10003). */
void orc_moe_experts_forward(const uint8_t *layer_blob, int hidden, int inter,
                             int group_size, int bits, int scale_dtype,
                             const float *x, const int *expert_idx,
                             const float *expert_w, int K, int guard,
                             float *moe_out, float *expert_out,
                             float *gate_out, float *up_out, float *act_out,
                             int nthreads);

/* infer.m:1766-1777 */
void orc_rms_norm(const float *x, const uint16_t *w_bf16, float *out, int dim, float eps);

/* The tail of a layer's expert command buffer (infer.m:9608-9760): shared-expert SwiGLU
 * and down projection, hidden = h_mid + sum_k params[k]*expert_out[k] +
 * sigmoid(params[8])*shared_out (shaders.metal:2196-2231), next layer's input RMS norm
 * with bf16 weights (shaders.metal:1134-1205).  params[10] as buf_combine_params. */
void orc_layer_tail(const void *sdW, const uint16_t *sdS, const uint16_t *sdB,
                    int hidden, int shared_inter, int group_size, int bits, int scale_dtype,
                    const float *h_mid, const float *expert_out, const float *params, int K,
                    const float *shared_gate, const float *shared_up,
                    const uint16_t *next_norm_w, float eps,
                    float *hidden_out, float *next_in);

/* GGUF routed-expert block (infer.m:3153-3347, CPU twin infer.m:10011-10099):
 * gate/up/down slabs are the stacked per-layer tensors, expert e at e*slab. */
void orc_moe_gguf_forward(const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                          int gate_type, int up_type, int down_type,
                          int hidden, int inter,
                          const float *x, const int *expert_idx,
                          const float *expert_w, int K, int guard,
                          float *moe_out, float *expert_out, int nthreads);

/* prefill numerics model: what a bf16-MFMA grouped GEMM is allowed to do —
 * weights dequantized in fp32 then RNE-rounded to bf16, activations rounded to
 * bf16, products accumulated in fp32 (order free).  Used to bound the GPU GEMM
 * against the per-token fp32 path. */
void orc_dequant_matvec_bf16model(const void *W, const uint16_t *S, const uint16_t *B,
                                  const float *x, float *out, int out_dim, int in_dim,
                                  int group_size, int bits, int scale_dtype);

#ifdef __cplusplus
}
#endif
#endif
