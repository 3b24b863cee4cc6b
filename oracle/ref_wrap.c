/*
 * ref_wrap.c — exported names around the reference's own CPU functions.
 *
 * TEST INFRASTRUCTURE ONLY.  build_ref.sh cuts the dependency-free C functions of the
 * path out of the reference where it lies (finchmoe/infer.m:686-702 bf16 widening,
 * 1575-1881 GGUF block decode, cpu_dequant_matvec, RMS norm, SwiGLU, softmax, top-K,
 * normalise, vec_madd) into a temporary file and compiles this wrapper with REF_BODY
 * naming it; the reference's text is never stored in this repository and only the
 * built library lands in oracle/_ref/.  The functions are `static` in the reference,
 * so each gets an exported twin here; nothing else is added and no stand-in header is
 * needed (the cut needs <stdint.h> <string.h> <math.h> <stdlib.h> only).
 *
 * Used by tests/test_oracle_ref.py to pin the restatement in fm_oracle.c bit for bit,
 * and by bench.py's cpu_baseline leg as the "reference" kind.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef REF_BODY
#error "build with -DREF_BODY='\"/path/to/the/cut.inc\"' (see build_ref.sh)"
#endif
#include REF_BODY

#define EXPORT __attribute__((visibility("default")))

EXPORT float ref_bf16_to_f32(uint16_t v) { return bf16_to_f32(v); }
EXPORT uint16_t ref_f32_to_bf16(float f) { return f32_to_bf16(f); }
EXPORT float ref_fp16_to_f32(uint16_t h) { return fp16_to_f32(h); }
EXPORT void ref_get_scale_min_k4(int j, const uint8_t *scales, uint8_t *sc, uint8_t *m) {
    get_scale_min_k4(j, scales, sc, m);
}
EXPORT void ref_gguf_dequant_row(const void *row, float *y, int n, int ggml_type) {
    gguf_dequant_row(row, y, n, ggml_type);
}
EXPORT void ref_cpu_dequant_matvec(const uint32_t *W, const uint16_t *scales, const uint16_t *biases,
                                   const float *x, float *out, int out_dim, int in_dim,
                                   int group_size, int bits) {
    cpu_dequant_matvec(W, scales, biases, x, out, out_dim, in_dim, group_size, bits);
}
EXPORT void ref_cpu_rms_norm(const float *x, const uint16_t *w_bf16, float *out, int dim, float eps) {
    cpu_rms_norm(x, w_bf16, out, dim, eps);
}
EXPORT void ref_cpu_swiglu(const float *gate, const float *up, float *out, int dim) {
    cpu_swiglu(gate, up, out, dim);
}
EXPORT float ref_cpu_sigmoid(float x) { return cpu_sigmoid(x); }
EXPORT void ref_cpu_softmax(float *x, int dim) { cpu_softmax(x, dim); }
EXPORT void ref_cpu_topk(const float *scores, int dim, int K, int *indices, float *values) {
    cpu_topk(scores, dim, K, indices, values);
}
EXPORT void ref_cpu_normalize_weights(float *weights, int K) { cpu_normalize_weights(weights, K); }
EXPORT void ref_cpu_vec_madd(float *dst, const float *src, float scale, int dim) {
    cpu_vec_madd(dst, src, scale, dim);
}
/* the remaining helpers of the cut are referenced so that -Wall stays quiet */
EXPORT int ref_cpu_argmax(const float *x, int dim) { return cpu_argmax(x, dim); }
EXPORT void ref_cpu_vec_copy(float *dst, const float *src, int dim) { cpu_vec_copy(dst, src, dim); }
