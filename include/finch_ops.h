/*
 * finch_ops.h — C host layer with the reference's own operator names, on top of
 * the C ABI of libfinchhip.so.  A caller written against the static functions of
 * finchmoe/infer.m (the engine's C core) links this instead and keeps its call
 * sites: same names, same argument meaning, same synchronous behaviour, same
 * packed layouts; the weights it points at are uploaded to HBM on first use and
 * stay resident.
 *
 * Differences from the reference, all deliberate:
 *   - nothing aborts: a failed matvec call fills its output with zeros (the call sites
 *     take a void result and go on to read it), a failed expert call returns 0 and
 *     leaves moe_out as it was, and both record a status readable with
 *     finch_ops_last_status() / finch_ops_last_error()
 *     (the reference abort()s on a BF16 tensor reaching a 4-bit kernel,
 *     infer.m:2879-2885, and falls back to the CPU elsewhere; there is no CPU
 *     fallback here)
 *   - expert weights are made resident per layer with finch_ops_load_* instead
 *     of being pread per token (infer.m:9556)
 */
#ifndef FINCH_OPS_H
#define FINCH_OPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* finchmoe/infer.m:3401-3411 */
typedef struct {
    const void *W;        /* packed weights */
    const void *scales;   /* 16-bit scales  */
    const void *biases;   /* 16-bit biases  */
    float *out_cpu;       /* result is written here */
    uint32_t out_dim;
    uint32_t in_dim;
    uint32_t group_size;
    int batch_slot;       /* kept for source compatibility; unused */
    int bits;             /* 3, 4 or 8 */
} BatchMatvecSpec;

/* replaces metal_setup (finchmoe/infer.m:2388-2811): one context on `device` */
int finch_ops_init(int device);
void finch_ops_shutdown(void);
int finch_ops_last_status(void);
const char *finch_ops_last_error(void);
/* scale/bias type of tensors registered from now on: 0 = BF16 (reference), 1 = FP16 */
void finch_ops_set_scale_dtype(int scale_dtype);

/* finchmoe/infer.m:3369 — bits 3/4/8 affine; bits 10/11 with scales == NULL = Q4_K/Q6_K */
void fast_dequant_matvec(const uint32_t *W, const uint16_t *scales, const uint16_t *biases,
                         const float *x, float *out, int out_dim, int in_dim, int group_size,
                         int bits);
/* finchmoe/infer.m:4477 — N matvecs sharing one input */
void fast_batch_matvec(const float *x, uint32_t x_dim, BatchMatvecSpec *specs, int num_specs);
/* M positions, x [M][in_dim] -> out [M][out_dim] (gpu_encode_prefill_matvec, infer.m:3672) */
void fast_prefill_matvec(const uint32_t *W, const uint16_t *scales, const uint16_t *biases,
                         const float *x, float *out, int out_dim, int in_dim, int group_size,
                         int bits, int M);
/* upload a tensor now rather than on its first use (a loader's warm-up) */
int finch_ops_make_resident(const void *W, const uint16_t *scales, const uint16_t *biases,
                            int out_dim, int in_dim, int group_size, int bits);
/* forget the HBM copy of a tensor whose host memory is about to be reused */
void finch_ops_forget_tensor(const void *W);

/* expert residency: verbatim layer_XX.bin bytes (finchmoe/repack_experts.py:336-392) */
int finch_ops_config_experts(int n_layers, int n_experts, int hidden, int inter, int bits);
int finch_ops_load_expert_layer(int layer, const void *blob, size_t nbytes);
/* GGUF stacked expert tensors of one layer (finchmoe/infer.m:1017-1022) */
int finch_ops_config_gguf_experts(int n_layers, int n_experts, int hidden, int inter,
                                  int gate_type, int up_type, int down_type);
int finch_ops_load_gguf_layer(int layer, const void *gate, size_t gate_bytes, const void *up,
                              size_t up_bytes, const void *down, size_t down_bytes);

/* routed experts of one layer: moe_out += sum_k w_k * expert_k(h_post), slot order, with
 * the CPU path's finite guard + renormalisation (finchmoe/infer.m:10109-10204).
 * Returns 1 on success, 0 on failure (the reference's "fall back" return). */
int moe_experts_forward(int layer_idx, const float *h_post, const int *expert_indices,
                        const float *expert_weights, int K, float *moe_out);
/* finchmoe/infer.m:3153 (ctx and wf arguments dropped: the layer's slabs are resident) */
int gpu_gguf_experts_forward(int layer_idx, const float *h_post, const int *expert_indices,
                             const float *expert_weights, int K, float *moe_out);
/* chunk of M positions (prefill_chunk_cmd3_encode per position, infer.m:10704):
 * h_post [M][hidden], indices/weights [M][K], moe_out [M][hidden] accumulated into */
int moe_experts_forward_chunk(int layer_idx, const float *h_post, const int *expert_indices,
                              const float *expert_weights, int M, int K, float *moe_out);

/* the same chunk with the positions as BF16 bits (an engine that keeps its residual stream in
 * bf16; the reference's prefill buffers are fp32, infer.m:10704-10765) */
int moe_experts_forward_chunk_bf16(int layer_idx, const uint16_t *h_post_bf16, const int *expert_indices,
                                   const float *expert_weights, int M, int K, float *moe_out);
/* chunk of M positions on the GGUF store (prefill_chunk_cmd3_batch_general, infer.m:10958-11059:
 * the *_pool_prefill kernels once per position; here grouped by expert from 32 positions on) */
int gpu_gguf_experts_forward_chunk(int layer_idx, const float *h_post, const int *expert_indices,
                                   const float *expert_weights, int M, int K, float *moe_out);

/* routing runs on the CPU in the reference (finchmoe/infer.m:1794-1840, 9285-9289) */
void cpu_softmax(float *x, int dim);
void cpu_topk(const float *scores, int dim, int K, int *indices, float *values);
void cpu_normalize_weights(float *weights, int K);

#ifdef __cplusplus
}
#endif
#endif
