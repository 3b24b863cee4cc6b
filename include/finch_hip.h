/*
 * finch_hip.h — C ABI of libfinchhip.so: FinchMoE's quantized-expert operator
 * path (dequant fused with the matrix products) on one MI355X (gfx950).
 *
 * The reference has no header or FFI for this path: its "operator API" is a set
 * of static C functions in finchmoe/infer.m driving Metal kernels.  Each entry
 * point below names the reference function whose operand contract it keeps
 * (paths relative to the reference tree).  Packed weights are accepted in the
 * reference's own layouts, byte for byte:
 *   - affine expert blobs  packed_experts_{N}bit/layer_XX.bin
 *                          (finchmoe/repack_experts.py:76-163, 336-392;
 *                           finchmoe/infer.m:174-234)
 *   - dense affine tensors .weight U32 / .scales / .biases
 *                          (finchmoe/quantize_non_experts.py:294, 365-386;
 *                           finchmoe/quantize_model.py:19-47)
 *   - GGUF expert slabs    Q4_K / Q6_K stacked tensors
 *                          (finchmoe/infer.m:1017-1022, 1120-1148, 1604-1657)
 *
 * Conventions
 *   - every function returns an fm_status (0 = ok, negative = error); nothing
 *     aborts; fm_last_error() gives a message for the last failure on a context
 *   - *_dev entry points take DEVICE pointers, enqueue on the context's stream
 *     and return without waiting; host-pointer entry points (no suffix) copy
 *     in, run, copy out and wait, like the reference's synchronous calls
 *   - a context is not re-entrant: one caller thread at a time, one stream
 *     (the reference's compute path is single-threaded, infer.m:13874)
 *   - weights are immutable after upload; host copies may be freed afterwards
 *   - there is no CPU fallback: without a GPU every compute call fails
 */
#ifndef FINCH_HIP_H
#define FINCH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FM_API __attribute__((visibility("default")))

typedef struct fm_ctx fm_ctx;

typedef enum {
    FM_OK = 0,
    FM_ERR_ARG = -1,          /* bad argument (null, range, shape, alignment)  */
    FM_ERR_HIP = -2,          /* a HIP runtime call failed                     */
    FM_ERR_STATE = -3,        /* store not configured / layer not resident     */
    FM_ERR_UNSUPPORTED = -4,  /* format or shape this build has no kernel for  */
    FM_ERR_NOMEM = -5
} fm_status;

/* 16-bit type of the per-group scale and bias.  The reference stores BF16
 * (finchmoe/repack_experts.py:232-234, finchmoe/infer.m:690-695). */
enum { FM_SCALE_BF16 = 0, FM_SCALE_FP16 = 1 };

/* ggml tensor types accepted for GGUF slabs (finchmoe/infer.m:1606, 1631) */
enum { FM_GGML_Q4_K = 12, FM_GGML_Q6_K = 14 };

/* flags of the routed-expert calls */
enum {
    FM_ACCUMULATE = 1,  /* out += result (gpu_gguf_experts_forward adds into
                           moe_out, infer.m:3340); default overwrites          */
    FM_GUARD = 2        /* CPU-path combine: skip an expert whose output has a
                           non-finite or >=1e20 sum of squares, renormalise
                           when 0 < sum of kept weights < 0.99
                           (infer.m:10190-10204).  Default is the GPU path's
                           plain slot-order sum (shaders.metal:2213-2228).    */
};

/* which matrix of an expert (dequant entry points) */
enum { FM_MAT_GATE = 0, FM_MAT_UP = 1, FM_MAT_DOWN = 2 };

/* ---------------------------------------------------------------- context
 * Replaces MetalCtx + metal_setup (finchmoe/infer.m:2190-2811). */
FM_API int fm_ctx_create(int device, fm_ctx **out);
FM_API int fm_ctx_destroy(fm_ctx *ctx);
FM_API int fm_sync(fm_ctx *ctx);
FM_API void *fm_stream(fm_ctx *ctx);                 /* the hipStream_t of the context */
FM_API const char *fm_last_error(fm_ctx *ctx);
FM_API const char *fm_status_string(int status);
/* event pair on the context's stream around whatever is enqueued in between */
FM_API int fm_timer_start(fm_ctx *ctx);
FM_API int fm_timer_stop(fm_ctx *ctx, float *elapsed_ms);   /* waits for the stop event */

/* Timing of the routed-expert decode calls with events on the context's stream.
 * mode 1: events around the operator as it is launched (one fused kernel where the
 *         shape allows): fm_kernel_timing_read returns its duration in gate_up_ms
 *         and ~0 in down_ms.
 * mode 2: the phases run as separate kernels (gate+up+SwiGLU, then down+combine)
 *         and each is timed.
 * mode 0: off.  While on, every fm_*moe_decode*_dev call waits for its events, so the
 * call becomes synchronous; the durations accumulate until read.  For measurement
 * runs only (the reference's --timing accumulators, finchmoe/infer.m:281-298, play
 * this role). */
FM_API int fm_kernel_timing(fm_ctx *ctx, int mode);
/* Bound of the waits inside the fused decode kernel (a workgroup waiting for a
 * vector another workgroup produces), in polls of about a microsecond; default
 * 1 << 20.  A wait that runs out does not hang: the kernel goes on, and the next
 * fm_sync / host-pointer call returns FM_ERR_HIP ("results are invalid").  No
 * counterpart in the reference (its kernels are separate Metal dispatches). */
FM_API int fm_set_wait_limit(fm_ctx *ctx, unsigned int polls);
/* Where the library has two forms of a kernel it picks one by shape.  For A/B measurements
 * (and for callers that want the forms whose results are bitwise those of the one-position
 * call) the choice can be overridden, process-wide; 0 restores the default.  No counterpart
 * in the reference. */
#define FM_FORM_PLAIN_DENSE 1u     /* dense affine GEMV: the plain kernel for every shape */
#define FM_FORM_PLAIN_GGUF 2u      /* GGUF experts and tensors: the plain kernels for every shape */
#define FM_FORM_NO_DENSE_GEMM 4u   /* fm_matvec_prefill*: one GEMV per position for every M */
#define FM_FORM_NO_GGUF_GROUP 8u   /* fm_gguf_moe_prefill*: the per-position kernels for every M */
#define FM_FORM_GGUF_PHASES 16u    /* fm_gguf_moe_decode*: gate/up, down and combine as three launches */
#define FM_FORM_GGUF_ONE_LAUNCH 32u /* fm_gguf_moe_decode*: the one launch also for more than 13 layers / 8 positions */
FM_API int fm_set_kernel_forms(unsigned int forms);
/* sums in milliseconds since the last read, and the number of calls; resets */
/* Calls captured into a HIP graph (hipStreamBeginCapture on fm_stream()).  A graph records the
 * addresses of the context's scratch buffers, which grow on demand otherwise.  So: reserve
 * first — scratch for steps of up to n_groups layers and chunks of up to M positions on the
 * configured stores, the layer tail's scratch, at least workspace_bytes of workspace (dense
 * prefill products) — then capture.  From the first call issued under capture on, a call that
 * would have to grow a buffer returns FM_ERR_STATE instead of moving it under the graph's
 * feet; fm_release_graphs() lifts that once no such graph will be replayed.  No counterpart in
 * the reference (its command buffers are re-encoded per token). */
FM_API int fm_reserve(fm_ctx *ctx, int n_groups, int M, size_t workspace_bytes);
FM_API int fm_release_graphs(fm_ctx *ctx);

FM_API int fm_kernel_timing_read(fm_ctx *ctx, double *gate_up_ms, double *down_ms, int *calls);

/* Streaming probe: reads nbytes (whole 4 KB slots) of the device buffer d_buf once, with the
 * access structure of the expert kernels (one workgroup of twelve waves per CU, LDS-direct
 * 16-byte loads into a ring of two slots per wave) and no arithmetic; asynchronous on the context's stream.
 * pattern: 0 = slots dealt out over all waves of the chip (one dense window at any moment),
 * 1 = a contiguous share per workgroup, its waves interleaved (the decode kernels' order),
 * 2 = a contiguous share per wave (3..7: groups of workgroups in turn).  The loads carry the
 * non-temporal hint the decode kernels use for weights that a launch reads once; pattern + 8 is
 * the same walk with ordinary caching.  Timed with fm_timer_start/stop it gives the rate the
 * memory system delivers to a kernel of that structure.  No counterpart in the reference. */
FM_API int fm_stream_probe_dev(fm_ctx *ctx, const void *d_buf, size_t nbytes, int pattern);

/* ---------------------------------------------------------------- expert store, affine
 * Replaces the packed-expert files + pread/LRU machinery
 * (finchmoe/infer.m:5816-6575, 15421-15425) by HBM residency.
 * bits: 3 or 4.  hidden, inter multiples of 128.  group_size 64. */
FM_API int fm_experts_config(fm_ctx *ctx, int n_layers, int n_experts, int hidden, int inter,
                      int group_size, int bits, int scale_dtype);
FM_API size_t fm_experts_expert_size(fm_ctx *ctx);   /* bytes of one expert, 0 if unconfigured */
/* verbatim bytes of layer_XX.bin: n_experts * expert_size */
FM_API int fm_experts_upload_layer(fm_ctx *ctx, int layer, const void *host_blob, size_t nbytes);
/* same layout already in device memory owned by the caller (16-byte aligned);
 * must stay valid until the context is destroyed or the layer is replaced */
FM_API int fm_experts_adopt_layer(fm_ctx *ctx, int layer, const void *dev_blob, size_t nbytes);

/* ---------------------------------------------------------------- routed experts, decode
 * Replaces gpu_encode_experts_batched + moe_combine_residual's weighted sum
 * (finchmoe/infer.m:4065-4383, finchmoe/shaders.metal:2196-2231) and the CPU
 * twin (infer.m:10109-10204).
 *   x[hidden] fp32, idx[K] int32 (distinct experts, any order), w[K] fp32
 *   out[hidden] = sum_k w[k] * down_k(SiLU(gate_k x) * up_k x), k in slot order
 *   expert_out (may be NULL) receives the K per-expert vectors [K][hidden]
 *   K in 1..8.  w[k] == 0 keeps the slot but adds nothing (valid[k]=0,
 *   infer.m:9672).  An index outside 0..n_experts-1 is treated as w[k] = 0. */
FM_API int fm_moe_decode_dev(fm_ctx *ctx, int layer, const float *d_x, const int32_t *d_idx,
                      const float *d_w, int K, float *d_out, float *d_expert_out, int flags);
FM_API int fm_moe_decode(fm_ctx *ctx, int layer, const float *x, const int32_t *idx,
                  const float *w, int K, float *out, float *expert_out, int flags);
/* n_layers consecutive layers in one submission, each with its own x, idx, w:
 * x[n_layers][hidden], idx[n_layers][K], w[n_layers][K], out[n_layers][hidden],
 * expert_out[n_layers][K][hidden] or NULL.  (The per-token loop over layers,
 * infer.m:15771, with the expert blocks of all layers batched.) */
FM_API int fm_moe_decode_step_dev(fm_ctx *ctx, int layer0, int n_layers, const float *d_x,
                           const int32_t *d_idx, const float *d_w, int K, float *d_out,
                           float *d_expert_out, int flags);

/* fm_moe_decode_step_dev without a per-expert output, for callers that cannot allocate (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  It calls no hipMalloc / hipFree / allocating routine: the
 * intermediate vectors and dependency counters live in a fixed 4 MiB array that is part of the
 * library's device image (one copy per GPU, held until the process ends).  Limit:
 *   n_layers * 8 * (hidden + inter) * 4 + n_layers * 9 * 4 bytes <= 4 MiB
 * (40 layers at hidden 2048 / inter 512 need 3.13 MiB); larger calls return FM_ERR_ARG.
 * Results are bit for bit those of fm_moe_decode_step_dev.  All contexts on one GPU share
 * that GPU's array: calls that overlap on one GPU (two contexts, two streams) race. */
FM_API int fm_moe_decode_step_noalloc_dev(fm_ctx *ctx, int layer0, int n_layers, const float *d_x,
                                   const int32_t *d_idx, const float *d_w, int K, float *d_out,
                                   int flags);

/* ---------------------------------------------------------------- routed experts, chunked prefill
 * Replaces prefill_chunk_cmd3_encode / prefill_chunk_cmd3_batch_general
 * (finchmoe/infer.m:10704-11059): M positions, each with its own top-K.
 *   X[M][hidden] fp32, idx[M][K], w[M][K], out[M][hidden] fp32; X and out 16-byte
 *   aligned (fp32 vectors are read and written four at a time throughout the library).
 * Result contract: the same as fm_moe_decode per position.  1 <= M <= 65535. */
FM_API int fm_moe_prefill_dev(fm_ctx *ctx, int layer, const float *d_X, const int32_t *d_idx,
                       const float *d_w, int M, int K, float *d_out, int flags);
FM_API int fm_moe_prefill(fm_ctx *ctx, int layer, const float *X, const int32_t *idx,
                   const float *w, int M, int K, float *out, int flags);
/* the same chunk with the activations as bfloat16 bits, X[M][hidden] uint16 (a prefill chunk
 * of bf16 hidden states; the widening to fp32 the reference's callers do before
 * prefill_chunk_cmd3_encode, finchmoe/infer.m:10704, is skipped).  Result contract: what
 * fm_moe_prefill gives on the widened X.  From 32 positions on this is the fast form of the
 * grouped product: a bf16 value is one matrix-core operand, an fp32 value two. */
FM_API int fm_moe_prefill_bf16_dev(fm_ctx *ctx, int layer, const uint16_t *d_X, const int32_t *d_idx,
                            const float *d_w, int M, int K, float *d_out, int flags);
FM_API int fm_moe_prefill_bf16(fm_ctx *ctx, int layer, const uint16_t *X, const int32_t *idx,
                        const float *w, int M, int K, float *out, int flags);

/* ---------------------------------------------------------------- dense affine tensors
 * Replaces fast_dequant_matvec / BatchMatvecSpec + fast_batch_matvec /
 * gpu_encode_prefill_matvec (finchmoe/infer.m:3369, 3401-3411, 4477, 3672;
 * kernels dequant_matvec_4bit_v3 and _prefill, shaders.metal:374-463, 2460-2529).
 * W: u32 [out_dim][in_dim*bits/32] (bits 1, 2, 4 or 8; LSB first) or bytes
 * [out_dim][in_dim*3/8] (bits 3); S, B: 16-bit [out_dim][in_dim/group_size].  in_dim:
 * 128 * 2^j up to 8192 for bits 3, 4, 8; any multiple of 64 up to 16384 for the legacy widths
 * 1 and 2 (cpu_dequant_matvec's generic branch, finchmoe/infer.m:1734-1760), which run a plain
 * kernel of their own and are not accepted by fm_layer_tail_dev.
 * S == NULL or B == NULL: an unquantized BF16 tensor [out_dim][in_dim] (cpu_dequant_matvec's
 * raw branch, finchmoe/infer.m:1689-1701).
 * bits 10 / 11 (the reference's own codes, finchmoe/infer.m:1684-1688, 3378-3388): a GGUF Q4_K /
 * Q6_K tensor, rows of in_dim/256 blocks of 144 / 210 bytes, S and B ignored — the vocabulary
 * projection and embedding of a GGUF model (lm_head_forward and embed_lookup,
 * finchmoe/infer.m:5738-5746, 5675-5683).  in_dim a multiple of 256. */
typedef int fm_tensor;   /* handle >= 0 */
FM_API int fm_tensor_register(fm_ctx *ctx, const void *W, const void *S, const void *B,
                       int out_dim, int in_dim, int group_size, int bits,
                       int scale_dtype, fm_tensor *out);
/* device-resident W, S, B owned by the caller (16-byte aligned) */
FM_API int fm_tensor_adopt(fm_ctx *ctx, const void *d_W, const void *d_S, const void *d_B,
                    int out_dim, int in_dim, int group_size, int bits,
                    int scale_dtype, fm_tensor *out);
FM_API int fm_tensor_release(fm_ctx *ctx, fm_tensor t);
/* n matvecs sharing one input vector (all tensors must have the same in_dim) */
FM_API int fm_matvec_batch_dev(fm_ctx *ctx, const fm_tensor *tensors, int n, const float *d_x,
                        float *const *d_outs);
FM_API int fm_matvec_batch(fm_ctx *ctx, const fm_tensor *tensors, int n, const float *x,
                    float *const *outs);
/* M positions: X[M][in_dim] -> out[M][out_dim] (gpu_encode_prefill_matvec,
 * finchmoe/infer.m:3672).  Fewer than 16 positions (and shapes the matrix-core kernel does
 * not cover) run one GEMV per position, bitwise equal to the one-position call; from 16
 * positions on a 3-/4-bit tensor with in_dim a multiple of 2048 and out_dim a multiple of 64,
 * or in_dim 512 and out_dim a multiple of 256, is multiplied on the matrix cores (equal to the
 * one-position call within the parity bar; d_X must be 16-byte aligned for it) as long as
 * ceil(M / 16) * (out_dim / 64) -- out_dim / 256 at in_dim 512 -- does not exceed the number of
 * compute units; larger products run one GEMV per position. */
FM_API int fm_matvec_prefill_dev(fm_ctx *ctx, fm_tensor t, const float *d_X, float *d_out, int M);
/* n tensors against the same X[M][in_dim] (each tensor as fm_matvec_prefill_dev; tensors the
 * matrix-core kernel covers share one preparation of X) */
FM_API int fm_matvec_prefill_batch_dev(fm_ctx *ctx, const fm_tensor *tensors, int n, const float *d_X,
                                float *const *d_outs, int M);
FM_API int fm_matvec_prefill(fm_ctx *ctx, fm_tensor t, const float *X, float *out, int M);

/* ---------------------------------------------------------------- routing
 * Replaces cpu_softmax + cpu_topk + cpu_normalize_weights between the routing GEMVs and
 * the expert launch (finchmoe/infer.m:1794-1840, 9285-9289), on the device: softmax over
 * logits[n_experts] (the 8-bit mlp.gate GEMV's output, fm_matvec_batch_dev), the K largest
 * in the reference's slot order (a score replaces the smallest kept one when strictly
 * larger; among equal minima the lowest slot), weights renormalised to sum 1.
 * idx[K], w[K] feed fm_moe_decode_dev as they are.  params (optional, [10]) is filled as
 * the reference's buf_combine_params: w[0..K-1], zeros, *seg_score (the shared expert's
 * gate score, optional) at [8] — the operand of fm_layer_tail_dev. */
FM_API int fm_route_topk_dev(fm_ctx *ctx, const float *d_logits, int n_experts, int K,
                      const float *d_seg_score, int32_t *d_idx, float *d_w, float *d_params);

/* fm_matvec_batch_dev followed by fm_route_topk_dev over tensor 0's outputs (the gate logits),
 * as ONE launch when the batch is small enough for the plain GEMV kernel — the workgroup that
 * finishes last routes — and as the two launches otherwise; same results either way.  The
 * per-layer loop's first step: 8-bit mlp.gate + shared_expert_gate and the 4-bit shared
 * gate/up projections on one x, then softmax/top-K (finchmoe/infer.m:9285-9300, 1794-1840).
 * d_seg_score is normally d_outs[1]. */
FM_API int fm_matvec_batch_route_dev(fm_ctx *ctx, const fm_tensor *tensors, int n, const float *d_x,
                              float *const *d_outs, int K, const float *d_seg_score,
                              int32_t *d_idx, float *d_w, float *d_params);

/* ---------------------------------------------------------------- layer tail
 * Replaces the five dispatches the reference appends to a layer's expert command
 * buffer (finchmoe/infer.m:9608-9760): swiglu_fused on the shared expert's gate/up
 * outputs, its down projection (dequant_matvec), moe_combine_residual
 * (shaders.metal:2196-2231), rms_norm_sum_sq + rms_norm_apply_bf16
 * (shaders.metal:1134-1205).
 *   shared_down : registered tensor [hidden][shared_inter], 3/4/8-bit g64
 *   h_mid[hidden], expert_out[K][hidden] (as fm_moe_decode leaves them),
 *   params[10] = expert weights 0..7 (0 for an invalid slot), shared gate score
 *   at [8] (buf_combine_params), shared_gate / shared_up [shared_inter],
 *   next_norm_w[hidden] bf16 + next_input[hidden], both NULL for the last layer.
 *   K == 0 with expert_out != NULL: expert_out is ONE vector [hidden], the routed experts'
 *   weighted sum as fm_moe_decode_dev leaves it in `out` when it is called without a buffer
 *   for the per-expert vectors (same slot order, same arithmetic: the results are identical,
 *   and the expert launch is the faster one that never writes the K vectors).
 * hidden_out = h_mid + sum_k params[k]*expert_out[k] + sigmoid(params[8])*shared_out;
 * next_input = hidden_out / sqrt(mean(hidden_out^2) + eps) * next_norm_w.
 * All pointers device memory; asynchronous on the context's stream. */
FM_API int fm_layer_tail_dev(fm_ctx *ctx, fm_tensor shared_down, const float *d_h_mid,
                      const float *d_expert_out, const float *d_params, int K,
                      const float *d_shared_gate, const float *d_shared_up,
                      const uint16_t *d_next_norm_w, float eps, float *d_hidden_out,
                      float *d_next_input);

/* The routed experts of one layer and the layer tail in ONE launch — the reference's CMD3 command
 * buffer from the expert dispatches to the next layer's norm (finchmoe/infer.m:9608-9760):
 * fm_moe_decode_dev(ctx, layer, d_x, d_idx, d_w, K, sum, NULL, 0) followed by
 * fm_layer_tail_dev(ctx, shared_down, d_h_mid, sum, d_params, 0, ...), with identical results
 * bit for bit.  d_params: only [8] (the shared-expert gate score) is read; the experts' weights are
 * d_w.  One launch when shared_down is 4-bit with the experts' down shape (the workgroup that
 * owns rows of the experts' sum runs the same rows of the shared projection, and the workgroup
 * that finishes last normalises); other shapes, split-phase mode and calls under stream capture
 * run as the two launches. */
FM_API int fm_moe_decode_tail_dev(fm_ctx *ctx, int layer, const float *d_x, const int32_t *d_idx,
                           const float *d_w, int K, fm_tensor shared_down, const float *d_h_mid,
                           const float *d_params, const float *d_shared_gate,
                           const float *d_shared_up, const uint16_t *d_next_norm_w, float eps,
                           float *d_hidden_out, float *d_next_input);

/* The MoE half of a layer (finchmoe/infer.m:9285-9760: routing_batch_fused, the CPU routing,
 * CMD3) in two launches and without a host round trip:
 *   route_tensors[4] = router gate [n_experts][hidden] (8-bit upstream), shared-expert gate
 *   [1][hidden], shared expert's gate and up projections [inter][hidden] — all multiplied with
 *   d_x in the first launch (fm_matvec_batch_dev), results in d_logits, d_seg_score,
 *   d_shared_gate, d_shared_up;
 *   second launch: softmax + top-K + normalisation of the logits (every workgroup runs the
 *   routing wave on them; d_idx, d_w, d_params[10] receive the result), the routed experts of
 *   `layer` on d_x, and the layer tail as fm_moe_decode_tail_dev.
 * Identical to fm_matvec_batch_route_dev + fm_moe_decode_dev + fm_layer_tail_dev (K = 0 form);
 * shapes the one-launch kernel does not cover run as those launches. */
FM_API int fm_moe_layer_dev(fm_ctx *ctx, int layer, const fm_tensor *route_tensors, const float *d_x, int K,
                     fm_tensor shared_down, const float *d_h_mid, const uint16_t *d_next_norm_w,
                     float eps, float *d_logits, float *d_seg_score, float *d_shared_gate,
                     float *d_shared_up, int32_t *d_idx, float *d_w, float *d_params,
                     float *d_hidden_out, float *d_next_input);

/* ---------------------------------------------------------------- GGUF expert store
 * Replaces GgufExpertInfo + the slab copies of gpu_gguf_experts_forward
 * (finchmoe/infer.m:1017-1022, 3239-3290).  gate/up/down are the stacked
 * per-layer tensors, expert e at e*slab; gate and up must be Q4_K, down Q4_K or
 * Q6_K (infer.m:3166). */
FM_API int fm_gguf_config(fm_ctx *ctx, int n_layers, int n_experts, int hidden, int inter,
                   int gate_type, int up_type, int down_type);
/* the byte counts must equal n_experts * slab of the configured geometry (a file whose
 * dimensions or types differ from the configuration is refused instead of over-read);
 * on any failure the layer keeps what it held before */
FM_API int fm_gguf_upload_layer(fm_ctx *ctx, int layer, const void *gate, size_t gate_bytes,
                         const void *up, size_t up_bytes, const void *down, size_t down_bytes);
FM_API int fm_gguf_adopt_layer(fm_ctx *ctx, int layer, const void *d_gate, size_t gate_bytes,
                        const void *d_up, size_t up_bytes, const void *d_down, size_t down_bytes);
/* gpu_gguf_experts_forward (finchmoe/infer.m:3153-3366) */
FM_API int fm_gguf_moe_decode_dev(fm_ctx *ctx, int layer, const float *d_x, const int32_t *d_idx,
                           const float *d_w, int K, float *d_out, float *d_expert_out,
                           int flags);
FM_API int fm_gguf_moe_decode(fm_ctx *ctx, int layer, const float *x, const int32_t *idx,
                       const float *w, int K, float *out, float *expert_out, int flags);
FM_API int fm_gguf_moe_decode_step_dev(fm_ctx *ctx, int layer0, int n_layers, const float *d_x,
                                const int32_t *d_idx, const float *d_w, int K,
                                float *d_out, float *d_expert_out, int flags);
/* prefill_chunk_cmd3_batch_general in GGUF mode (finchmoe/infer.m:10958-11059) */
FM_API int fm_gguf_moe_prefill_dev(fm_ctx *ctx, int layer, const float *d_X, const int32_t *d_idx,
                            const float *d_w, int M, int K, float *d_out, int flags);
FM_API int fm_gguf_moe_prefill(fm_ctx *ctx, int layer, const float *X, const int32_t *idx,
                        const float *w, int M, int K, float *out, int flags);
/* single Q4_K / Q6_K matvec (gpu_gguf_dequant_matvec, finchmoe/infer.m:3050;
 * kernel dequant_matvec_qk, shaders.metal:3216-3299); host pointers */
FM_API int fm_gguf_matvec(fm_ctx *ctx, const void *W, int ggml_type, const float *x, float *out,
                   int out_dim, int in_dim);

/* ---------------------------------------------------------------- embedding lookup
 * embed_lookup(wf, token_id, out) (finchmoe/infer.m:5664-5722): row token_id of a registered
 * tensor [vocab][hidden], dequantized to fp32.  Affine tensors (the 4-/8-bit branch):
 * out[j] = (float)code * scale + bias; GGUF tensors registered with bits 10 / 11 (the
 * block-format branch, finchmoe/infer.m:5675-5683): gguf_dequant_row of the token's row.  Either
 * way the same value fm_dequant_tensor gives for that row.
 * The _dev form takes n ids from device memory (one row each, out [n][in_dim], asynchronous
 * on the context's stream); an id outside the tensor gives a row of zeros. */
FM_API int fm_embed_lookup_dev(fm_ctx *ctx, fm_tensor t, const int32_t *d_token_ids, int n_tokens,
                        float *d_out);
FM_API int fm_embed_lookup(fm_ctx *ctx, fm_tensor t, int token_id, float *out);

/* ---------------------------------------------------------------- dequant (bit-exact checks)
 * The reference has no such call; these expose what its kernels compute on the
 * fly — code = field of the packed word, w = (float)code * scale + bias in fp32
 * (finchmoe/infer.m:1725, 1757; shaders.metal:598-605) — so tests can compare
 * codes and weights bit for bit.  Host output buffers, any may be NULL:
 * codes u8 [rows][cols], w_f32 [rows][cols], w_f16 = RNE(w_f32) as IEEE half. */
FM_API int fm_dequant_expert(fm_ctx *ctx, int layer, int expert, int which, uint8_t *codes,
                      float *w_f32, uint16_t *w_f16);
FM_API int fm_dequant_tensor(fm_ctx *ctx, fm_tensor t, uint8_t *codes, float *w_f32,
                      uint16_t *w_f16);
/* GGUF: w_f32 = the block formula (finchmoe/infer.m:1604-1657) */
FM_API int fm_gguf_dequant_expert(fm_ctx *ctx, int layer, int expert, int which, float *w_f32);

#ifdef __cplusplus
}
#endif
#endif /* FINCH_HIP_H */
