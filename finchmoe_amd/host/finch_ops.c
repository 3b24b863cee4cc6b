/* finch_ops.c — see finch_ops.h.  Plain C99 over the C ABI of libfinchhip.so. */
#include "finch_ops.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "finch_hip.h"

static fm_ctx *g_ctx = NULL;
static int g_status = FM_OK;
static char g_err[512] = "";
static int g_scale_dtype = FM_SCALE_BF16;
static int g_hidden = 0, g_gguf_hidden = 0;

static int fail(int status, const char *what) {
    g_status = status;
    snprintf(g_err, sizeof g_err, "%s: %s (%s)", what, fm_status_string(status),
             g_ctx ? fm_last_error(g_ctx) : "no context");
    fprintf(stderr, "finch_ops: %s\n", g_err);
    return status;
}

/* ---- host pointer -> resident tensor (the reference wraps mmap'd tensors into
 * Metal buffers lazily the same way, finchmoe/infer.m:2813-2870) ---- */
typedef struct {
    const void *key;
    fm_tensor t;
    int out_dim, in_dim, bits;
} slot;
static slot *g_tab = NULL;
static size_t g_cap = 0, g_used = 0;

static size_t hash_ptr(const void *p) {
    uintptr_t v = (uintptr_t)p;
    v ^= v >> 33;
    v *= 0xff51afd7ed558ccdULL;
    v ^= v >> 29;
    return (size_t)v;
}

/* NULL: no such key (insert == 0), or no memory for the table */
static slot *tab_find(const void *key, int insert) {
    if (!key) return NULL;               /* NULL marks an empty slot */
    if (!g_cap) {
        g_tab = (slot *)calloc(1024, sizeof(slot));
        if (!g_tab) return NULL;
        g_cap = 1024;
    }
    if (insert && (g_used + 1) * 2 > g_cap) {
        slot *bigger = (slot *)calloc(2 * g_cap, sizeof(slot));
        if (!bigger) return NULL;
        slot *old = g_tab;
        const size_t oc = g_cap;
        g_tab = bigger;
        g_cap = 2 * oc;
        g_used = 0;
        for (size_t i = 0; i < oc; i++)
            if (old[i].key) {
                slot *s = tab_find(old[i].key, 1);     /* cannot fail: the table is half empty */
                *s = old[i];
            }
        free(old);
    }
    size_t i = hash_ptr(key) & (g_cap - 1);
    while (g_tab[i].key && g_tab[i].key != key) i = (i + 1) & (g_cap - 1);
    if (!g_tab[i].key) {
        if (!insert) return NULL;
        g_tab[i].key = key;
        g_tab[i].t = -1;
        g_used++;
    }
    return &g_tab[i];
}

static int resident(const void *W, const void *S, const void *B, int out_dim, int in_dim,
                    int group_size, int bits, fm_tensor *t) {
    /* bits 10 / 11: a GGUF Q4_K / Q6_K tensor, which carries no scales (infer.m:1684-1688,
     * 3378-3388); scales == NULL otherwise: an unquantized BF16 tensor (infer.m:1689); bits 0
     * means 4 (infer.m:4491).  Normalised here so that the table compares like with like. */
    if (bits == 10 || bits == 11) S = B = NULL;
    else if (!S || !B) { S = B = NULL; bits = 16; }
    else if (bits == 0) bits = 4;
    if (!W) return FM_ERR_ARG;
    slot *s = tab_find(W, 1);
    if (!s) return FM_ERR_NOMEM;
    if (s->t >= 0 && (s->out_dim != out_dim || s->in_dim != in_dim || s->bits != bits)) {
        fm_tensor_release(g_ctx, s->t);   /* host memory was reused for another tensor */
        s->t = -1;
    }
    if (s->t < 0) {
        int rc = fm_tensor_register(g_ctx, W, S, B, out_dim, in_dim, group_size, bits,
                                    g_scale_dtype, &s->t);
        if (rc) {
            s->t = -1;
            return rc;
        }
        s->out_dim = out_dim;
        s->in_dim = in_dim;
        s->bits = bits;
    }
    *t = s->t;
    return FM_OK;
}

int finch_ops_init(int device) {
    if (g_ctx) return FM_OK;
    int rc = fm_ctx_create(device, &g_ctx);
    if (rc) {
        g_ctx = NULL;
        return fail(rc, "finch_ops_init");
    }
    g_status = FM_OK;
    return FM_OK;
}

void finch_ops_shutdown(void) {
    if (g_ctx) fm_ctx_destroy(g_ctx);
    g_ctx = NULL;
    free(g_tab);
    g_tab = NULL;
    g_cap = g_used = 0;
}

int finch_ops_last_status(void) { return g_status; }
const char *finch_ops_last_error(void) { return g_err; }
void finch_ops_set_scale_dtype(int d) { g_scale_dtype = d; }

int finch_ops_make_resident(const void *W, const uint16_t *scales, const uint16_t *biases,
                            int out_dim, int in_dim, int group_size, int bits) {
    if (!g_ctx) return fail(FM_ERR_STATE, "finch_ops_make_resident");
    fm_tensor t;
    int rc = resident(W, scales, biases, out_dim, in_dim, group_size, bits, &t);
    return rc ? fail(rc, "finch_ops_make_resident") : FM_OK;
}

void finch_ops_forget_tensor(const void *W) {
    slot *s = g_tab ? tab_find(W, 0) : NULL;
    if (s && s->t >= 0) {
        fm_tensor_release(g_ctx, s->t);
        s->t = -1;
    }
}

void fast_dequant_matvec(const uint32_t *W, const uint16_t *scales, const uint16_t *biases,
                         const float *x, float *out, int out_dim, int in_dim, int group_size,
                         int bits) {
    if (!g_ctx) { fail(FM_ERR_STATE, "fast_dequant_matvec"); return; }
    /* quantized; bits 10 / 11: GGUF block rows (infer.m:3378-3388); scales == NULL otherwise: raw
     * BF16 [out_dim][in_dim] (infer.m:1689-1701).  The tensor stays resident after its first use. */
    fm_tensor t;
    int rc = resident(W, scales, biases, out_dim, in_dim, group_size, bits, &t);
    if (!rc) {
        float *outs[1] = {out};
        rc = fm_matvec_batch(g_ctx, &t, 1, x, outs);
    }
    if (rc) {
        /* the reference's call sites take a void result: never leave `out` uninitialised */
        memset(out, 0, (size_t)out_dim * sizeof(float));
        fail(rc, "fast_dequant_matvec");
    } else {
        g_status = FM_OK;
    }
}

static void zero_batch_outputs(BatchMatvecSpec *specs, int num_specs) {
    for (int i = 0; i < num_specs; i++)
        if (specs[i].out_cpu) memset(specs[i].out_cpu, 0, (size_t)specs[i].out_dim * sizeof(float));
}

void fast_batch_matvec(const float *x, uint32_t x_dim, BatchMatvecSpec *specs, int num_specs) {
    if (!g_ctx) { fail(FM_ERR_STATE, "fast_batch_matvec"); return; }
    if (num_specs < 1 || num_specs > 64) { fail(FM_ERR_ARG, "fast_batch_matvec"); return; }
    fm_tensor ts[64];
    float *outs[64];
    int rc = FM_OK;
    const char *what = "fast_batch_matvec";
    for (int i = 0; i < num_specs && !rc; i++) {
        if (specs[i].in_dim != x_dim) {
            rc = FM_ERR_ARG;
            what = "fast_batch_matvec (in_dim != x_dim)";
        } else {
            rc = resident(specs[i].W, specs[i].scales, specs[i].biases, (int)specs[i].out_dim,
                          (int)specs[i].in_dim, (int)specs[i].group_size, specs[i].bits, &ts[i]);
        }
        outs[i] = specs[i].out_cpu;
    }
    if (!rc) rc = fm_matvec_batch(g_ctx, ts, num_specs, x, outs);
    if (rc) {
        zero_batch_outputs(specs, num_specs);   /* void result: never leave outputs uninitialised */
        fail(rc, what);
    } else {
        g_status = FM_OK;
    }
}

void fast_prefill_matvec(const uint32_t *W, const uint16_t *scales, const uint16_t *biases,
                         const float *x, float *out, int out_dim, int in_dim, int group_size,
                         int bits, int M) {
    if (!g_ctx) { fail(FM_ERR_STATE, "fast_prefill_matvec"); return; }
    fm_tensor t;
    int rc = resident(W, scales, biases, out_dim, in_dim, group_size, bits, &t);
    if (!rc) rc = fm_matvec_prefill(g_ctx, t, x, out, M);
    if (rc) {
        if (out && out_dim > 0 && M > 0) memset(out, 0, (size_t)M * (size_t)out_dim * sizeof(float));
        fail(rc, "fast_prefill_matvec");
    } else {
        g_status = FM_OK;
    }
}

int finch_ops_config_experts(int n_layers, int n_experts, int hidden, int inter, int bits) {
    if (!g_ctx) return fail(FM_ERR_STATE, "finch_ops_config_experts");
    int rc = fm_experts_config(g_ctx, n_layers, n_experts, hidden, inter, 64, bits, g_scale_dtype);
    if (rc) return fail(rc, "finch_ops_config_experts");
    g_hidden = hidden;
    return FM_OK;
}

int finch_ops_load_expert_layer(int layer, const void *blob, size_t nbytes) {
    if (!g_ctx) return fail(FM_ERR_STATE, "finch_ops_load_expert_layer");
    int rc = fm_experts_upload_layer(g_ctx, layer, blob, nbytes);
    return rc ? fail(rc, "finch_ops_load_expert_layer") : FM_OK;
}

int finch_ops_config_gguf_experts(int n_layers, int n_experts, int hidden, int inter,
                                  int gate_type, int up_type, int down_type) {
    if (!g_ctx) return fail(FM_ERR_STATE, "finch_ops_config_gguf_experts");
    int rc = fm_gguf_config(g_ctx, n_layers, n_experts, hidden, inter, gate_type, up_type, down_type);
    if (rc) return fail(rc, "finch_ops_config_gguf_experts");
    g_gguf_hidden = hidden;
    return FM_OK;
}

int finch_ops_load_gguf_layer(int layer, const void *gate, size_t gate_bytes, const void *up,
                              size_t up_bytes, const void *down, size_t down_bytes) {
    if (!g_ctx) return fail(FM_ERR_STATE, "finch_ops_load_gguf_layer");
    int rc = fm_gguf_upload_layer(g_ctx, layer, gate, gate_bytes, up, up_bytes, down, down_bytes);
    return rc ? fail(rc, "finch_ops_load_gguf_layer") : FM_OK;
}

int moe_experts_forward(int layer_idx, const float *h_post, const int *expert_indices,
                        const float *expert_weights, int K, float *moe_out) {
    if (!g_ctx) { fail(FM_ERR_STATE, "moe_experts_forward"); return 0; }
    int rc = fm_moe_decode(g_ctx, layer_idx, h_post, expert_indices, expert_weights, K, moe_out,
                           NULL, FM_ACCUMULATE | FM_GUARD);
    if (rc) { fail(rc, "moe_experts_forward"); return 0; }
    g_status = FM_OK;
    return 1;
}

int gpu_gguf_experts_forward(int layer_idx, const float *h_post, const int *expert_indices,
                             const float *expert_weights, int K, float *moe_out) {
    if (!g_ctx) { fail(FM_ERR_STATE, "gpu_gguf_experts_forward"); return 0; }
    int rc = fm_gguf_moe_decode(g_ctx, layer_idx, h_post, expert_indices, expert_weights, K,
                                moe_out, NULL, FM_ACCUMULATE | FM_GUARD);
    if (rc) { fail(rc, "gpu_gguf_experts_forward"); return 0; }
    g_status = FM_OK;
    return 1;
}

int moe_experts_forward_chunk(int layer_idx, const float *h_post, const int *expert_indices,
                              const float *expert_weights, int M, int K, float *moe_out) {
    if (!g_ctx) { fail(FM_ERR_STATE, "moe_experts_forward_chunk"); return 0; }
    int rc = fm_moe_prefill(g_ctx, layer_idx, h_post, expert_indices, expert_weights, M, K,
                            moe_out, FM_ACCUMULATE);
    if (rc) { fail(rc, "moe_experts_forward_chunk"); return 0; }
    g_status = FM_OK;
    return 1;
}

int moe_experts_forward_chunk_bf16(int layer_idx, const uint16_t *h_post_bf16, const int *expert_indices,
                                   const float *expert_weights, int M, int K, float *moe_out) {
    if (!g_ctx) { fail(FM_ERR_STATE, "moe_experts_forward_chunk_bf16"); return 0; }
    int rc = fm_moe_prefill_bf16(g_ctx, layer_idx, h_post_bf16, expert_indices, expert_weights, M, K,
                                 moe_out, FM_ACCUMULATE);
    if (rc) { fail(rc, "moe_experts_forward_chunk_bf16"); return 0; }
    g_status = FM_OK;
    return 1;
}

int gpu_gguf_experts_forward_chunk(int layer_idx, const float *h_post, const int *expert_indices,
                                   const float *expert_weights, int M, int K, float *moe_out) {
    if (!g_ctx) { fail(FM_ERR_STATE, "gpu_gguf_experts_forward_chunk"); return 0; }
    int rc = fm_gguf_moe_prefill(g_ctx, layer_idx, h_post, expert_indices, expert_weights, M, K,
                                 moe_out, FM_ACCUMULATE);
    if (rc) { fail(rc, "gpu_gguf_experts_forward_chunk"); return 0; }
    g_status = FM_OK;
    return 1;
}

/* ---- routing (finchmoe/infer.m:1794-1840): runs on the host in the reference too ---- */
void cpu_softmax(float *x, int dim) {
    float mx = x[0];
    for (int i = 1; i < dim; i++) mx = x[i] > mx ? x[i] : mx;
    float sum = 0.0f;
    for (int i = 0; i < dim; i++) {
        x[i] = expf(x[i] - mx);
        sum += x[i];
    }
    float inv = 1.0f / sum;
    for (int i = 0; i < dim; i++) x[i] *= inv;
}

void cpu_topk(const float *scores, int dim, int K, int *indices, float *values) {
    for (int k = 0; k < K; k++) {
        values[k] = -1e30f;
        indices[k] = 0;
    }
    for (int i = 0; i < dim; i++) {
        int lowest = 0;   /* first slot holding the smallest kept value */
        for (int k = 1; k < K; k++)
            if (values[k] < values[lowest]) lowest = k;
        if (scores[i] > values[lowest]) {
            values[lowest] = scores[i];
            indices[lowest] = i;
        }
    }
}

void cpu_normalize_weights(float *weights, int K) {
    float sum = 0.0f;
    for (int k = 0; k < K; k++) sum += weights[k];
    if (sum > 0.0f) {
        float inv = 1.0f / sum;
        for (int k = 0; k < K; k++) weights[k] *= inv;
    }
}
