/* Driver for tests/test_host_fuzz.py: the host layer's bookkeeping (finch_ops.c: the table
 * from host weight pointers to resident tensors, the batch wrapper, the error paths) under the
 * host sanitizers, against doubles of the C ABI that only count.  What is checked: every
 * registered tensor is released at most once and only while registered, a pointer whose
 * shape changed is registered again, failing calls write zeros and never reach the
 * library, and the table survives tens of thousands of keys.  No GPU. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../finchmoe_amd/host/finch_ops.c"

/* ---- doubles of the C ABI ---- */
#define MAXT 200000
static unsigned char live[MAXT];
static int n_reg, n_rel, n_batch, bad;
static int fail_register_after = -1;
struct fm_ctx { int dummy; };
static struct fm_ctx the_ctx;
int fm_ctx_create(int device, fm_ctx **out) { (void)device; *out = &the_ctx; return FM_OK; }
int fm_ctx_destroy(fm_ctx *c) { (void)c; return FM_OK; }
const char *fm_last_error(fm_ctx *c) { (void)c; return "double"; }
const char *fm_status_string(int s) { (void)s; return "status"; }
int fm_tensor_register(fm_ctx *c, const void *W, const void *S, const void *B, int out_dim, int in_dim,
                       int group_size, int bits, int scale_dtype, fm_tensor *t) {
    (void)c; (void)S; (void)B; (void)group_size; (void)scale_dtype;
    if (!W || out_dim < 1 || in_dim < 1) return FM_ERR_ARG;
    if ((S == NULL) != (B == NULL)) { bad++; return FM_ERR_ARG; }     /* the wrapper normalises this */
    if (!S && bits != 16 && bits != 10 && bits != 11) { bad++; return FM_ERR_ARG; }   /* raw BF16 or GGUF */
    if (fail_register_after >= 0 && n_reg >= fail_register_after) return FM_ERR_NOMEM;
    if (n_reg >= MAXT) return FM_ERR_NOMEM;
    live[n_reg] = 1;
    *t = n_reg++;
    return FM_OK;
}
int fm_tensor_release(fm_ctx *c, fm_tensor t) {
    (void)c;
    if (t < 0 || t >= n_reg || !live[t]) { bad++; return FM_ERR_ARG; }
    live[t] = 0;
    n_rel++;
    return FM_OK;
}
int fm_matvec_batch(fm_ctx *c, const fm_tensor *ts, int n, const float *x, float *const *outs) {
    (void)c; (void)x;
    for (int i = 0; i < n; i++) {
        if (ts[i] < 0 || ts[i] >= n_reg || !live[ts[i]]) bad++;
        if (outs[i]) outs[i][0] = 1.0f;
    }
    n_batch++;
    return FM_OK;
}
int fm_matvec_prefill(fm_ctx *c, fm_tensor t, const float *X, float *out, int M) {
    (void)c; (void)X; (void)M;
    if (t < 0 || t >= n_reg || !live[t]) bad++;
    out[0] = 1.0f;
    return FM_OK;
}
int fm_gguf_matvec(fm_ctx *c, const void *W, int type, const float *x, float *out, int out_dim, int in_dim) {
    (void)c; (void)W; (void)type; (void)x; (void)out_dim; (void)in_dim;
    out[0] = 2.0f;
    return FM_OK;
}
int fm_experts_config(fm_ctx *c, int a, int b, int d, int e, int f, int g, int h) { (void)c; (void)a; (void)b; (void)d; (void)e; (void)f; (void)g; (void)h; return FM_OK; }
int fm_experts_upload_layer(fm_ctx *c, int l, const void *p, size_t n) { (void)c; (void)l; (void)p; (void)n; return FM_OK; }
int fm_gguf_config(fm_ctx *c, int a, int b, int d, int e, int f, int g, int h) { (void)c; (void)a; (void)b; (void)d; (void)e; (void)f; (void)g; (void)h; return FM_OK; }
int fm_gguf_upload_layer(fm_ctx *c, int l, const void *g, size_t gb, const void *u, size_t ub, const void *d, size_t db) { (void)c; (void)l; (void)g; (void)gb; (void)u; (void)ub; (void)d; (void)db; return FM_OK; }
int fm_moe_decode(fm_ctx *c, int l, const float *x, const int32_t *i, const float *w, int K, float *o, float *e, int f) { (void)c; (void)l; (void)x; (void)i; (void)w; (void)K; (void)e; (void)f; o[0] = 3.0f; return FM_OK; }
int fm_gguf_moe_decode(fm_ctx *c, int l, const float *x, const int32_t *i, const float *w, int K, float *o, float *e, int f) { (void)c; (void)l; (void)x; (void)i; (void)w; (void)K; (void)e; (void)f; o[0] = 4.0f; return FM_OK; }
int fm_moe_prefill(fm_ctx *c, int l, const float *X, const int32_t *i, const float *w, int M, int K, float *o, int f) { (void)c; (void)l; (void)X; (void)i; (void)w; (void)M; (void)K; (void)f; o[0] = 5.0f; return FM_OK; }

int fm_moe_prefill_bf16(fm_ctx *c, int l, const uint16_t *X, const int32_t *i, const float *w, int M, int K, float *o, int f) { (void)c; (void)l; (void)X; (void)i; (void)w; (void)M; (void)K; o[0] = f == FM_ACCUMULATE ? 6.0f : -1.0f; return l < 0 ? FM_ERR_ARG : FM_OK; }
int fm_gguf_moe_prefill(fm_ctx *c, int l, const float *X, const int32_t *i, const float *w, int M, int K, float *o, int f) { (void)c; (void)l; (void)X; (void)i; (void)w; (void)M; (void)K; o[0] = f == FM_ACCUMULATE ? 7.0f : -1.0f; return l < 0 ? FM_ERR_ARG : FM_OK; }

#define CHECK(cond) do { if (!(cond)) { printf("FAILED line %d: %s\n", __LINE__, #cond); return 1; } } while (0)

int main(void) {
    static uint32_t arena[70000];          /* distinct addresses to key the table with */
    uint16_t sb[4] = {0};
    float x[64] = {0}, out[256];
    /* before init: an error, zeros, nothing reaches the library */
    out[0] = 7.0f;
    fast_dequant_matvec(arena, sb, sb, x, out, 4, 64, 64, 4);
    CHECK(finch_ops_last_status() == FM_ERR_STATE && n_reg == 0);
    CHECK(finch_ops_make_resident(arena, sb, sb, 4, 64, 64, 4) == FM_ERR_STATE);
    finch_ops_forget_tensor(arena);        /* no table yet */
    CHECK(finch_ops_init(0) == FM_OK && finch_ops_init(0) == FM_OK);

    /* one key per address: the table grows from 1024 slots through several doublings */
    const int N = 60000;
    for (int i = 0; i < N; i++) CHECK(finch_ops_make_resident(&arena[i], sb, sb, 4, 64, 64, 4) == FM_OK);
    CHECK(n_reg == N && n_rel == 0);
    for (int i = 0; i < N; i += 7) CHECK(finch_ops_make_resident(&arena[i], sb, sb, 4, 64, 64, 4) == FM_OK);
    CHECK(n_reg == N);                                      /* known pointers are not registered again */
    /* bits 0 means 4 (finchmoe/infer.m:4491): the same tensor */
    CHECK(finch_ops_make_resident(&arena[5], sb, sb, 4, 64, 64, 0) == FM_OK && n_reg == N);
    /* host memory reused for another shape: released and registered again */
    CHECK(finch_ops_make_resident(&arena[5], sb, sb, 8, 64, 64, 4) == FM_OK && n_reg == N + 1 && n_rel == 1);
    /* scales without biases: an unquantized BF16 tensor, whatever bits says */
    CHECK(finch_ops_make_resident(&arena[6], sb, NULL, 4, 64, 64, 4) == FM_OK && n_reg == N + 2 && n_rel == 2);
    CHECK(finch_ops_make_resident(NULL, sb, sb, 4, 64, 64, 4) != FM_OK);
    /* forget: released once, a second forget and an unknown pointer do nothing */
    finch_ops_forget_tensor(&arena[9]);
    finch_ops_forget_tensor(&arena[9]);
    finch_ops_forget_tensor(&arena[69999]);
    CHECK(n_rel == 3);
    CHECK(finch_ops_make_resident(&arena[9], sb, sb, 4, 64, 64, 4) == FM_OK && n_reg == N + 3);

    /* the batch wrapper: outputs written on success, zeroed on any failure */
    BatchMatvecSpec sp[3];
    memset(sp, 0, sizeof sp);
    for (int i = 0; i < 3; i++) {
        sp[i].W = &arena[60100 + i]; sp[i].scales = sb; sp[i].biases = sb; sp[i].out_cpu = out + 64 * i;
        sp[i].out_dim = 4; sp[i].in_dim = 64; sp[i].group_size = 64; sp[i].bits = 4;
    }
    fast_batch_matvec(x, 64, sp, 3);
    CHECK(finch_ops_last_status() == FM_OK && out[0] == 1.0f && out[64] == 1.0f && out[128] == 1.0f);
    sp[1].in_dim = 128;                                     /* does not match x */
    out[0] = out[64] = out[128] = 9.0f;
    const int batches = n_batch;
    fast_batch_matvec(x, 64, sp, 3);
    CHECK(finch_ops_last_status() == FM_ERR_ARG && n_batch == batches && out[0] == 0.0f && out[64] == 0.0f && out[128] == 0.0f);
    sp[1].in_dim = 64;
    sp[2].scales = NULL; sp[2].bits = 10;                   /* a GGUF spec inside a batch: a resident tensor like the others */
    out[128] = 9.0f;
    fast_batch_matvec(x, 64, sp, 3);
    CHECK(finch_ops_last_status() == FM_OK && n_batch == batches + 1 && out[128] == 1.0f);
    fast_batch_matvec(x, 64, sp, 0);
    CHECK(finch_ops_last_status() == FM_ERR_ARG);
    fast_batch_matvec(x, 64, sp, 65);
    CHECK(finch_ops_last_status() == FM_ERR_ARG);
    /* a GGUF tensor on its own is registered once (bits 11, no scales) and stays resident */
    {
        const int regs = n_reg;
        fast_dequant_matvec(&arena[60200], NULL, NULL, x, out, 4, 256, 64, 11);
        CHECK(finch_ops_last_status() == FM_OK && out[0] == 1.0f && n_reg == regs + 1);
        fast_dequant_matvec(&arena[60200], NULL, NULL, x, out, 4, 256, 64, 11);
        CHECK(finch_ops_last_status() == FM_OK && n_reg == regs + 1);
    }
    /* registration failing inside the library: an error, zeros, the slot stays usable */
    fail_register_after = n_reg;
    out[0] = 9.0f;
    fast_dequant_matvec(&arena[60300], sb, sb, x, out, 4, 64, 64, 4);
    CHECK(finch_ops_last_status() == FM_ERR_NOMEM && out[0] == 0.0f);
    out[0] = 9.0f;
    fast_prefill_matvec(&arena[60300], sb, sb, x, out, 4, 64, 64, 4, 2);
    CHECK(finch_ops_last_status() == FM_ERR_NOMEM && out[0] == 0.0f);
    fail_register_after = -1;
    fast_dequant_matvec(&arena[60300], sb, sb, x, out, 4, 64, 64, 4);
    CHECK(finch_ops_last_status() == FM_OK && out[0] == 1.0f);

    /* the chunk wrappers: 1 / 0 like the reference's expert functions, accumulate flag passed on */
    {
        uint16_t xb[64] = {0};
        int idx[8] = {0};
        float w8[8] = {0};
        CHECK(moe_experts_forward_chunk_bf16(0, xb, idx, w8, 1, 8, out) == 1 && out[0] == 6.0f);
        CHECK(gpu_gguf_experts_forward_chunk(0, x, idx, w8, 1, 8, out) == 1 && out[0] == 7.0f);
        CHECK(moe_experts_forward_chunk_bf16(-1, xb, idx, w8, 1, 8, out) == 0 && finch_ops_last_status() == FM_ERR_ARG);
        CHECK(gpu_gguf_experts_forward_chunk(-1, x, idx, w8, 1, 8, out) == 0 && finch_ops_last_status() == FM_ERR_ARG);
    }

    finch_ops_shutdown();
    finch_ops_shutdown();
    CHECK(finch_ops_make_resident(arena, sb, sb, 4, 64, 64, 4) == FM_ERR_STATE);
    CHECK(bad == 0);
    printf("done registered=%d released=%d\n", n_reg, n_rel);
    return 0;
}
