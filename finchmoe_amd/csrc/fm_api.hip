// fm_api.hip — the C ABI of libfinchhip.so (include/finch_hip.h): context,
// HBM-resident weight stores, argument validation and kernel submission.
// Host logic only; kernels live in fm_decode / fm_dense / fm_dequant / fm_gguf /
// fm_prefill.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>
#include <string>
#include <algorithm>
#include <vector>

#include "fm_common.h"
#include "fm_route.h"     // RouteArgs

// ---- launchers implemented in the kernel files ------------------------------
extern "C" {
int fm_launch_decode_affine(const uint8_t *const *d_layer_ptrs, const FmExpertGeom *g,
                            int layer0, int layer_stride, int n_layers, const float *d_x,
                            const int32_t *d_idx, const float *d_w, int K, float *d_act,
                            float *d_expert_out, float *d_out, FmDecodeFlags *df, int flags,
                            int n_cu, hipStream_t st, hipEvent_t *kev, const FmTailArgs *tail);
int fm_launch_dense(FmDenseSpec *specs, int n, int in_dim, int bits, int scale_fp16,
                    const float *d_x, int M, int n_cu, hipStream_t st, const FmDenseSpec *riders,
                    int n_riders, int *riders_done);
int fm_launch_dense_mixed(FmDenseSpec *specs, int n, int in_dim, int scale_fp16, const float *d_x,
                          int n_cu, const RouteArgs *route, unsigned int *ticket, hipStream_t st);
int fm_launch_dense_bf16(const FmDenseSpec *specs, int n, int in_dim, const float *d_x, int M,
                         hipStream_t st);
int fm_launch_dense_lowbit(const FmDenseSpec *specs, int n, int in_dim, int bits, int scale_fp16,
                           const float *d_x, int M, hipStream_t st);
int fm_launch_stream_probe(const void *d_buf, size_t nbytes, int pattern, unsigned int *d_sink,
                           int n_cu, hipStream_t st);
int fm_launch_dequant_affine(const void *W, const void *S, const void *B, int out_dim,
                             int in_dim, int group_size, int bits, int scale_fp16,
                             uint8_t *codes, float *w32, uint16_t *w16, hipStream_t st);
int fm_launch_dequant_gguf(const void *W, int out_dim, int in_dim, int ggml_type, float *w32,
                           hipStream_t st);
int fm_launch_decode_gguf(const uint8_t *const *d_gate, const uint8_t *const *d_up,
                          const uint8_t *const *d_down, const FmGgufGeom *g, int layer0,
                          int layer_stride, int n_layers, const float *d_x,
                          const int32_t *d_idx, const float *d_w, int K, float *d_act,
                          float *d_expert_out, float *d_out, FmDecodeFlags *df,
                          int flags, int n_cu, hipStream_t st, hipEvent_t *kev);
int fm_launch_gguf_matvec(const uint8_t *d_W, int ggml_type, const float *d_x, float *d_out,
                          int out_dim, int in_dim, int n_cu, hipStream_t st);
int fm_launch_gguf_dense(const uint8_t *d_W, int ggml_type, const float *d_x, float *d_out, int out_dim,
                         int in_dim, int n_cu, hipStream_t st);
int fm_launch_embed_rows_gguf(const void *W, int rows, int in_dim, int ggml_type, const int32_t *d_ids,
                              int n, float *d_out, hipStream_t st);
int fm_launch_prefill_affine(const uint8_t *d_layer, const FmExpertGeom *g, const void *d_X,
                             int x_bf16, const int32_t *d_idx, const float *d_w, int M, int K,
                             float *d_out, void *d_ws, size_t ws_bytes, int flags, int n_cu,
                             hipStream_t st);
size_t fm_prefill_affine_ws_bytes(const FmExpertGeom *g, int M, int K, int x_bf16);
int fm_launch_widen_bf16(const uint16_t *d_src, float *d_dst, size_t n, hipStream_t st);
int fm_launch_layer_tail(const FmTailArgs *a, int bits, int scale_fp16, hipStream_t st);
int fm_launch_route(const float *d_logits, int n, int K, const float *d_seg_score, int32_t *d_idx,
                    float *d_w, float *d_params, hipStream_t st);
}

// ---- scratch of the entry point that allocates nothing (fm_moe_decode_step_noalloc_dev) ----
// One array per GPU, part of the library's device image, held until the process ends.  In
// host code the array's name is only a handle for hipGetSymbolAddress: the address kernels
// can use is looked up once per device (fm_ctx_create) and kept in g_noalloc_ptr.
#define FM_NOALLOC_BYTES (4u << 20)
static __device__ __align__(256) unsigned char fm_noalloc_scratch[FM_NOALLOC_BYTES];

namespace {

constexpr int FM_API_MAX_DEVICES = 64;
unsigned char *g_noalloc_ptr[FM_API_MAX_DEVICES] = {};
std::mutex g_noalloc_mutex;

// with `device` current
int noalloc_lookup(int device, unsigned char **out) {
    *out = nullptr;
    if (device < 0 || device >= FM_API_MAX_DEVICES) return FM_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (!g_noalloc_ptr[device]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(fm_noalloc_scratch)) != hipSuccess || !p)
            return FM_ERR_HIP;
        g_noalloc_ptr[device] = (unsigned char *)p;
    }
    *out = g_noalloc_ptr[device];
    return FM_OK;
}

// `bits` of a tensor registered without scales and biases: unquantized BF16 [out_dim][in_dim]
// (cpu_dequant_matvec's scales == NULL branch, finchmoe/infer.m:1689-1701)
constexpr int FM_BITS_RAW_BF16 = 16;

// `bits` of a GGUF block-format tensor, the reference's own convention for cpu_dequant_matvec
// and BatchMatvecSpec (finchmoe/infer.m:1684-1688): 10 = Q4_K, 11 = Q6_K
constexpr int FM_BITS_GGUF_Q4K = 10, FM_BITS_GGUF_Q6K = 11;

struct Tensor {
    bool used = false, owned = false;
    void *W = nullptr, *S = nullptr, *B = nullptr;
    int out_dim = 0, in_dim = 0, group_size = 0, bits = 0, scale_fp16 = 0;
    bool raw_bf16() const { return bits == FM_BITS_RAW_BF16; }
    bool gguf() const { return bits == FM_BITS_GGUF_Q4K || bits == FM_BITS_GGUF_Q6K; }
    int ggml_type() const { return bits == FM_BITS_GGUF_Q4K ? FM_GGML_Q4_K : FM_GGML_Q6_K; }
};

struct LayerBuf {
    void *ptr = nullptr;
    bool owned = false;
};

}  // namespace

#define FM_TAIL_PARTIALS 4096
#define FM_TAIL_VECTOR 16384
// positions of one chunk: the chunk kernels index pairs x hidden in 32 bits
#define FM_MAX_CHUNK 65535

struct fm_ctx {
    int device = 0;
    int n_cu = 256;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    hipEvent_t kev[3] = {nullptr, nullptr, nullptr};
    int ktiming = 0;   // 0 off, 1 whole operator, 2 phases as separate kernels
    // fused decode kernel: the word a timed-out wait raises (pinned host memory the
    // device writes directly, so checking it after a sync costs nothing) and the
    // dependency counters (allocated with the scratch)
    unsigned int *h_err = nullptr, *d_err = nullptr;
    FmDecodeFlags dflags{};
    bool scratch_pinned = false;   // a call has been issued under stream capture
    unsigned int wait_limit = 1u << 20;
    bool split_phases = false;     // run the phases as separate kernels
    bool sync_unchecked = false;   // a fused launch has not had its error flag read yet
    double k1_ms = 0.0, k2_ms = 0.0;
    int kcalls = 0;
    std::string err;

    // affine expert store
    bool aff_cfg = false;
    FmExpertGeom geom{};
    int n_layers = 0;
    std::vector<LayerBuf> layers;
    uint8_t **d_layer_ptrs = nullptr;

    // GGUF expert store
    bool gguf_cfg = false;
    FmGgufGeom ggeom{};
    int g_layers = 0;
    std::vector<LayerBuf> g_gate, g_up, g_down;
    uint8_t **d_gg_ptrs = nullptr;   // [3][g_layers]

    // scratch shared by both stores, sized for `cap_groups` groups of FM_MAX_K slots
    int cap_groups = 0, cap_hidden = 0, cap_inter = 0;
    float *d_act = nullptr, *d_eo = nullptr;
    unsigned int *d_counters = nullptr;
    // staging for the host-pointer entry points
    void *d_stage = nullptr;
    void *h_stage = nullptr;   // pinned mirror of d_stage: one copy in, one copy out per call
    size_t stage_bytes = 0;
    void *d_ws = nullptr;
    size_t ws_bytes = 0;
    // layer tail: one partial sum per workgroup, then the ticket counter
    float *d_tail = nullptr;
    // this device's copy of fm_noalloc_scratch
    unsigned char *noalloc = nullptr;

    std::vector<Tensor> tensors;
};

namespace {

int fail(fm_ctx *c, int code, const char *fmt, ...) {
    if (c) {
        char buf[512];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof buf, fmt, ap);
        va_end(ap);
        c->err = buf;
    }
    return code;
}

#define HIPCHK(c, call)                                                              \
    do {                                                                             \
        hipError_t e_ = (call);                                                      \
        if (e_ != hipSuccess)                                                        \
            return fail((c), FM_ERR_HIP, "%s: %s", #call, hipGetErrorString(e_));    \
    } while (0)

struct DeviceGuard {
    int prev = -1;
    explicit DeviceGuard(int dev) {
        (void)hipGetDevice(&prev);
        if (prev != dev) (void)hipSetDevice(dev);
        else prev = -1;
    }
    ~DeviceGuard() {
        if (prev >= 0) (void)hipSetDevice(prev);
    }
};

int ensure_stage(fm_ctx *c, size_t bytes) {
    if (c->stage_bytes >= bytes) return FM_OK;
    HIPCHK(c, hipStreamSynchronize(c->stream));
    if (c->d_stage) HIPCHK(c, hipFree(c->d_stage));
    if (c->h_stage) HIPCHK(c, hipHostFree(c->h_stage));
    c->d_stage = c->h_stage = nullptr;
    c->stage_bytes = 0;
    HIPCHK(c, hipMalloc(&c->d_stage, bytes));
    HIPCHK(c, hipHostMalloc(&c->h_stage, bytes, hipHostMallocDefault));
    c->stage_bytes = bytes;
    return FM_OK;
}

// A graph captured from this context's stream has the scratch addresses of the moment baked in:
// from the first call issued under capture on, the scratch buffers are pinned — a call that
// would have to reallocate them is refused instead (FM_ERR_STATE), until fm_release_graphs().
// Sizes are reserved before capturing with fm_reserve().
bool note_capture(fm_ctx *c) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(c->stream, &cs);
    const bool capturing = cs == hipStreamCaptureStatusActive;
    if (capturing) c->scratch_pinned = true;
    return capturing;
}
int refuse_growth(fm_ctx *c, const char *what) {
    return fail(c, FM_ERR_STATE,
                "%s would have to grow, but a captured graph holds the current addresses: call "
                "fm_reserve() before capturing (or fm_release_graphs() once the graphs are gone)", what);
}

int ensure_ws(fm_ctx *c, size_t bytes) {
    note_capture(c);
    if (c->ws_bytes >= bytes) return FM_OK;
    if (c->scratch_pinned) return refuse_growth(c, "the workspace");
    HIPCHK(c, hipStreamSynchronize(c->stream));    // queued work may still use the old one
    if (c->d_ws) HIPCHK(c, hipFree(c->d_ws));
    c->d_ws = nullptr;
    c->ws_bytes = 0;
    HIPCHK(c, hipMalloc(&c->d_ws, bytes));
    c->ws_bytes = bytes;
    return FM_OK;
}

// scratch for `groups` groups (layers of a step, or positions of a chunk)
int ensure_scratch(fm_ctx *c, int groups, int hidden, int inter) {
    note_capture(c);
    if (groups <= c->cap_groups && hidden <= c->cap_hidden && inter <= c->cap_inter)
        return FM_OK;
    if (c->scratch_pinned) return refuse_growth(c, "the expert scratch");
    int g = groups > c->cap_groups ? groups : c->cap_groups;
    int h = hidden > c->cap_hidden ? hidden : c->cap_hidden;
    int in = inter > c->cap_inter ? inter : c->cap_inter;
    HIPCHK(c, hipStreamSynchronize(c->stream));
    if (c->d_act) (void)hipFree(c->d_act);
    if (c->d_eo) (void)hipFree(c->d_eo);
    if (c->d_counters) (void)hipFree(c->d_counters);
    if (c->dflags.set[0]) (void)hipFree(c->dflags.set[0]);
    if (c->dflags.act_set[0]) (void)hipFree(c->dflags.act_set[0]);
    c->d_act = c->d_eo = nullptr;
    c->d_counters = nullptr;
    c->dflags = FmDecodeFlags{};
    c->cap_groups = 0;
    HIPCHK(c, hipMalloc((void **)&c->d_act, (size_t)g * FM_MAX_K * in * sizeof(float)));
    HIPCHK(c, hipMalloc((void **)&c->d_eo, (size_t)g * FM_MAX_K * h * sizeof(float)));
    HIPCHK(c, hipMalloc((void **)&c->d_counters, (size_t)g * sizeof(unsigned int)));
    HIPCHK(c, hipMemsetAsync(c->d_counters, 0, (size_t)g * sizeof(unsigned int), c->stream));
    {   // three sets of (pairs + groups) dependency counters, cleared once
        const size_t cap = (size_t)g * (FM_MAX_K + 1);
        unsigned int *p = nullptr;
        HIPCHK(c, hipMalloc((void **)&p, 3 * cap * sizeof(unsigned int)));
        HIPCHK(c, hipMemsetAsync(p, 0, 3 * cap * sizeof(unsigned int), c->stream));
        c->dflags.set[0] = p;
        c->dflags.set[1] = p + cap;
        c->dflags.graph_set = p + 2 * cap;
        c->dflags.cap = (unsigned int)cap;
        c->dflags.err = c->d_err;
        c->dflags.spin_limit = c->wait_limit;
    }
    {   // three activation sets of the launch that sums in LDS, every element marked "not
        // produced yet" (0xFFC5A3E1, FM_ACT_EMPTY of fm_decode.hip)
        // (+ hidden: the per-row-block sums of squares of the launch that takes the layer tail along)
        const size_t cap = (size_t)g * FM_MAX_K * in + (size_t)h;
        float *p = nullptr;
        HIPCHK(c, hipMalloc((void **)&p, 3 * cap * sizeof(float)));
        HIPCHK(c, hipMemsetD32Async((hipDeviceptr_t)p, (int)0xFFC5A3E1u, 3 * cap, c->stream));
        c->dflags.act_set[0] = p;
        c->dflags.act_set[1] = p + cap;
        c->dflags.act_graph = p + 2 * cap;
        c->dflags.act_cap = (unsigned int)cap;
    }
    c->cap_groups = g;
    c->cap_hidden = h;
    c->cap_inter = in;
    return FM_OK;
}

void free_layers(std::vector<LayerBuf> &v) {
    for (auto &l : v)
        if (l.owned && l.ptr) (void)hipFree(l.ptr);
    v.clear();
}

int set_layer(fm_ctx *c, std::vector<LayerBuf> &v, int layer, const void *src, size_t nbytes,
              bool adopt) {
    LayerBuf &lb = v[layer];
    if (adopt) {
        if (lb.owned && lb.ptr) HIPCHK(c, hipFree(lb.ptr));
        lb.ptr = const_cast<void *>(src);
        lb.owned = false;
        return FM_OK;
    }
    if (!lb.owned || !lb.ptr) {
        lb.ptr = nullptr;
        lb.owned = false;
        HIPCHK(c, hipMalloc(&lb.ptr, nbytes));
        lb.owned = true;
    }
    HIPCHK(c, hipMemcpy(lb.ptr, src, nbytes, hipMemcpyHostToDevice));
    return FM_OK;
}

bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }

size_t gguf_row_bytes(int in_dim, int type) {
    return (size_t)(in_dim / 256) * (type == FM_GGML_Q4_K ? 144u : 210u);
}

}  // namespace

// ============================================================================
// context
// ============================================================================
unsigned int fm_kernel_forms = 0;

extern "C" int fm_set_kernel_forms(unsigned int forms) {
    if (forms & ~(unsigned)(FM_FORM_PLAIN_DENSE | FM_FORM_PLAIN_GGUF | FM_FORM_NO_DENSE_GEMM | FM_FORM_NO_GGUF_GROUP |
                           FM_FORM_GGUF_PHASES | FM_FORM_GGUF_ONE_LAUNCH))
        return FM_ERR_ARG;
    fm_kernel_forms = forms;
    return FM_OK;
}

extern "C" int fm_ctx_create(int device, fm_ctx **out) {
    if (!out) return FM_ERR_ARG;
    *out = nullptr;
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || device < 0 || device >= ndev)
        return FM_ERR_HIP;   // no GPU: there is no CPU fallback
    fm_ctx *c = new (std::nothrow) fm_ctx;
    if (!c) return FM_ERR_NOMEM;
    c->device = device;
    DeviceGuard dg(device);
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess && prop.multiProcessorCount > 0)
        c->n_cu = prop.multiProcessorCount;
    if (hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreate(&c->ev0) != hipSuccess || hipEventCreate(&c->ev1) != hipSuccess) {
        delete c;
        return FM_ERR_HIP;
    }
    for (auto &e : c->kev)
        if (hipEventCreate(&e) != hipSuccess) {
            delete c;
            return FM_ERR_HIP;
        }
    if (hipHostMalloc((void **)&c->h_err, sizeof(unsigned int), hipHostMallocMapped) !=
            hipSuccess ||
        hipHostGetDevicePointer((void **)&c->d_err, c->h_err, 0) != hipSuccess) {
        delete c;
        return FM_ERR_NOMEM;
    }
    *c->h_err = 0u;
    if (noalloc_lookup(device, &c->noalloc) != FM_OK) {
        (void)hipHostFree(c->h_err);
        delete c;
        return FM_ERR_HIP;
    }
    if (const char *e = getenv("FINCH_DECODE_SPLIT")) c->split_phases = e[0] == '1';
    *out = c;
    return FM_OK;
}

extern "C" int fm_ctx_destroy(fm_ctx *c) {
    if (!c) return FM_ERR_ARG;
    DeviceGuard dg(c->device);
    (void)hipStreamSynchronize(c->stream);
    free_layers(c->layers);
    free_layers(c->g_gate);
    free_layers(c->g_up);
    free_layers(c->g_down);
    for (auto &t : c->tensors)
        if (t.used && t.owned) {
            (void)hipFree(t.W);
            if (t.S) (void)hipFree(t.S);
            if (t.B) (void)hipFree(t.B);
        }
    if (c->h_err) (void)hipHostFree(c->h_err);
    void *ptrs[] = {c->d_layer_ptrs, c->d_gg_ptrs, c->d_act, c->d_eo, c->d_counters,
                    c->dflags.set[0], c->dflags.act_set[0],
                    c->d_stage, c->d_ws, c->d_tail};
    if (c->h_stage) (void)hipHostFree(c->h_stage);
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    (void)hipEventDestroy(c->ev0);
    (void)hipEventDestroy(c->ev1);
    for (auto &e : c->kev) (void)hipEventDestroy(e);
    (void)hipStreamDestroy(c->stream);
    delete c;
    return FM_OK;
}

// After the stream has drained: did a fused decode launch give up on a wait?
static int check_grid_error(fm_ctx *c) {
    if (!c->sync_unchecked) return FM_OK;
    c->sync_unchecked = false;
    volatile unsigned int *flag = c->h_err;
    if (!*flag) return FM_OK;
    *flag = 0u;
    return fail(c, FM_ERR_HIP, "decode kernel: a wait on another workgroup timed out, results are invalid");
}

extern "C" int fm_sync(fm_ctx *c) {
    if (!c) return FM_ERR_ARG;
    DeviceGuard dg(c->device);
    HIPCHK(c, hipStreamSynchronize(c->stream));
    return check_grid_error(c);
}

extern "C" void *fm_stream(fm_ctx *c) { return c ? (void *)c->stream : nullptr; }

extern "C" const char *fm_last_error(fm_ctx *c) { return c ? c->err.c_str() : "null context"; }

extern "C" const char *fm_status_string(int s) {
    switch (s) {
        case FM_OK: return "ok";
        case FM_ERR_ARG: return "bad argument";
        case FM_ERR_HIP: return "HIP runtime error";
        case FM_ERR_STATE: return "store not configured or layer not resident";
        case FM_ERR_UNSUPPORTED: return "unsupported format or shape";
        case FM_ERR_NOMEM: return "out of memory";
        default: return "unknown status";
    }
}

extern "C" int fm_timer_start(fm_ctx *c) {
    if (!c) return FM_ERR_ARG;
    DeviceGuard dg(c->device);
    HIPCHK(c, hipEventRecord(c->ev0, c->stream));
    return FM_OK;
}

extern "C" int fm_timer_stop(fm_ctx *c, float *ms) {
    if (!c || !ms) return FM_ERR_ARG;
    DeviceGuard dg(c->device);
    HIPCHK(c, hipEventRecord(c->ev1, c->stream));
    // (the stream, not the event, is waited for: the runtime's wait for a stream returns about
    // 20 microseconds sooner, which a caller that also brackets a short run with a wall clock sees)
    HIPCHK(c, hipStreamSynchronize(c->stream));
    HIPCHK(c, hipEventElapsedTime(ms, c->ev0, c->ev1));
    return FM_OK;
}

extern "C" int fm_kernel_timing(fm_ctx *c, int enable) {
    if (!c) return FM_ERR_ARG;
    c->ktiming = enable < 0 ? 0 : (enable > 2 ? 2 : enable);
    c->k1_ms = c->k2_ms = 0.0;
    c->kcalls = 0;
    return FM_OK;
}

extern "C" int fm_set_wait_limit(fm_ctx *c, unsigned int polls) {
    if (!c) return FM_ERR_ARG;
    c->wait_limit = polls;
    c->dflags.spin_limit = polls;
    return FM_OK;
}

// Scratch for steps of up to n_groups layers and chunks of up to M positions on the configured
// stores, the layer tail's scratch, and at least workspace_bytes of workspace — so that no
// later call of those sizes allocates (a precondition for capturing calls into a HIP graph).
extern "C" int fm_reserve(fm_ctx *c, int n_groups, int M, size_t workspace_bytes) {
    if (!c) return FM_ERR_ARG;
    if (n_groups < 0 || M < 0) return fail(c, FM_ERR_ARG, "negative size");
    DeviceGuard dg(c->device);
    if (note_capture(c)) return fail(c, FM_ERR_STATE, "fm_reserve under stream capture");
    const int groups = n_groups > M ? n_groups : M;   // small chunks run as groups of the decode kernels
    int rc = FM_OK;
    size_t ws = workspace_bytes;
    if (c->aff_cfg) {
        if (groups > 0 && (rc = ensure_scratch(c, groups, c->geom.hidden, c->geom.inter))) return rc;
        if (M > 0) {
            const size_t widen = (size_t)M * c->geom.hidden * sizeof(float);
            const size_t a0 = fm_prefill_affine_ws_bytes(&c->geom, M, FM_MAX_K, 0);
            const size_t a1 = fm_prefill_affine_ws_bytes(&c->geom, M, FM_MAX_K, 1);
            ws = std::max(ws, std::max(widen, std::max(a0, a1)));
        }
    }
    if (c->gguf_cfg && groups > 0 && (rc = ensure_scratch(c, groups, c->ggeom.hidden, c->ggeom.inter))) return rc;
    if (ws && (rc = ensure_ws(c, ws))) return rc;
    if (!c->d_tail) {
        HIPCHK(c, hipMalloc((void **)&c->d_tail, (FM_TAIL_PARTIALS + 64 + FM_TAIL_VECTOR) * sizeof(float)));
        HIPCHK(c, hipMemsetAsync(c->d_tail, 0, (FM_TAIL_PARTIALS + 64) * sizeof(float), c->stream));
    }
    return FM_OK;
}

// The caller no longer replays any graph captured from this context: scratch may move again.
extern "C" int fm_release_graphs(fm_ctx *c) {
    if (!c) return FM_ERR_ARG;
    c->scratch_pinned = false;
    return FM_OK;
}

extern "C" int fm_kernel_timing_read(fm_ctx *c, double *k1, double *k2, int *calls) {
    if (!c) return FM_ERR_ARG;
    if (k1) *k1 = c->k1_ms;
    if (k2) *k2 = c->k2_ms;
    if (calls) *calls = c->kcalls;
    c->k1_ms = c->k2_ms = 0.0;
    c->kcalls = 0;
    return FM_OK;
}

// after a decode launch with the three timing events recorded
static int ktiming_collect(fm_ctx *c) {
    HIPCHK(c, hipEventSynchronize(c->kev[2]));
    float a = 0.0f, b = 0.0f;
    HIPCHK(c, hipEventElapsedTime(&a, c->kev[0], c->kev[1]));
    HIPCHK(c, hipEventElapsedTime(&b, c->kev[1], c->kev[2]));
    c->k1_ms += a;
    c->k2_ms += b;
    c->kcalls++;
    return check_grid_error(c);
}

extern "C" int fm_stream_probe_dev(fm_ctx *c, const void *d_buf, size_t nbytes, int pattern) {
    if (!c) return FM_ERR_ARG;
    if (!d_buf || nbytes < 4096 || ((uintptr_t)d_buf & 15) || pattern < 0 || pattern > 15)
        return fail(c, FM_ERR_ARG, "stream probe: a 16-byte aligned buffer of 4 KB or more, pattern 0..15");
    DeviceGuard dg(c->device);
    int rc = fm_launch_stream_probe(d_buf, nbytes, pattern, nullptr, c->n_cu, c->stream);
    if (rc) return fail(c, rc, "stream probe launch failed: %s", hipGetErrorString(hipGetLastError()));
    return FM_OK;
}

// ============================================================================
// affine expert store
// ============================================================================
extern "C" int fm_experts_config(fm_ctx *c, int n_layers, int n_experts, int hidden, int inter,
                                 int group_size, int bits, int scale_dtype) {
    if (!c) return FM_ERR_ARG;
    if (n_layers < 1 || n_experts < 1 || hidden < 1 || inter < 1)
        return fail(c, FM_ERR_ARG, "experts_config: non-positive dimension");
    if (group_size != 64) return fail(c, FM_ERR_UNSUPPORTED, "group_size %d (only 64)", group_size);
    if (bits != 3 && bits != 4) return fail(c, FM_ERR_UNSUPPORTED, "expert bits %d (3 or 4)", bits);
    if (scale_dtype != FM_SCALE_BF16 && scale_dtype != FM_SCALE_FP16)
        return fail(c, FM_ERR_ARG, "scale_dtype %d", scale_dtype);
    // a lane owns 128 columns; 4..32 lanes per gate/up row, 1..16 per down row
    int lu = hidden / 128, ld = inter / 128;
    if (hidden % 128 || inter % 128 || !pow2(lu) || !pow2(ld) || lu < 4 || lu > 32 || ld > 16 ||
        inter % (4 * (64 / lu)) || hidden % (4 * (64 / ld)))
        return fail(c, FM_ERR_UNSUPPORTED, "hidden %d / inter %d: need 128*2^j columns", hidden,
                    inter);
    DeviceGuard dg(c->device);
    HIPCHK(c, hipStreamSynchronize(c->stream));
    free_layers(c->layers);
    if (c->d_layer_ptrs) HIPCHK(c, hipFree(c->d_layer_ptrs));
    c->d_layer_ptrs = nullptr;
    c->aff_cfg = false;

    FmExpertGeom &g = c->geom;
    g.hidden = hidden;
    g.inter = inter;
    g.group_size = group_size;
    g.bits = bits;
    g.scale_fp16 = scale_dtype == FM_SCALE_FP16;
    g.n_experts = n_experts;
    // finchmoe/repack_experts.py:76-87, 141-151: W, scales, biases of gate, up, down
    uint64_t gu_w = (uint64_t)inter * hidden * bits / 8, gu_s = (uint64_t)inter * (hidden / 64) * 2;
    uint64_t d_w = (uint64_t)hidden * inter * bits / 8, d_s = (uint64_t)hidden * (inter / 64) * 2;
    uint64_t o = 0;
    g.gate_w = (uint32_t)o; o += gu_w; g.gate_s = (uint32_t)o; o += gu_s; g.gate_b = (uint32_t)o; o += gu_s;
    g.up_w = (uint32_t)o;   o += gu_w; g.up_s = (uint32_t)o;   o += gu_s; g.up_b = (uint32_t)o;   o += gu_s;
    g.down_w = (uint32_t)o; o += d_w;  g.down_s = (uint32_t)o; o += d_s;  g.down_b = (uint32_t)o; o += d_s;
    g.expert_size = o;
    c->n_layers = n_layers;
    c->layers.assign(n_layers, LayerBuf());
    HIPCHK(c, hipMalloc((void **)&c->d_layer_ptrs, (size_t)n_layers * sizeof(uint8_t *)));
    HIPCHK(c, hipMemset(c->d_layer_ptrs, 0, (size_t)n_layers * sizeof(uint8_t *)));
    c->aff_cfg = true;
    return FM_OK;
}

extern "C" size_t fm_experts_expert_size(fm_ctx *c) {
    return (c && c->aff_cfg) ? (size_t)c->geom.expert_size : 0;
}

static int experts_set_layer(fm_ctx *c, int layer, const void *blob, size_t nbytes, bool adopt) {
    if (!c) return FM_ERR_ARG;
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    if (!blob || layer < 0 || layer >= c->n_layers) return fail(c, FM_ERR_ARG, "layer %d", layer);
    size_t want = (size_t)c->geom.n_experts * c->geom.expert_size;
    if (nbytes != want)
        return fail(c, FM_ERR_ARG, "layer blob is %zu bytes, expected %zu", nbytes, want);
    if (adopt && ((uintptr_t)blob & 15)) return fail(c, FM_ERR_ARG, "device blob not 16-byte aligned");
    DeviceGuard dg(c->device);
    HIPCHK(c, hipStreamSynchronize(c->stream));
    int rc = set_layer(c, c->layers, layer, blob, nbytes, adopt);
    if (rc) return rc;
    HIPCHK(c, hipMemcpy(c->d_layer_ptrs + layer, &c->layers[layer].ptr, sizeof(void *),
                        hipMemcpyHostToDevice));
    return FM_OK;
}

extern "C" int fm_experts_upload_layer(fm_ctx *c, int layer, const void *blob, size_t nbytes) {
    return experts_set_layer(c, layer, blob, nbytes, false);
}
extern "C" int fm_experts_adopt_layer(fm_ctx *c, int layer, const void *blob, size_t nbytes) {
    return experts_set_layer(c, layer, blob, nbytes, true);
}

// ============================================================================
// routed experts, decode
// ============================================================================
static int check_layers(fm_ctx *c, const std::vector<LayerBuf> &v, int layer0, int n) {
    if (layer0 < 0 || n < 1 || layer0 + n > (int)v.size())
        return fail(c, FM_ERR_ARG, "layers %d..%d out of range", layer0, layer0 + n - 1);
    for (int l = layer0; l < layer0 + n; l++)
        if (!v[l].ptr) return fail(c, FM_ERR_STATE, "layer %d not resident", l);
    return FM_OK;
}

extern "C" int fm_moe_decode_step_dev(fm_ctx *c, int layer0, int n_layers, const float *d_x,
                                      const int32_t *d_idx, const float *d_w, int K,
                                      float *d_out, float *d_expert_out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    if (!d_x || !d_idx || !d_w || !d_out) return fail(c, FM_ERR_ARG, "null pointer");
    if (K < 1 || K > FM_MAX_K) return fail(c, FM_ERR_ARG, "K %d outside 1..%d", K, FM_MAX_K);
    int rc = check_layers(c, c->layers, layer0, n_layers);
    if (rc) return rc;
    DeviceGuard dg(c->device);
    rc = ensure_scratch(c, n_layers, c->geom.hidden, c->geom.inter);
    if (rc) return rc;
    const bool split = c->split_phases || c->ktiming == 2;
    rc = fm_launch_decode_affine(c->d_layer_ptrs, &c->geom, layer0, 1, n_layers, d_x, d_idx, d_w,
                                 K, c->d_act, d_expert_out ? d_expert_out : c->d_eo, d_out,
                                 split ? nullptr : &c->dflags,
                                 flags | (d_expert_out ? 0 : FM_INT_NO_EXPERT_OUT), c->n_cu, c->stream,
                                 c->ktiming ? c->kev : nullptr, nullptr);
    if (rc) return fail(c, rc, "decode launch failed: %s", hipGetErrorString(hipGetLastError()));
    if (!split) c->sync_unchecked = true;
    if (c->ktiming) return ktiming_collect(c);
    return FM_OK;
}

extern "C" int fm_moe_decode_dev(fm_ctx *c, int layer, const float *d_x, const int32_t *d_idx,
                                 const float *d_w, int K, float *d_out, float *d_expert_out,
                                 int flags) {
    return fm_moe_decode_step_dev(c, layer, 1, d_x, d_idx, d_w, K, d_out, d_expert_out, flags);
}

// fm_moe_decode_step_dev for callers that must not allocate: the SwiGLU activations, the
// per-expert vectors and one set of dependency counters live in this device's copy of
// fm_noalloc_scratch instead of the context's growable buffers.  The array keeps the last
// call's contents: the counters are cleared by a kernel in front of the operator (a fill
// kernel, not a memset, so that the pair can be captured into a graph); the vectors are
// fully rewritten before they are read.
extern "C" int fm_moe_decode_step_noalloc_dev(fm_ctx *c, int layer0, int n_layers, const float *d_x,
                                              const int32_t *d_idx, const float *d_w, int K,
                                              float *d_out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    if (!d_x || !d_idx || !d_w || !d_out) return fail(c, FM_ERR_ARG, "null pointer");
    if (K < 1 || K > FM_MAX_K) return fail(c, FM_ERR_ARG, "K %d outside 1..%d", K, FM_MAX_K);
    int rc = check_layers(c, c->layers, layer0, n_layers);
    if (rc) return rc;
    if (!c->noalloc) return fail(c, FM_ERR_STATE, "no scratch array on device %d", c->device);
    // layout: act [n_layers][8][inter] | expert_out [n_layers][8][hidden] | counters
    const size_t act_b = (size_t)n_layers * FM_MAX_K * c->geom.inter * sizeof(float);
    const size_t eo_b = (size_t)n_layers * FM_MAX_K * c->geom.hidden * sizeof(float);
    const size_t cnt_n = (size_t)n_layers * (FM_MAX_K + 1);
    const size_t need = act_b + eo_b + cnt_n * sizeof(unsigned int);
    if (need > FM_NOALLOC_BYTES)
        return fail(c, FM_ERR_ARG,
                    "%d layers of hidden %d / inter %d need %zu bytes of scratch, the fixed array "
                    "holds %u (use fm_moe_decode_step_dev)", n_layers, c->geom.hidden, c->geom.inter,
                    need, (unsigned)FM_NOALLOC_BYTES);
    DeviceGuard dg(c->device);
    unsigned char *s = c->noalloc;
    FmDecodeFlags df{};
    df.graph_set = (unsigned int *)(s + act_b + eo_b);
    df.cap = (unsigned int)cnt_n;
    df.err = c->d_err;
    df.spin_limit = c->wait_limit;
    df.always_graph_set = 1;
    rc = fm_launch_decode_affine(c->d_layer_ptrs, &c->geom, layer0, 1, n_layers, d_x, d_idx, d_w,
                                 K, (float *)s, (float *)(s + act_b), d_out,
                                 c->split_phases ? nullptr : &df, flags, c->n_cu, c->stream,
                                 nullptr, nullptr);
    if (rc) return fail(c, rc, "decode launch failed: %s", hipGetErrorString(hipGetLastError()));
    if (!c->split_phases) c->sync_unchecked = true;
    return FM_OK;
}

// host-pointer wrapper shared by the affine and GGUF stores and by decode
// (M = 1) and prefill (M positions)
typedef int (*moe_dev_fn)(fm_ctx *, int, const float *, const int32_t *, const float *, int, int,
                          float *, float *, int);

// (x_elem: bytes per activation of x — 4 for fp32, 2 for bf16 bits; fn gets the staged x as
// a float pointer either way and knows what it holds)
static int moe_host_call(fm_ctx *c, moe_dev_fn fn, int hidden, int layer, const void *x,
                         const int32_t *idx, const float *w, int M, int K, float *out,
                         float *expert_out, int flags, size_t x_elem = 4) {
    if (!x || !idx || !w || !out) return fail(c, FM_ERR_ARG, "null pointer");
    if (M < 1 || M > FM_MAX_CHUNK) return fail(c, FM_ERR_ARG, "M %d outside 1..%d", M, FM_MAX_CHUNK);
    if (K < 1 || K > FM_MAX_K) return fail(c, FM_ERR_ARG, "K %d outside 1..%d", K, FM_MAX_K);
    DeviceGuard dg(c->device);
    size_t nx = (size_t)M * hidden * 4, ni = (size_t)M * K * 4, ne = (size_t)M * K * hidden * 4;
    const size_t nxi = (size_t)M * hidden * x_elem;
    size_t off_x = 0, off_i = off_x + ((nxi + 255) & ~(size_t)255), off_w = off_i + ((ni + 255) & ~(size_t)255);
    size_t off_o = off_w + ((ni + 255) & ~(size_t)255), off_e = off_o + nx;
    int rc = ensure_stage(c, off_e + (expert_out ? ne : 0));
    if (rc) return rc;
    // inputs through the pinned mirror: one copy in (x | idx | w | out if accumulating), one
    // copy out (out | expert_out) — pageable copies cost ~10 us each
    char *st = (char *)c->d_stage, *hs = (char *)c->h_stage;
    // A synchronous caller can be given a second try: if the one-launch kernel reports that a
    // wait on another workgroup ran out (its grid was not resident at once, say under another
    // tenant of the GPU), the call is repeated once as separate kernels, which wait for nothing.
    const bool split_before = c->split_phases;
    for (int attempt = 0; attempt < 2; attempt++) {
        memcpy(hs + off_x, x, nxi);
        memcpy(hs + off_i, idx, ni);
        memcpy(hs + off_w, w, ni);
        size_t in_bytes = off_w + ni;
        if (flags & FM_ACCUMULATE) {
            memcpy(hs + off_o, out, nx);
            in_bytes = off_o + nx;
        }
        HIPCHK(c, hipMemcpyAsync(st, hs, in_bytes, hipMemcpyHostToDevice, c->stream));
        rc = fn(c, layer, (const float *)(st + off_x), (const int32_t *)(st + off_i),
                (const float *)(st + off_w), M, K, (float *)(st + off_o),
                expert_out ? (float *)(st + off_e) : nullptr, flags);
        c->split_phases = split_before;
        if (rc) return rc;
        const size_t out_bytes = nx + (expert_out ? ne : 0);
        HIPCHK(c, hipMemcpyAsync(hs + off_o, st + off_o, out_bytes, hipMemcpyDeviceToHost, c->stream));
        HIPCHK(c, hipStreamSynchronize(c->stream));
        rc = check_grid_error(c);
        if (rc == FM_OK) break;
        if (attempt == 1 || split_before) return rc;
        c->split_phases = true;
    }
    memcpy(out, hs + off_o, nx);
    if (expert_out) memcpy(expert_out, hs + off_e, ne);
    return FM_OK;
}

static int aff_decode_fn(fm_ctx *c, int layer, const float *x, const int32_t *idx, const float *w,
                         int, int K, float *out, float *eo, int flags) {
    return fm_moe_decode_step_dev(c, layer, 1, x, idx, w, K, out, eo, flags);
}

extern "C" int fm_moe_decode(fm_ctx *c, int layer, const float *x, const int32_t *idx,
                             const float *w, int K, float *out, float *expert_out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    return moe_host_call(c, aff_decode_fn, c->geom.hidden, layer, x, idx, w, 1, K, out,
                         expert_out, flags);
}

// ============================================================================
// routed experts, chunked prefill
// ============================================================================
// Chunks below this many positions run the decode kernels once per position
// (grid-batched); larger chunks are grouped by expert for the MFMA GEMM.
#define FM_PREFILL_GEMM_MIN_M 32

static int moe_prefill_any(fm_ctx *c, int layer, const void *d_X, bool x_bf16, const int32_t *d_idx,
                           const float *d_w, int M, int K, float *d_out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    if (!d_X || !d_idx || !d_w || !d_out) return fail(c, FM_ERR_ARG, "null pointer");
    if (M < 1 || M > FM_MAX_CHUNK) return fail(c, FM_ERR_ARG, "M %d outside 1..%d", M, FM_MAX_CHUNK);
    if (K < 1 || K > FM_MAX_K) return fail(c, FM_ERR_ARG, "K %d outside 1..%d", K, FM_MAX_K);
    if (((uintptr_t)d_X | (uintptr_t)d_out) & 15)
        return fail(c, FM_ERR_ARG, "X / out not 16-byte aligned");
    int rc = check_layers(c, c->layers, layer, 1);
    if (rc) return rc;
    DeviceGuard dg(c->device);
    if (M >= FM_PREFILL_GEMM_MIN_M && !(flags & FM_GUARD)) {
        size_t ws = fm_prefill_affine_ws_bytes(&c->geom, M, K, x_bf16);
        if (ws) {
            rc = ensure_ws(c, ws);
            if (rc) return rc;
            rc = fm_launch_prefill_affine((const uint8_t *)c->layers[layer].ptr, &c->geom, d_X, x_bf16,
                                          d_idx, d_w, M, K, d_out, c->d_ws, c->ws_bytes, flags,
                                          c->n_cu, c->stream);
            if (rc != FM_ERR_UNSUPPORTED) {
                if (rc) return fail(c, rc, "prefill launch failed: %s",
                                    hipGetErrorString(hipGetLastError()));
                return FM_OK;
            }
        }
    }
    // one decode group per position (small chunks, guarded calls, widths without a GEMM); the
    // decode kernels read fp32: bf16 activations are widened into the workspace first
    const float *xf = (const float *)d_X;
    if (x_bf16) {
        const size_t nx = (size_t)M * c->geom.hidden;
        rc = ensure_ws(c, nx * sizeof(float));
        if (rc) return rc;
        rc = fm_launch_widen_bf16((const uint16_t *)d_X, (float *)c->d_ws, nx, c->stream);
        if (rc) return fail(c, rc, "widening launch failed: %s", hipGetErrorString(hipGetLastError()));
        xf = (const float *)c->d_ws;
    }
    rc = ensure_scratch(c, M, c->geom.hidden, c->geom.inter);
    if (rc) return rc;
    rc = fm_launch_decode_affine(c->d_layer_ptrs, &c->geom, layer, 0, M, xf, d_idx, d_w, K,
                                 c->d_act, c->d_eo, d_out, c->split_phases ? nullptr : &c->dflags,
                                 flags | FM_INT_NO_EXPERT_OUT, c->n_cu, c->stream, nullptr, nullptr);
    if (rc) return fail(c, rc, "prefill launch failed: %s", hipGetErrorString(hipGetLastError()));
    if (!c->split_phases) c->sync_unchecked = true;
    return FM_OK;
}

extern "C" int fm_moe_prefill_dev(fm_ctx *c, int layer, const float *d_X, const int32_t *d_idx,
                                  const float *d_w, int M, int K, float *d_out, int flags) {
    return moe_prefill_any(c, layer, d_X, false, d_idx, d_w, M, K, d_out, flags);
}

extern "C" int fm_moe_prefill_bf16_dev(fm_ctx *c, int layer, const uint16_t *d_X, const int32_t *d_idx,
                                       const float *d_w, int M, int K, float *d_out, int flags) {
    return moe_prefill_any(c, layer, d_X, true, d_idx, d_w, M, K, d_out, flags);
}

static int aff_prefill_fn(fm_ctx *c, int layer, const float *x, const int32_t *idx,
                          const float *w, int M, int K, float *out, float *, int flags) {
    return fm_moe_prefill_dev(c, layer, x, idx, w, M, K, out, flags);
}

extern "C" int fm_moe_prefill(fm_ctx *c, int layer, const float *X, const int32_t *idx,
                              const float *w, int M, int K, float *out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    return moe_host_call(c, aff_prefill_fn, c->geom.hidden, layer, X, idx, w, M, K, out, nullptr,
                         flags);
}

static int aff_prefill_bf16_fn(fm_ctx *c, int layer, const float *x, const int32_t *idx,
                               const float *w, int M, int K, float *out, float *, int flags) {
    return fm_moe_prefill_bf16_dev(c, layer, (const uint16_t *)x, idx, w, M, K, out, flags);
}

extern "C" int fm_moe_prefill_bf16(fm_ctx *c, int layer, const uint16_t *X, const int32_t *idx,
                                   const float *w, int M, int K, float *out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    return moe_host_call(c, aff_prefill_bf16_fn, c->geom.hidden, layer, X, idx, w, M, K, out, nullptr,
                         flags, 2);
}

// ============================================================================
// dense affine tensors
// ============================================================================
static int tensor_add(fm_ctx *c, const void *W, const void *S, const void *B, int out_dim,
                      int in_dim, int group_size, int bits, int scale_dtype, bool adopt,
                      fm_tensor *out) {
    if (!c) return FM_ERR_ARG;
    if (!W || !out) return fail(c, FM_ERR_ARG, "null pointer");
    if (out_dim < 1 || in_dim < 1) return fail(c, FM_ERR_ARG, "non-positive dimension");
    // scales == NULL or biases == NULL: an unquantized BF16 weight, as in cpu_dequant_matvec
    // (finchmoe/infer.m:1689); `bits` and `group_size` say nothing about it then
    // bits 10 / 11: a GGUF Q4_K / Q6_K tensor (block rows, no separate scales: S and B are ignored)
    const bool gguf = bits == FM_BITS_GGUF_Q4K || bits == FM_BITS_GGUF_Q6K;
    const bool raw = !gguf && (!S || !B);
    if (gguf && (in_dim < 256 || in_dim % 256 || in_dim > 16384))
        return fail(c, FM_ERR_UNSUPPORTED, "GGUF tensor in_dim %d: need a multiple of 256 up to 16384", in_dim);
    if (!raw && !gguf) {
        if (bits == 0) bits = 4;   // BatchMatvecSpec default, finchmoe/infer.m:4491
        if (group_size != 64) return fail(c, FM_ERR_UNSUPPORTED, "group_size %d (only 64)", group_size);
        if (bits != 1 && bits != 2 && bits != 3 && bits != 4 && bits != 8)
            return fail(c, FM_ERR_UNSUPPORTED, "tensor bits %d (1, 2, 3, 4 or 8)", bits);
        if (scale_dtype != FM_SCALE_BF16 && scale_dtype != FM_SCALE_FP16)
            return fail(c, FM_ERR_ARG, "scale_dtype %d", scale_dtype);
        int lpr = in_dim / 128;
        if (bits <= 2) {         // the legacy widths: a kernel of their own, any multiple of a group
            if (in_dim % 64 || in_dim > 16384)
                return fail(c, FM_ERR_UNSUPPORTED, "in_dim %d: need a multiple of 64 up to 16384", in_dim);
        } else if (in_dim % 128 || !pow2(lpr) || lpr > 64)
            return fail(c, FM_ERR_UNSUPPORTED, "in_dim %d: need 128*2^j, j<=6", in_dim);
    }
    DeviceGuard dg(c->device);
    Tensor t;
    t.used = true;
    t.out_dim = out_dim;
    t.in_dim = in_dim;
    t.group_size = group_size;
    t.bits = raw ? FM_BITS_RAW_BF16 : bits;
    t.scale_fp16 = !raw && !gguf && scale_dtype == FM_SCALE_FP16;
    const bool plain = raw || gguf;        // W only
    size_t wb = gguf ? (size_t)out_dim * gguf_row_bytes(in_dim, t.ggml_type()) : (size_t)out_dim * in_dim * t.bits / 8;
    size_t sb = (size_t)out_dim * (in_dim / 64) * 2;
    if (adopt) {
        if (((uintptr_t)W & (raw ? 1 : 15)) || (!plain && (((uintptr_t)S & 3) || ((uintptr_t)B & 3))))
            return fail(c, FM_ERR_ARG, "device tensor not aligned (W 16, S/B 4 bytes; raw BF16 2)");
        t.W = const_cast<void *>(W);
        t.S = plain ? nullptr : const_cast<void *>(S);
        t.B = plain ? nullptr : const_cast<void *>(B);
    } else {
        t.owned = true;
        HIPCHK(c, hipMalloc(&t.W, wb));
        HIPCHK(c, hipMemcpy(t.W, W, wb, hipMemcpyHostToDevice));
        if (!plain) {
            HIPCHK(c, hipMalloc(&t.S, sb));
            HIPCHK(c, hipMalloc(&t.B, sb));
            HIPCHK(c, hipMemcpy(t.S, S, sb, hipMemcpyHostToDevice));
            HIPCHK(c, hipMemcpy(t.B, B, sb, hipMemcpyHostToDevice));
        }
    }
    for (size_t i = 0; i < c->tensors.size(); i++)
        if (!c->tensors[i].used) {
            c->tensors[i] = t;
            *out = (fm_tensor)i;
            return FM_OK;
        }
    c->tensors.push_back(t);
    *out = (fm_tensor)(c->tensors.size() - 1);
    return FM_OK;
}

extern "C" int fm_tensor_register(fm_ctx *c, const void *W, const void *S, const void *B,
                                  int out_dim, int in_dim, int group_size, int bits,
                                  int scale_dtype, fm_tensor *out) {
    return tensor_add(c, W, S, B, out_dim, in_dim, group_size, bits, scale_dtype, false, out);
}
extern "C" int fm_tensor_adopt(fm_ctx *c, const void *W, const void *S, const void *B,
                               int out_dim, int in_dim, int group_size, int bits,
                               int scale_dtype, fm_tensor *out) {
    return tensor_add(c, W, S, B, out_dim, in_dim, group_size, bits, scale_dtype, true, out);
}

static Tensor *get_tensor(fm_ctx *c, fm_tensor t) {
    if (t < 0 || (size_t)t >= c->tensors.size() || !c->tensors[t].used) return nullptr;
    return &c->tensors[t];
}

extern "C" int fm_tensor_release(fm_ctx *c, fm_tensor t) {
    if (!c) return FM_ERR_ARG;
    Tensor *p = get_tensor(c, t);
    if (!p) return fail(c, FM_ERR_ARG, "bad tensor handle %d", t);
    DeviceGuard dg(c->device);
    HIPCHK(c, hipStreamSynchronize(c->stream));
    if (p->owned) {
        (void)hipFree(p->W);
        if (p->S) (void)hipFree(p->S);
        if (p->B) (void)hipFree(p->B);
    }
    *p = Tensor();
    return FM_OK;
}

static int matvec_dev(fm_ctx *c, const fm_tensor *ts, int n, const float *d_x,
                      float *const *d_outs, int M, const RouteArgs *route = nullptr,
                      bool *routed = nullptr) {
    if (!ts || !d_x || !d_outs) return fail(c, FM_ERR_ARG, "null pointer");
    if (n < 1) return fail(c, FM_ERR_ARG, "n %d", n);
    DeviceGuard dg(c->device);
    // One position, up to 8 small affine tensors of different code widths: one launch (each
    // tensor's rows are computed as its own launch would; two launches would pay the start-up
    // latency twice).  "Small": the whole batch is below the size from which a width's tensors
    // take the streaming kernel.
    if (M == 1 && n >= 2 && n <= 8) {
        FmDenseSpec specs[8];
        bool ok = true, mixed = false;
        long rows = 0;
        Tensor *t0 = get_tensor(c, ts[0]);
        for (int k = 0; ok && k < n; k++) {
            Tensor *t = get_tensor(c, ts[k]);
            ok = t && t0 && !t->raw_bf16() && !t->gguf() && t->in_dim == t0->in_dim && t->scale_fp16 == t0->scale_fp16 &&
                 t->group_size == 64 && d_outs[k] && (t->bits == 3 || t->bits == 4 || t->bits == 8);
            if (!ok) break;
            mixed = mixed || t->bits != t0->bits;
            rows += t->out_dim;
            specs[k].W = (const uint8_t *)t->W;
            specs[k].S = (const uint8_t *)t->S;
            specs[k].B = (const uint8_t *)t->B;
            specs[k].out = d_outs[k];
            specs[k].out_dim = t->out_dim;
            specs[k].first_item = 0;
            specs[k].bits = t->bits;
        }
        const int lpr = ok ? t0->in_dim / 128 : 0;
        if (ok && (mixed || route) && lpr >= 1 && lpr <= 64 && rows * lpr / 64 < 8L * c->n_cu) {
            unsigned int *ticket = route && c->d_tail ? (unsigned int *)(c->d_tail + FM_TAIL_PARTIALS) + 1 : nullptr;
            int rc = fm_launch_dense_mixed(specs, n, t0->in_dim, t0->scale_fp16, d_x, c->n_cu,
                                           ticket ? route : nullptr, ticket, c->stream);
            if (rc == FM_OK) {
                if (routed) *routed = ticket != nullptr;
                return FM_OK;
            }
            if (rc != FM_ERR_UNSUPPORTED)
                return fail(c, rc, "matvec launch failed: %s", hipGetErrorString(hipGetLastError()));
        }
    }
    // batches of up to 8 tensors with equal in_dim / bits / scale type
    int i = 0;
    while (i < n) {
        Tensor *t0 = get_tensor(c, ts[i]);
        if (!t0) return fail(c, FM_ERR_ARG, "bad tensor handle %d", ts[i]);
        if (t0->gguf()) {
            // a block-format tensor is a launch of its own (one per position)
            if (!d_outs[i]) return fail(c, FM_ERR_ARG, "null output %d", i);
            for (int pos = 0; pos < M; pos++) {
                int rc = fm_launch_gguf_dense((const uint8_t *)t0->W, t0->ggml_type(), d_x + (size_t)pos * t0->in_dim,
                                              d_outs[i] + (size_t)pos * t0->out_dim, t0->out_dim, t0->in_dim,
                                              c->n_cu, c->stream);
                if (rc) return fail(c, rc, "GGUF matvec launch failed: %s", hipGetErrorString(hipGetLastError()));
            }
            i++;
            continue;
        }
        FmDenseSpec specs[8];
        int m = 0;
        while (i < n && m < 8) {
            Tensor *t = get_tensor(c, ts[i]);
            if (!t) return fail(c, FM_ERR_ARG, "bad tensor handle %d", ts[i]);
            if (t->in_dim != t0->in_dim)
                return fail(c, FM_ERR_ARG, "tensors of one batch must share in_dim (%d vs %d)",
                            t->in_dim, t0->in_dim);
            if (t->bits != t0->bits || t->scale_fp16 != t0->scale_fp16) break;
            if (!d_outs[i]) return fail(c, FM_ERR_ARG, "null output %d", i);
            specs[m].W = (const uint8_t *)t->W;
            specs[m].S = (const uint8_t *)t->S;
            specs[m].B = (const uint8_t *)t->B;
            specs[m].out = d_outs[i];
            specs[m].out_dim = t->out_dim;
            specs[m].first_item = 0;
            specs[m].bits = t->bits;
            m++;
            i++;
        }
        // up to two raw-BF16 tensors right behind an affine group can ride along in its launch
        // (the b / a rows behind qkv / z, finchmoe/infer.m:8118-8122)
        FmDenseSpec riders[2];
        int n_riders = 0, riders_done = 0;
        if (!t0->raw_bf16() && t0->bits > 2) {
            for (int k = i; k < n && n_riders < 2; k++) {
                Tensor *t = get_tensor(c, ts[k]);
                if (!t || !t->raw_bf16() || t->in_dim != t0->in_dim || !d_outs[k]) break;
                riders[n_riders].W = (const uint8_t *)t->W;
                riders[n_riders].S = riders[n_riders].B = nullptr;
                riders[n_riders].out = d_outs[k];
                riders[n_riders].out_dim = t->out_dim;
                riders[n_riders].first_item = 0;
                riders[n_riders].bits = 16;
                n_riders++;
            }
        }
        int rc = t0->raw_bf16()
                     ? fm_launch_dense_bf16(specs, m, t0->in_dim, d_x, M, c->stream)
                 : t0->bits <= 2
                     ? fm_launch_dense_lowbit(specs, m, t0->in_dim, t0->bits, t0->scale_fp16, d_x, M, c->stream)
                     : fm_launch_dense(specs, m, t0->in_dim, t0->bits, t0->scale_fp16, d_x, M,
                                       c->n_cu, c->stream, n_riders ? riders : nullptr, n_riders,
                                       &riders_done);
        if (rc) return fail(c, rc, "matvec launch failed: %s", hipGetErrorString(hipGetLastError()));
        if (riders_done) i += n_riders;
    }
    return FM_OK;
}

extern "C" int fm_matvec_batch_dev(fm_ctx *c, const fm_tensor *ts, int n, const float *d_x,
                                   float *const *d_outs) {
    if (!c) return FM_ERR_ARG;
    return matvec_dev(c, ts, n, d_x, d_outs, 1);
}

static int ensure_tail_scratch(fm_ctx *c);

// fm_matvec_batch_dev followed by fm_route_topk_dev over tensor 0's outputs, as ONE launch when
// the batch is small enough for the plain kernel (the last workgroup to finish routes), else as
// the two launches: the results are the same either way.
extern "C" int fm_matvec_batch_route_dev(fm_ctx *c, const fm_tensor *ts, int n, const float *d_x,
                                         float *const *d_outs, int K, const float *d_seg_score,
                                         int32_t *d_idx, float *d_w, float *d_params) {
    if (!c) return FM_ERR_ARG;
    if (!ts || !d_outs || n < 1 || !d_idx || !d_w) return fail(c, FM_ERR_ARG, "null pointer");
    Tensor *t0 = get_tensor(c, ts[0]);
    if (!t0) return fail(c, FM_ERR_ARG, "bad tensor handle %d", ts[0]);
    const int n_experts = t0->out_dim;
    if (K < 1 || K > FM_MAX_K || K > n_experts)
        return fail(c, FM_ERR_ARG, "K %d outside 1..min(%d, n_experts)", K, FM_MAX_K);
    DeviceGuard dg(c->device);
    int rc = ensure_tail_scratch(c);
    if (rc) return rc;
    const RouteArgs ra{d_outs[0], n_experts, K, d_seg_score, d_idx, d_w, d_params};
    bool routed = false;
    rc = matvec_dev(c, ts, n, d_x, d_outs, 1, &ra, &routed);
    if (rc || routed) return rc;
    return fm_route_topk_dev(c, d_outs[0], n_experts, K, d_seg_score, d_idx, d_w, d_params);
}

extern "C" size_t fm_prefill_dense_ws_bytes(int out_dim, int in_dim, int group_size, int bits, int M);
extern "C" int fm_launch_prefill_dense(const void *d_W, const void *d_S, const void *d_B, int out_dim,
                                       int in_dim, int group_size, int bits, int scale_fp16,
                                       const float *d_X, int M, float *d_out, void *d_ws,
                                       size_t ws_bytes, int flags, int prepare, int n_cu,
                                       hipStream_t st);

// positions from which the dense product runs on the matrix cores (below: one GEMV per position)
#define FM_DENSE_GEMM_MIN_M 16

// n tensors against the same M positions.  Tensors the matrix-core kernel covers share one
// pass that turns X into operand registers (per code width); the others run one GEMV per position.
extern "C" int fm_matvec_prefill_batch_dev(fm_ctx *c, const fm_tensor *ts, int n, const float *d_X,
                                           float *const *d_outs, int M) {
    if (!c) return FM_ERR_ARG;
    if (!ts || !d_X || !d_outs) return fail(c, FM_ERR_ARG, "null pointer");
    if (n < 1 || n > 64) return fail(c, FM_ERR_ARG, "n %d outside 1..64", n);
    if (M < 1 || M > 65535) return fail(c, FM_ERR_ARG, "M %d outside 1..65535", M);
    const bool no_gemm = (fm_kernel_forms & FM_FORM_NO_DENSE_GEMM) != 0;
    int prepared_bits = 0, prepared_in = 0;
    for (int i = 0; i < n; i++) {   // one X for all: the tensors must agree on its width
        Tensor *p = get_tensor(c, ts[i]), *p0 = get_tensor(c, ts[0]);
        if (!p) return fail(c, FM_ERR_ARG, "bad tensor handle %d", ts[i]);
        if (p->in_dim != p0->in_dim)
            return fail(c, FM_ERR_ARG, "tensors of one batch must share in_dim (%d vs %d)", p->in_dim,
                        p0->in_dim);
    }
    for (int i = 0; i < n; i++) {
        Tensor *p = get_tensor(c, ts[i]);
        if (!d_outs[i]) return fail(c, FM_ERR_ARG, "null output %d", i);
        size_t ws = 0;
        if (!no_gemm && !p->raw_bf16() && !p->gguf() && M >= FM_DENSE_GEMM_MIN_M && ((uintptr_t)d_X & 15) == 0 && ((uintptr_t)d_outs[i] & 3) == 0)
            ws = fm_prefill_dense_ws_bytes(p->out_dim, p->in_dim, p->group_size, p->bits, M);
        if (ws) {
            DeviceGuard dg(c->device);
            // (growing the workspace drops what was prepared in it)
            if (c->ws_bytes < ws) prepared_bits = 0;
            int rc = ensure_ws(c, ws);
            if (rc) return rc;
            const int prepare = !(prepared_bits == p->bits && prepared_in == p->in_dim);
            rc = fm_launch_prefill_dense(p->W, p->S, p->B, p->out_dim, p->in_dim, p->group_size,
                                         p->bits, p->scale_fp16, d_X, M, d_outs[i], c->d_ws, c->ws_bytes,
                                         0, prepare, c->n_cu, c->stream);
            if (rc == FM_OK) {
                prepared_bits = p->bits;
                prepared_in = p->in_dim;
                continue;
            }
            if (rc != FM_ERR_UNSUPPORTED)
                return fail(c, rc, "dense prefill launch failed: %s", hipGetErrorString(hipGetLastError()));
        }
        float *outs[1] = {d_outs[i]};
        int rc = matvec_dev(c, &ts[i], 1, d_X, outs, M);
        if (rc) return rc;
    }
    return FM_OK;
}

extern "C" int fm_matvec_prefill_dev(fm_ctx *c, fm_tensor t, const float *d_X, float *d_out,
                                     int M) {
    float *outs[1] = {d_out};
    return fm_matvec_prefill_batch_dev(c, &t, 1, d_X, outs, M);
}

static int matvec_host(fm_ctx *c, const fm_tensor *ts, int n, const float *x, float *const *outs,
                       int M) {
    if (!ts || !x || !outs) return fail(c, FM_ERR_ARG, "null pointer");
    if (n < 1 || n > 64) return fail(c, FM_ERR_ARG, "n %d outside 1..64", n);
    Tensor *t0 = get_tensor(c, ts[0]);
    if (!t0) return fail(c, FM_ERR_ARG, "bad tensor handle %d", ts[0]);
    DeviceGuard dg(c->device);
    size_t nx = (size_t)M * t0->in_dim * 4, total = nx;
    std::vector<size_t> offs(n);
    for (int i = 0; i < n; i++) {
        Tensor *t = get_tensor(c, ts[i]);
        if (!t) return fail(c, FM_ERR_ARG, "bad tensor handle %d", ts[i]);
        if (!outs[i]) return fail(c, FM_ERR_ARG, "null output %d", i);
        if (t->in_dim != t0->in_dim)   // the staging area holds one X of t0's width
            return fail(c, FM_ERR_ARG, "tensors of one batch must share in_dim (%d vs %d)", t->in_dim,
                        t0->in_dim);
        offs[i] = total;
        total += ((size_t)M * t->out_dim * 4 + 255) & ~(size_t)255;
    }
    int rc = ensure_stage(c, total);
    if (rc) return rc;
    char *st = (char *)c->d_stage;
    HIPCHK(c, hipMemcpyAsync(st, x, nx, hipMemcpyHostToDevice, c->stream));
    std::vector<float *> d_outs(n);
    for (int i = 0; i < n; i++) d_outs[i] = (float *)(st + offs[i]);
    // (M positions: the same path as the device-pointer entry, matrix cores from 16 positions on)
    rc = M > 1 ? fm_matvec_prefill_batch_dev(c, ts, n, (const float *)st, d_outs.data(), M)
               : matvec_dev(c, ts, n, (const float *)st, d_outs.data(), M);
    if (rc) return rc;
    for (int i = 0; i < n; i++)
        HIPCHK(c, hipMemcpyAsync(outs[i], d_outs[i], (size_t)M * get_tensor(c, ts[i])->out_dim * 4,
                                 hipMemcpyDeviceToHost, c->stream));
    HIPCHK(c, hipStreamSynchronize(c->stream));
    return FM_OK;
}

extern "C" int fm_matvec_batch(fm_ctx *c, const fm_tensor *ts, int n, const float *x,
                               float *const *outs) {
    if (!c) return FM_ERR_ARG;
    return matvec_host(c, ts, n, x, outs, 1);
}

extern "C" int fm_matvec_prefill(fm_ctx *c, fm_tensor t, const float *X, float *out, int M) {
    if (!c) return FM_ERR_ARG;
    if (M < 1 || M > 65535) return fail(c, FM_ERR_ARG, "M %d outside 1..65535", M);
    float *outs[1] = {out};
    return matvec_host(c, &t, 1, X, outs, M);
}

// ============================================================================
// routing
// ============================================================================
extern "C" int fm_route_topk_dev(fm_ctx *c, const float *d_logits, int n_experts, int K,
                                 const float *d_seg_score, int32_t *d_idx, float *d_w,
                                 float *d_params) {
    if (!c) return FM_ERR_ARG;
    if (!d_logits || !d_idx || !d_w) return fail(c, FM_ERR_ARG, "null pointer");
    if (K < 1 || K > FM_MAX_K || K > n_experts)
        return fail(c, FM_ERR_ARG, "K %d outside 1..min(%d, n_experts)", K, FM_MAX_K);
    DeviceGuard dg(c->device);
    int rc = fm_launch_route(d_logits, n_experts, K, d_seg_score, d_idx, d_w, d_params, c->stream);
    if (rc) return fail(c, rc, "routing over %d experts has no kernel (1..4096)", n_experts);
    return FM_OK;
}

// ============================================================================
// layer tail
// ============================================================================

// partial sums of the norm + the ticket words of the tail and of the fused routing
static int ensure_tail_scratch(fm_ctx *c) {
    if (c->d_tail) return FM_OK;
    if (note_capture(c)) return refuse_growth(c, "the layer tail's scratch");
    // partial sums | ticket words | one vector of up to FM_TAIL_VECTOR floats (the experts' sum
    // between the two launches of fm_moe_decode_tail_dev when it runs as two)
    HIPCHK(c, hipMalloc((void **)&c->d_tail, (FM_TAIL_PARTIALS + 64 + FM_TAIL_VECTOR) * sizeof(float)));
    HIPCHK(c, hipMemsetAsync(c->d_tail, 0, (FM_TAIL_PARTIALS + 64) * sizeof(float), c->stream));
    return FM_OK;
}

extern "C" int fm_layer_tail_dev(fm_ctx *c, fm_tensor shared_down, const float *d_h_mid,
                                 const float *d_expert_out, const float *d_params, int K,
                                 const float *d_shared_gate, const float *d_shared_up,
                                 const uint16_t *d_next_norm_w, float eps, float *d_hidden_out,
                                 float *d_next_input) {
    if (!c) return FM_ERR_ARG;
    Tensor *t = get_tensor(c, shared_down);
    if (!t) return fail(c, FM_ERR_ARG, "bad tensor handle %d", shared_down);
    if (!d_h_mid || !d_params || !d_shared_gate || !d_shared_up || !d_hidden_out ||
        (K > 0 && !d_expert_out))
        return fail(c, FM_ERR_ARG, "null pointer");
    if (K < 0 || K > FM_MAX_K) return fail(c, FM_ERR_ARG, "K %d outside 0..%d", K, FM_MAX_K);
    if ((d_next_input != nullptr) != (d_next_norm_w != nullptr))
        return fail(c, FM_ERR_ARG, "next input and its norm weights go together");
    if (((uintptr_t)d_shared_gate | (uintptr_t)d_shared_up) & 3)
        return fail(c, FM_ERR_ARG, "vector not 4-byte aligned");
    if (t->raw_bf16() || t->gguf() || t->bits <= 2 || t->group_size != 64)
        return fail(c, FM_ERR_UNSUPPORTED, "shared down projection must be 3/4/8-bit, group size 64");
    if (t->out_dim / 4 > FM_TAIL_PARTIALS) return fail(c, FM_ERR_UNSUPPORTED, "hidden %d", t->out_dim);
    DeviceGuard dg(c->device);
    int rc0 = ensure_tail_scratch(c);
    if (rc0) return rc0;
    FmTailArgs a;
    a.W = (const uint8_t *)t->W;
    a.S = (const uint8_t *)t->S;
    a.B = (const uint8_t *)t->B;
    a.hidden = t->out_dim;
    a.inter = t->in_dim;
    a.K = K;
    a.h_mid = d_h_mid;
    a.expert_out = d_expert_out;
    a.params = d_params;
    a.shared_gate = d_shared_gate;
    a.shared_up = d_shared_up;
    a.norm_w = d_next_norm_w;
    a.eps = eps;
    a.hidden_out = d_hidden_out;
    a.next_in = d_next_input;
    a.partial = c->d_tail;
    a.counter = (unsigned int *)(c->d_tail + FM_TAIL_PARTIALS);
    int rc = fm_launch_layer_tail(&a, t->bits, t->scale_fp16, c->stream);
    if (rc) return fail(c, rc, "layer tail: shape [%d, %d] at %d bits has no kernel", t->out_dim,
                        t->in_dim, t->bits);
    return FM_OK;
}

// One layer's routed experts and the layer's tail in one launch: fm_moe_decode_dev (without the
// per-expert vectors) followed by fm_layer_tail_dev in its K = 0 form, bit for bit.  Shapes the
// one-launch kernel does not cover (and calls under stream capture) run as those two launches.
// route: the token's routing (fm_route_topk_dev) at the start of the same launch, over logits
// that an earlier launch left in memory; d_idx / d_w / d_params are then outputs.
static int decode_tail(fm_ctx *c, int layer, const float *d_x, const int32_t *d_idx, const float *d_w, int K,
                       fm_tensor shared_down, const float *d_h_mid, const float *d_params,
                       const float *d_shared_gate, const float *d_shared_up, const uint16_t *d_next_norm_w,
                       float eps, float *d_hidden_out, float *d_next_input, const RouteArgs *route) {
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    Tensor *t = get_tensor(c, shared_down);
    if (!t) return fail(c, FM_ERR_ARG, "bad tensor handle %d", shared_down);
    if (!d_x || !d_idx || !d_w || !d_h_mid || !d_params || !d_shared_gate || !d_shared_up || !d_hidden_out)
        return fail(c, FM_ERR_ARG, "null pointer");
    if (K < 1 || K > FM_MAX_K) return fail(c, FM_ERR_ARG, "K %d outside 1..%d", K, FM_MAX_K);
    if ((d_next_input != nullptr) != (d_next_norm_w != nullptr))
        return fail(c, FM_ERR_ARG, "next input and its norm weights go together");
    if (((uintptr_t)d_shared_gate | (uintptr_t)d_shared_up) & 3)
        return fail(c, FM_ERR_ARG, "vector not 4-byte aligned");
    int rc = check_layers(c, c->layers, layer, 1);
    if (rc) return rc;
    DeviceGuard dg(c->device);
    rc = ensure_scratch(c, 1, c->geom.hidden, c->geom.inter);
    if (rc) return rc;
    rc = ensure_tail_scratch(c);
    if (rc) return rc;
    const bool one_launch = !c->split_phases && !c->ktiming && t->bits == 4 && !t->raw_bf16() && !t->gguf() &&
                            t->group_size == 64 && t->out_dim == c->geom.hidden && t->in_dim == c->geom.inter;
    if (one_launch) {
        FmTailArgs a{};
        a.W = (const uint8_t *)t->W;
        a.S = (const uint8_t *)t->S;
        a.B = (const uint8_t *)t->B;
        a.hidden = t->out_dim;
        a.inter = t->in_dim;
        a.K = 0;
        a.h_mid = d_h_mid;
        a.expert_out = nullptr;
        a.params = d_params;
        a.shared_gate = d_shared_gate;
        a.shared_up = d_shared_up;
        a.norm_w = d_next_norm_w;
        a.eps = eps;
        a.hidden_out = d_hidden_out;
        a.next_in = d_next_input;
        a.partial = c->d_tail;
        a.counter = (unsigned int *)(c->d_tail + FM_TAIL_PARTIALS);
        a.scale_fp16 = t->scale_fp16;
        if (route) {
            a.route_logits = route->logits;
            a.route_n = route->n;
            a.route_seg = route->seg_score;
            a.route_idx = route->idx;
            a.route_w = route->w;
            a.route_params = route->params;
        }
        rc = fm_launch_decode_affine(c->d_layer_ptrs, &c->geom, layer, 1, 1, d_x, d_idx, d_w, K, c->d_act, c->d_eo,
                                     d_hidden_out, &c->dflags, FM_INT_NO_EXPERT_OUT, c->n_cu, c->stream, nullptr, &a);
        if (rc == FM_OK) {
            c->sync_unchecked = true;
            return FM_OK;
        }
        if (rc != FM_ERR_UNSUPPORTED)
            return fail(c, rc, "decode + tail launch failed: %s", hipGetErrorString(hipGetLastError()));
    }
    // separate launches: the routing if it was asked for, the experts (their sum crosses in a
    // vector of the tail's scratch), the tail
    if (route) {
        rc = fm_route_topk_dev(c, route->logits, route->n, K, route->seg_score, route->idx, route->w, route->params);
        if (rc) return rc;
    }
    if (c->geom.hidden > FM_TAIL_VECTOR) return fail(c, FM_ERR_UNSUPPORTED, "hidden %d", c->geom.hidden);
    float *d_sum = c->d_tail + FM_TAIL_PARTIALS + 64;
    rc = fm_moe_decode_step_dev(c, layer, 1, d_x, d_idx, d_w, K, d_sum, nullptr, 0);
    if (rc) return rc;
    return fm_layer_tail_dev(c, shared_down, d_h_mid, d_sum, d_params, 0, d_shared_gate, d_shared_up,
                             d_next_norm_w, eps, d_hidden_out, d_next_input);
}

extern "C" int fm_moe_decode_tail_dev(fm_ctx *c, int layer, const float *d_x, const int32_t *d_idx,
                                      const float *d_w, int K, fm_tensor shared_down, const float *d_h_mid,
                                      const float *d_params, const float *d_shared_gate,
                                      const float *d_shared_up, const uint16_t *d_next_norm_w, float eps,
                                      float *d_hidden_out, float *d_next_input) {
    if (!c) return FM_ERR_ARG;
    return decode_tail(c, layer, d_x, d_idx, d_w, K, shared_down, d_h_mid, d_params, d_shared_gate, d_shared_up,
                       d_next_norm_w, eps, d_hidden_out, d_next_input, nullptr);
}

// The MoE half of a layer in two launches: the routing batch (gate logits, the shared expert's
// gate score and gate / up projections: fm_matvec_batch_dev over route_tensors[0..3], all from
// d_x), then the routing, the routed experts and the tail in one.  Identical to
// fm_matvec_batch_route_dev + fm_moe_decode_dev + fm_layer_tail_dev.
extern "C" int fm_moe_layer_dev(fm_ctx *c, int layer, const fm_tensor *route_tensors, const float *d_x, int K,
                                fm_tensor shared_down, const float *d_h_mid, const uint16_t *d_next_norm_w,
                                float eps, float *d_logits, float *d_seg_score, float *d_shared_gate,
                                float *d_shared_up, int32_t *d_idx, float *d_w, float *d_params,
                                float *d_hidden_out, float *d_next_input) {
    if (!c) return FM_ERR_ARG;
    if (!route_tensors || !d_logits || !d_seg_score || !d_shared_gate || !d_shared_up || !d_idx || !d_w || !d_params)
        return fail(c, FM_ERR_ARG, "null pointer");
    Tensor *t0 = get_tensor(c, route_tensors[0]);
    if (!t0) return fail(c, FM_ERR_ARG, "bad tensor handle %d", route_tensors[0]);
    const int n_experts = t0->out_dim;
    if (K < 1 || K > FM_MAX_K || K > n_experts)
        return fail(c, FM_ERR_ARG, "K %d outside 1..min(%d, n_experts)", K, FM_MAX_K);
    float *outs[4] = {d_logits, d_seg_score, d_shared_gate, d_shared_up};
    int rc = matvec_dev(c, route_tensors, 4, d_x, outs, 1);
    if (rc) return rc;
    const RouteArgs ra{d_logits, n_experts, K, d_seg_score, d_idx, d_w, d_params};
    return decode_tail(c, layer, d_x, d_idx, d_w, K, shared_down, d_h_mid, d_params, d_shared_gate, d_shared_up,
                       d_next_norm_w, eps, d_hidden_out, d_next_input, &ra);
}

// ============================================================================
// GGUF expert store
// ============================================================================
extern "C" int fm_gguf_config(fm_ctx *c, int n_layers, int n_experts, int hidden, int inter,
                              int gate_type, int up_type, int down_type) {
    if (!c) return FM_ERR_ARG;
    if (n_layers < 1 || n_experts < 1) return fail(c, FM_ERR_ARG, "non-positive dimension");
    // finchmoe/infer.m:3166: the fused gate+up kernel is Q4_K only
    if (gate_type != FM_GGML_Q4_K || up_type != FM_GGML_Q4_K)
        return fail(c, FM_ERR_UNSUPPORTED, "gate/up must be Q4_K (12), got %d/%d", gate_type, up_type);
    if (down_type != FM_GGML_Q4_K && down_type != FM_GGML_Q6_K)
        return fail(c, FM_ERR_UNSUPPORTED, "down must be Q4_K (12) or Q6_K (14), got %d", down_type);
    if (hidden % 256 || inter % 256 || hidden < 256 || inter < 256 || hidden > 16384 || inter > 16384)
        return fail(c, FM_ERR_UNSUPPORTED, "hidden %d / inter %d: need multiples of 256", hidden, inter);
    DeviceGuard dg(c->device);
    HIPCHK(c, hipStreamSynchronize(c->stream));
    free_layers(c->g_gate);
    free_layers(c->g_up);
    free_layers(c->g_down);
    if (c->d_gg_ptrs) HIPCHK(c, hipFree(c->d_gg_ptrs));
    c->d_gg_ptrs = nullptr;
    c->gguf_cfg = false;
    FmGgufGeom &g = c->ggeom;
    g.hidden = hidden;
    g.inter = inter;
    g.n_experts = n_experts;
    g.gate_type = gate_type;
    g.up_type = up_type;
    g.down_type = down_type;
    g.gu_row_bytes = (uint32_t)gguf_row_bytes(hidden, gate_type);
    g.down_row_bytes = (uint32_t)gguf_row_bytes(inter, down_type);
    // finchmoe/infer.m:1141-1146: slab = out rows x row bytes
    g.gate_slab = (uint64_t)inter * g.gu_row_bytes;
    g.up_slab = g.gate_slab;
    g.down_slab = (uint64_t)hidden * g.down_row_bytes;
    c->g_layers = n_layers;
    c->g_gate.assign(n_layers, LayerBuf());
    c->g_up.assign(n_layers, LayerBuf());
    c->g_down.assign(n_layers, LayerBuf());
    HIPCHK(c, hipMalloc((void **)&c->d_gg_ptrs, (size_t)3 * n_layers * sizeof(uint8_t *)));
    HIPCHK(c, hipMemset(c->d_gg_ptrs, 0, (size_t)3 * n_layers * sizeof(uint8_t *)));
    c->gguf_cfg = true;
    return FM_OK;
}

static int gguf_set_layer(fm_ctx *c, int layer, const void *gate, size_t gate_bytes,
                          const void *up, size_t up_bytes, const void *down, size_t down_bytes,
                          bool adopt) {
    if (!c) return FM_ERR_ARG;
    if (!c->gguf_cfg) return fail(c, FM_ERR_STATE, "GGUF store not configured");
    if (!gate || !up || !down || layer < 0 || layer >= c->g_layers)
        return fail(c, FM_ERR_ARG, "layer %d", layer);
    if (adopt && (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)down) & 15))
        return fail(c, FM_ERR_ARG, "device slab not 16-byte aligned");
    const FmGgufGeom &g = c->ggeom;
    const size_t want[3] = {(size_t)g.n_experts * g.gate_slab, (size_t)g.n_experts * g.up_slab,
                            (size_t)g.n_experts * g.down_slab};
    const size_t have[3] = {gate_bytes, up_bytes, down_bytes};
    for (int i = 0; i < 3; i++)
        if (have[i] != want[i])
            return fail(c, FM_ERR_ARG, "GGUF %s tensor is %zu bytes, expected %zu",
                        i == 0 ? "gate" : i == 1 ? "up" : "down", have[i], want[i]);
    DeviceGuard dg(c->device);
    HIPCHK(c, hipStreamSynchronize(c->stream));
    if (!adopt) {
        // all three copies land in fresh buffers before the layer's pointers change
        const void *src[3] = {gate, up, down};
        void *fresh[3] = {nullptr, nullptr, nullptr};
        hipError_t e = hipSuccess;
        for (int i = 0; i < 3 && e == hipSuccess; i++) {
            e = hipMalloc(&fresh[i], want[i]);
            if (e == hipSuccess) e = hipMemcpy(fresh[i], src[i], want[i], hipMemcpyHostToDevice);
        }
        if (e != hipSuccess) {
            for (void *f : fresh)
                if (f) (void)hipFree(f);
            return fail(c, FM_ERR_HIP, "GGUF layer upload: %s", hipGetErrorString(e));
        }
        std::vector<LayerBuf> *dst[3] = {&c->g_gate, &c->g_up, &c->g_down};
        for (int i = 0; i < 3; i++) {
            LayerBuf &lb = (*dst[i])[layer];
            if (lb.owned && lb.ptr) (void)hipFree(lb.ptr);
            lb.ptr = fresh[i];
            lb.owned = true;
        }
    } else {
        int rc = set_layer(c, c->g_gate, layer, gate, want[0], true);
        if (!rc) rc = set_layer(c, c->g_up, layer, up, want[1], true);
        if (!rc) rc = set_layer(c, c->g_down, layer, down, want[2], true);
        if (rc) return rc;
    }
    void *p[3] = {c->g_gate[layer].ptr, c->g_up[layer].ptr, c->g_down[layer].ptr};
    for (int i = 0; i < 3; i++)
        HIPCHK(c, hipMemcpy(c->d_gg_ptrs + (size_t)i * c->g_layers + layer, &p[i], sizeof(void *),
                            hipMemcpyHostToDevice));
    return FM_OK;
}

extern "C" int fm_gguf_upload_layer(fm_ctx *c, int layer, const void *gate, size_t gate_bytes,
                                    const void *up, size_t up_bytes, const void *down,
                                    size_t down_bytes) {
    return gguf_set_layer(c, layer, gate, gate_bytes, up, up_bytes, down, down_bytes, false);
}
extern "C" int fm_gguf_adopt_layer(fm_ctx *c, int layer, const void *gate, size_t gate_bytes,
                                   const void *up, size_t up_bytes, const void *down,
                                   size_t down_bytes) {
    return gguf_set_layer(c, layer, gate, gate_bytes, up, up_bytes, down, down_bytes, true);
}

static int gguf_decode_groups(fm_ctx *c, int layer0, int layer_stride, int groups,
                              const float *d_x, const int32_t *d_idx, const float *d_w, int K,
                              float *d_out, float *d_expert_out, int flags) {
    if (!c->gguf_cfg) return fail(c, FM_ERR_STATE, "GGUF store not configured");
    if (!d_x || !d_idx || !d_w || !d_out) return fail(c, FM_ERR_ARG, "null pointer");
    if (K < 1 || K > FM_MAX_K) return fail(c, FM_ERR_ARG, "K %d outside 1..%d", K, FM_MAX_K);
    int rc = check_layers(c, c->g_gate, layer0, layer_stride ? groups : 1);
    if (rc) return rc;
    DeviceGuard dg(c->device);
    rc = ensure_scratch(c, groups, c->ggeom.hidden, c->ggeom.inter);
    if (rc) return rc;
    rc = fm_launch_decode_gguf(c->d_gg_ptrs, c->d_gg_ptrs + c->g_layers,
                               c->d_gg_ptrs + 2 * (size_t)c->g_layers, &c->ggeom, layer0,
                               layer_stride, groups, d_x, d_idx, d_w, K, c->d_act,
                               d_expert_out ? d_expert_out : c->d_eo, d_out,
                               c->split_phases ? nullptr : &c->dflags,
                               flags | (d_expert_out ? 0 : FM_INT_NO_EXPERT_OUT),
                               c->n_cu, c->stream, c->ktiming ? c->kev : nullptr);
    if (rc) return fail(c, rc, "GGUF decode launch failed: %s", hipGetErrorString(hipGetLastError()));
    if (!c->split_phases) c->sync_unchecked = true;     // (the one-launch form may have run: its waits are bounded)
    if (c->ktiming) return ktiming_collect(c);
    return FM_OK;
}

extern "C" int fm_gguf_moe_decode_step_dev(fm_ctx *c, int layer0, int n_layers, const float *d_x,
                                           const int32_t *d_idx, const float *d_w, int K,
                                           float *d_out, float *d_expert_out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (n_layers < 1) return fail(c, FM_ERR_ARG, "n_layers %d", n_layers);
    return gguf_decode_groups(c, layer0, 1, n_layers, d_x, d_idx, d_w, K, d_out, d_expert_out, flags);
}

extern "C" int fm_gguf_moe_decode_dev(fm_ctx *c, int layer, const float *d_x, const int32_t *d_idx,
                                      const float *d_w, int K, float *d_out, float *d_expert_out,
                                      int flags) {
    if (!c) return FM_ERR_ARG;
    return gguf_decode_groups(c, layer, 1, 1, d_x, d_idx, d_w, K, d_out, d_expert_out, flags);
}

extern "C" size_t fm_prefill_gguf_ws_bytes(const FmGgufGeom *g, int M, int K);
extern "C" int fm_launch_prefill_gguf(const uint8_t *d_gate, const uint8_t *d_up, const uint8_t *d_down,
                                      const FmGgufGeom *g, const float *d_X, const int32_t *d_idx,
                                      const float *d_w, int M, int K, float *d_out, void *d_ws,
                                      size_t ws_bytes, int flags, int n_cu, hipStream_t st);

// Chunks of FM_PREFILL_GEMM_MIN_M positions and more with at least two (position, slot) pairs
// per expert take the grouped products (every routed
// expert streamed once per group of its positions; prefill_chunk_cmd3_batch_general,
// finchmoe/infer.m:10958-11059, streams it once per position) when the store is Q4_K gate/up
// with Q6_K down; smaller chunks, other type combinations and the finite guard run the decode
// kernels position by position.
extern "C" int fm_gguf_moe_prefill_dev(fm_ctx *c, int layer, const float *d_X, const int32_t *d_idx,
                                       const float *d_w, int M, int K, float *d_out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (M < 1 || M > FM_MAX_CHUNK) return fail(c, FM_ERR_ARG, "M %d outside 1..%d", M, FM_MAX_CHUNK);
    const bool no_group = (fm_kernel_forms & FM_FORM_NO_GGUF_GROUP) != 0;
    // (grouping pays from two (position, slot) pairs per expert on: measured at 256 experts, chunks of
    // 64 / 96 / 128 / 512 positions take 134 / 150 / 172 / 295 us grouped and 152 / 242 / 281 / 1050 us
    // position by position; at 32 positions, one pair per expert, both stream every expert once)
    if (c->gguf_cfg && M >= FM_PREFILL_GEMM_MIN_M && !(flags & FM_GUARD) && !no_group && d_X && d_idx &&
        d_w && d_out && K >= 1 && K <= FM_MAX_K && (long)M * K >= 2L * c->ggeom.n_experts) {
        const size_t ws = fm_prefill_gguf_ws_bytes(&c->ggeom, M, K);
        if (ws) {
            int rc = check_layers(c, c->g_gate, layer, 1);
            if (rc) return rc;
            DeviceGuard dg(c->device);
            if ((rc = ensure_ws(c, ws))) return rc;
            rc = fm_launch_prefill_gguf((const uint8_t *)c->g_gate[layer].ptr, (const uint8_t *)c->g_up[layer].ptr,
                                        (const uint8_t *)c->g_down[layer].ptr, &c->ggeom, d_X, d_idx, d_w, M,
                                        K, d_out, c->d_ws, c->ws_bytes, flags, c->n_cu, c->stream);
            if (rc == FM_OK) return FM_OK;
            if (rc != FM_ERR_UNSUPPORTED)
                return fail(c, rc, "GGUF prefill launch failed: %s", hipGetErrorString(hipGetLastError()));
        }
    }
    return gguf_decode_groups(c, layer, 0, M, d_X, d_idx, d_w, K, d_out, nullptr, flags);
}

static int gguf_decode_fn(fm_ctx *c, int layer, const float *x, const int32_t *idx, const float *w,
                          int, int K, float *out, float *eo, int flags) {
    return gguf_decode_groups(c, layer, 1, 1, x, idx, w, K, out, eo, flags);
}
static int gguf_prefill_fn(fm_ctx *c, int layer, const float *x, const int32_t *idx,
                           const float *w, int M, int K, float *out, float *, int flags) {
    return fm_gguf_moe_prefill_dev(c, layer, x, idx, w, M, K, out, flags);
}

extern "C" int fm_gguf_moe_decode(fm_ctx *c, int layer, const float *x, const int32_t *idx,
                                  const float *w, int K, float *out, float *expert_out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (!c->gguf_cfg) return fail(c, FM_ERR_STATE, "GGUF store not configured");
    return moe_host_call(c, gguf_decode_fn, c->ggeom.hidden, layer, x, idx, w, 1, K, out,
                         expert_out, flags);
}

extern "C" int fm_gguf_moe_prefill(fm_ctx *c, int layer, const float *X, const int32_t *idx,
                                   const float *w, int M, int K, float *out, int flags) {
    if (!c) return FM_ERR_ARG;
    if (!c->gguf_cfg) return fail(c, FM_ERR_STATE, "GGUF store not configured");
    return moe_host_call(c, gguf_prefill_fn, c->ggeom.hidden, layer, X, idx, w, M, K, out, nullptr,
                         flags);
}

extern "C" int fm_gguf_matvec(fm_ctx *c, const void *W, int ggml_type, const float *x, float *out,
                              int out_dim, int in_dim) {
    if (!c) return FM_ERR_ARG;
    if (!W || !x || !out) return fail(c, FM_ERR_ARG, "null pointer");
    if (ggml_type != FM_GGML_Q4_K && ggml_type != FM_GGML_Q6_K)
        return fail(c, FM_ERR_UNSUPPORTED, "ggml type %d", ggml_type);
    if (out_dim < 1 || in_dim < 256 || in_dim % 256 || in_dim > 16384)
        return fail(c, FM_ERR_UNSUPPORTED, "in_dim %d: need a multiple of 256 up to 16384", in_dim);
    DeviceGuard dg(c->device);
    size_t wb = (size_t)out_dim * gguf_row_bytes(in_dim, ggml_type);
    size_t off_x = (wb + 255) & ~(size_t)255, off_o = off_x + (((size_t)in_dim * 4 + 255) & ~(size_t)255);
    int rc = ensure_stage(c, off_o + (size_t)out_dim * 4);
    if (rc) return rc;
    char *st = (char *)c->d_stage;
    HIPCHK(c, hipMemcpyAsync(st, W, wb, hipMemcpyHostToDevice, c->stream));
    HIPCHK(c, hipMemcpyAsync(st + off_x, x, (size_t)in_dim * 4, hipMemcpyHostToDevice, c->stream));
    rc = fm_launch_gguf_matvec((const uint8_t *)st, ggml_type, (const float *)(st + off_x),
                               (float *)(st + off_o), out_dim, in_dim, c->n_cu, c->stream);
    if (rc) return fail(c, rc, "GGUF matvec launch failed");
    HIPCHK(c, hipMemcpyAsync(out, st + off_o, (size_t)out_dim * 4, hipMemcpyDeviceToHost, c->stream));
    HIPCHK(c, hipStreamSynchronize(c->stream));
    return FM_OK;
}

// ============================================================================
// dequant (bit-exact checks)
// ============================================================================
static int dequant_common(fm_ctx *c, const void *dW, const void *dS, const void *dB, int rows,
                          int cols, int bits, int scale_fp16, int ggml_type, uint8_t *codes,
                          float *w_f32, uint16_t *w_f16) {
    size_t n = (size_t)rows * cols;
    size_t off32 = (n + 255) & ~(size_t)255, off16 = off32 + n * 4;
    int rc = ensure_stage(c, off16 + n * 2);
    if (rc) return rc;
    char *st = (char *)c->d_stage;
    if (ggml_type) {
        rc = fm_launch_dequant_gguf(dW, rows, cols, ggml_type, (float *)(st + off32), c->stream);
    } else {
        rc = fm_launch_dequant_affine(dW, dS, dB, rows, cols, 64, bits, scale_fp16,
                                      (uint8_t *)st, (float *)(st + off32),
                                      (uint16_t *)(st + off16), c->stream);
    }
    if (rc) return fail(c, rc, "dequant launch failed");
    if (codes) HIPCHK(c, hipMemcpyAsync(codes, st, n, hipMemcpyDeviceToHost, c->stream));
    if (w_f32) HIPCHK(c, hipMemcpyAsync(w_f32, st + off32, n * 4, hipMemcpyDeviceToHost, c->stream));
    if (w_f16) HIPCHK(c, hipMemcpyAsync(w_f16, st + off16, n * 2, hipMemcpyDeviceToHost, c->stream));
    HIPCHK(c, hipStreamSynchronize(c->stream));
    return FM_OK;
}

extern "C" int fm_dequant_expert(fm_ctx *c, int layer, int expert, int which, uint8_t *codes,
                                 float *w_f32, uint16_t *w_f16) {
    if (!c) return FM_ERR_ARG;
    if (!c->aff_cfg) return fail(c, FM_ERR_STATE, "experts store not configured");
    int rc = check_layers(c, c->layers, layer, 1);
    if (rc) return rc;
    const FmExpertGeom &g = c->geom;
    if (expert < 0 || expert >= g.n_experts) return fail(c, FM_ERR_ARG, "expert %d", expert);
    if (which < FM_MAT_GATE || which > FM_MAT_DOWN) return fail(c, FM_ERR_ARG, "which %d", which);
    DeviceGuard dg(c->device);
    const uint8_t *e = (const uint8_t *)c->layers[layer].ptr + (size_t)expert * g.expert_size;
    uint32_t wo[3] = {g.gate_w, g.up_w, g.down_w}, so[3] = {g.gate_s, g.up_s, g.down_s},
             bo[3] = {g.gate_b, g.up_b, g.down_b};
    int rows = which == FM_MAT_DOWN ? g.hidden : g.inter, cols = which == FM_MAT_DOWN ? g.inter : g.hidden;
    return dequant_common(c, e + wo[which], e + so[which], e + bo[which], rows, cols, g.bits,
                          g.scale_fp16, 0, codes, w_f32, w_f16);
}

extern "C" int fm_dequant_tensor(fm_ctx *c, fm_tensor t, uint8_t *codes, float *w_f32,
                                 uint16_t *w_f16) {
    if (!c) return FM_ERR_ARG;
    Tensor *p = get_tensor(c, t);
    if (!p) return fail(c, FM_ERR_ARG, "bad tensor handle %d", t);
    if (p->raw_bf16()) return fail(c, FM_ERR_UNSUPPORTED, "tensor %d is raw BF16: nothing to dequantize", t);
    DeviceGuard dg(c->device);
    if (p->gguf()) {        // block formats have no integer codes or fp16 form here: fp32 values only
        if (codes || w_f16) return fail(c, FM_ERR_UNSUPPORTED, "GGUF tensor %d: fp32 weights only", t);
        return dequant_common(c, p->W, nullptr, nullptr, p->out_dim, p->in_dim, 0, 0, p->ggml_type(), nullptr,
                              w_f32, nullptr);
    }
    return dequant_common(c, p->W, p->S, p->B, p->out_dim, p->in_dim, p->bits, p->scale_fp16, 0,
                          codes, w_f32, w_f16);
}

extern "C" int fm_launch_embed_rows(const void *W, const void *S, const void *B, int rows, int in_dim,
                                    int group_size, int bits, int scale_fp16, const int32_t *d_ids,
                                    int n, float *d_out, hipStream_t st);

extern "C" int fm_embed_lookup_dev(fm_ctx *c, fm_tensor t, const int32_t *d_token_ids, int n_tokens,
                                   float *d_out) {
    if (!c) return FM_ERR_ARG;
    Tensor *p = get_tensor(c, t);
    if (!p) return fail(c, FM_ERR_ARG, "bad tensor handle %d", t);
    if (!d_token_ids || !d_out) return fail(c, FM_ERR_ARG, "null pointer");
    if (n_tokens < 1) return fail(c, FM_ERR_ARG, "n_tokens %d", n_tokens);
    if (p->raw_bf16()) return fail(c, FM_ERR_UNSUPPORTED, "embedding lookup needs a quantized tensor");
    DeviceGuard dg(c->device);
    if (p->gguf()) {
        int rc = fm_launch_embed_rows_gguf(p->W, p->out_dim, p->in_dim, p->ggml_type(), d_token_ids, n_tokens,
                                           d_out, c->stream);
        if (rc) return fail(c, rc, "embedding lookup launch failed: %s", hipGetErrorString(hipGetLastError()));
        return FM_OK;
    }
    int rc = fm_launch_embed_rows(p->W, p->S, p->B, p->out_dim, p->in_dim, p->group_size, p->bits,
                                  p->scale_fp16, d_token_ids, n_tokens, d_out, c->stream);
    if (rc) return fail(c, rc, "embedding lookup launch failed: %s", hipGetErrorString(hipGetLastError()));
    return FM_OK;
}

extern "C" int fm_embed_lookup(fm_ctx *c, fm_tensor t, int token_id, float *out) {
    if (!c) return FM_ERR_ARG;
    Tensor *p = get_tensor(c, t);
    if (!p) return fail(c, FM_ERR_ARG, "bad tensor handle %d", t);
    if (!out) return fail(c, FM_ERR_ARG, "null pointer");
    DeviceGuard dg(c->device);
    const size_t need = 256 + (size_t)p->in_dim * sizeof(float);
    int rc = ensure_stage(c, need);
    if (rc) return rc;
    *(int32_t *)c->h_stage = token_id;          // pinned mirror of the staging buffer
    HIPCHK(c, hipMemcpyAsync(c->d_stage, c->h_stage, sizeof(int32_t), hipMemcpyHostToDevice, c->stream));
    float *d_out = (float *)((char *)c->d_stage + 256);
    rc = fm_embed_lookup_dev(c, t, (const int32_t *)c->d_stage, 1, d_out);
    if (rc) return rc;
    HIPCHK(c, hipMemcpyAsync(out, d_out, (size_t)p->in_dim * sizeof(float), hipMemcpyDeviceToHost, c->stream));
    HIPCHK(c, hipStreamSynchronize(c->stream));
    return FM_OK;
}

extern "C" int fm_gguf_dequant_expert(fm_ctx *c, int layer, int expert, int which, float *w_f32) {
    if (!c) return FM_ERR_ARG;
    if (!c->gguf_cfg) return fail(c, FM_ERR_STATE, "GGUF store not configured");
    if (!w_f32) return fail(c, FM_ERR_ARG, "null pointer");
    int rc = check_layers(c, c->g_gate, layer, 1);
    if (rc) return rc;
    const FmGgufGeom &g = c->ggeom;
    if (expert < 0 || expert >= g.n_experts) return fail(c, FM_ERR_ARG, "expert %d", expert);
    if (which < FM_MAT_GATE || which > FM_MAT_DOWN) return fail(c, FM_ERR_ARG, "which %d", which);
    DeviceGuard dg(c->device);
    const uint8_t *base;
    int rows, cols, type;
    if (which == FM_MAT_GATE) {
        base = (const uint8_t *)c->g_gate[layer].ptr + (size_t)expert * g.gate_slab;
        rows = g.inter; cols = g.hidden; type = g.gate_type;
    } else if (which == FM_MAT_UP) {
        base = (const uint8_t *)c->g_up[layer].ptr + (size_t)expert * g.up_slab;
        rows = g.inter; cols = g.hidden; type = g.up_type;
    } else {
        base = (const uint8_t *)c->g_down[layer].ptr + (size_t)expert * g.down_slab;
        rows = g.hidden; cols = g.inter; type = g.down_type;
    }
    return dequant_common(c, base, nullptr, nullptr, rows, cols, 0, 0, type, nullptr, w_f32, nullptr);
}
