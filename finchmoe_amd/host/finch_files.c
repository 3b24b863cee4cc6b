/* finch_files.c — see finch_files.h.  C99 + POSIX (open/mmap). */
#define _POSIX_C_SOURCE 200809L
#include "finch_files.h"

#include <errno.h>
#include <fcntl.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include "finch_hip.h"
#include "finch_ops.h"

static char g_ferr[512] = "";

static int ffail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_ferr, sizeof g_ferr, fmt, ap);
    va_end(ap);
    return code;
}

const char *finch_files_last_error(void) { return g_ferr; }

/* ======================================================================================= */
/* quantizer                                                                               */
/* ======================================================================================= */

static uint16_t bf16_cut(float f) {      /* repack_experts.py:232-234: the upper 16 bits */
    uint32_t u;
    memcpy(&u, &f, 4);
    return (uint16_t)(u >> 16);
}

/* Every intermediate is rounded to fp32 where numpy rounds it (w - bias, then / scale, each an
 * fp32 array op); `volatile` keeps the compiler from carrying extra precision or fusing. */
static void quantize_group(const float *p, int n, float maxv, uint8_t *q, uint16_t *scale_bits,
                           uint16_t *bias_bits) {
    float lo = p[0], hi = p[0];
    for (int i = 1; i < n; i++) {
        if (p[i] < lo) lo = p[i];
        if (p[i] > hi) hi = p[i];
    }
    volatile float range = hi - lo;
    volatile float s0 = range / maxv;
    const float scale = s0 > 1e-8f ? s0 : 1e-8f;
    for (int i = 0; i < n; i++) {
        volatile float d = p[i] - lo;
        volatile float t = d / scale;
        float r = rintf(t);               /* round half to even, as numpy.round */
        /* (a NaN — only from non-finite weights, whose quantization numpy leaves to the
         * platform's float-to-integer cast as well — becomes code 0 instead of a cast of NaN) */
        if (!(r >= 0.0f)) r = 0.0f;
        if (r > maxv) r = maxv;
        q[i] = (uint8_t)r;
    }
    *scale_bits = bf16_cut(scale);
    *bias_bits = bf16_cut(lo);
}

int finch_quantize_affine_pack(const float *w, int out_dim, int in_dim, int group_size, int bits,
                               void *packed, uint16_t *scales, uint16_t *biases) {
    if (!w || !packed || !scales || !biases || out_dim <= 0 || in_dim <= 0 || group_size <= 0)
        return ffail(FM_ERR_ARG, "finch_quantize_affine_pack: null or non-positive argument");
    if (bits != 2 && bits != 3 && bits != 4 && bits != 8)
        return ffail(FM_ERR_UNSUPPORTED, "finch_quantize_affine_pack: %d bits", bits);
    if (in_dim % group_size || group_size > 4096)
        return ffail(FM_ERR_ARG, "finch_quantize_affine_pack: in_dim %d, group %d", in_dim, group_size);
    if (bits == 3 ? in_dim % 8 : in_dim % (32 / bits))
        return ffail(FM_ERR_ARG, "finch_quantize_affine_pack: in_dim %d does not fill whole words", in_dim);
    const int ng = in_dim / group_size;
    const float maxv = (float)((1 << bits) - 1);
    uint8_t *q = (uint8_t *)malloc((size_t)in_dim);
    if (!q) return ffail(FM_ERR_NOMEM, "finch_quantize_affine_pack: out of memory");
    const size_t row_bytes = (size_t)in_dim * bits / 8;
    for (int r = 0; r < out_dim; r++) {
        const float *row = w + (size_t)r * in_dim;
        for (int g = 0; g < ng; g++)
            quantize_group(row + (size_t)g * group_size, group_size, maxv, q + (size_t)g * group_size,
                           scales + (size_t)r * ng + g, biases + (size_t)r * ng + g);
        uint8_t *dst = (uint8_t *)packed + (size_t)r * row_bytes;
        if (bits == 3) {
            for (int t = 0; t < in_dim / 8; t++) {
                uint32_t v = 0;
                for (int j = 0; j < 8; j++) v |= (uint32_t)q[8 * t + j] << (3 * j);
                dst[3 * t] = (uint8_t)v;
                dst[3 * t + 1] = (uint8_t)(v >> 8);
                dst[3 * t + 2] = (uint8_t)(v >> 16);
            }
        } else {
            const int per = 32 / bits;
            for (int t = 0; t < in_dim / per; t++) {
                uint32_t v = 0;
                for (int j = 0; j < per; j++) v |= (uint32_t)q[per * t + j] << (bits * j);
                dst[4 * t] = (uint8_t)v;               /* little-endian, whatever the host is */
                dst[4 * t + 1] = (uint8_t)(v >> 8);
                dst[4 * t + 2] = (uint8_t)(v >> 16);
                dst[4 * t + 3] = (uint8_t)(v >> 24);
            }
        }
    }
    free(q);
    return FM_OK;
}

size_t finch_expert_blob_size(int hidden, int inter, int group_size, int bits) {
    if (hidden <= 0 || inter <= 0 || group_size <= 0 || hidden % group_size || inter % group_size) return 0;
    if (bits != 2 && bits != 3 && bits != 4 && bits != 8) return 0;
    const size_t gu = (size_t)inter * hidden * bits / 8 + 2 * (size_t)inter * (hidden / group_size) * 2;
    const size_t dn = (size_t)hidden * inter * bits / 8 + 2 * (size_t)hidden * (inter / group_size) * 2;
    return 2 * gu + dn;
}

int finch_quantize_expert(const float *gate, const float *up, const float *down, int hidden,
                          int inter, int group_size, int bits, void *blob) {
    if (!finch_expert_blob_size(hidden, inter, group_size, bits) || !blob)
        return ffail(FM_ERR_ARG, "finch_quantize_expert: geometry %dx%d, group %d, %d bits", hidden,
                     inter, group_size, bits);
    uint8_t *p = (uint8_t *)blob;
    const float *src[3] = {gate, up, down};
    for (int k = 0; k < 3; k++) {
        const int out_dim = k < 2 ? inter : hidden, in_dim = k < 2 ? hidden : inter;
        const size_t wb = (size_t)out_dim * in_dim * bits / 8, sb = (size_t)out_dim * (in_dim / group_size) * 2;
        int rc = finch_quantize_affine_pack(src[k], out_dim, in_dim, group_size, bits, p,
                                            (uint16_t *)(p + wb), (uint16_t *)(p + wb + sb));
        if (rc) return rc;
        p += wb + 2 * sb;
    }
    return FM_OK;
}

/* ======================================================================================= */
/* read-only file mappings                                                                 */
/* ======================================================================================= */

typedef struct {
    const uint8_t *p;
    size_t n;
} fmap;

static int map_file(const char *path, fmap *m) {
    m->p = NULL;
    m->n = 0;
    int fd = open(path, O_RDONLY);
    if (fd < 0) return ffail(FM_ERR_ARG, "cannot open %s: %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size <= 0) {
        close(fd);
        return ffail(FM_ERR_ARG, "%s is empty or cannot be examined", path);
    }
    void *p = mmap(NULL, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (p == MAP_FAILED) return ffail(FM_ERR_NOMEM, "mmap of %s failed: %s", path, strerror(errno));
    m->p = (const uint8_t *)p;
    m->n = (size_t)st.st_size;
    return FM_OK;
}

static void unmap_file(fmap *m) {
    if (m->p) munmap((void *)m->p, m->n);
    m->p = NULL;
    m->n = 0;
}

int finch_file_map(const char *path, const void **data, size_t *nbytes) {
    fmap m;
    if (!path || !data || !nbytes) return ffail(FM_ERR_ARG, "finch_file_map: null argument");
    int rc = map_file(path, &m);
    *data = m.p;
    *nbytes = m.n;
    return rc;
}

void finch_file_unmap(const void *data, size_t nbytes) {
    if (data && nbytes) munmap((void *)data, nbytes);
}

/* ======================================================================================= */
/* expert layer files                                                                      */
/* ======================================================================================= */

int finch_expert_layer_path(const char *dir, int layer, char *out, size_t out_size) {
    if (!dir || !out || layer < 0) return ffail(FM_ERR_ARG, "finch_expert_layer_path: bad argument");
    int n = snprintf(out, out_size, "%s/layer_%02d.bin", dir, layer);
    return n > 0 && (size_t)n < out_size ? FM_OK : ffail(FM_ERR_ARG, "finch_expert_layer_path: path too long");
}

int finch_ops_load_expert_dir(const char *dir, int n_layers) {
    if (!dir || n_layers <= 0) return ffail(FM_ERR_ARG, "finch_ops_load_expert_dir: bad argument");
    int loaded = 0;
    for (int l = 0; l < n_layers; l++) {
        char path[1024];
        int rc = finch_expert_layer_path(dir, l, path, sizeof path);
        if (rc) return rc;
        if (access(path, R_OK) != 0) continue;          /* layers without a file stay absent */
        fmap m;
        if ((rc = map_file(path, &m))) return rc;
        const size_t nbytes = m.n;
        rc = finch_ops_load_expert_layer(l, m.p, nbytes);   /* the store checks the size */
        unmap_file(&m);
        if (rc) return ffail(rc, "%s (%zu bytes): %s", path, nbytes, finch_ops_last_error());
        loaded++;
    }
    return loaded;
}

/* ======================================================================================= */
/* JSON (just enough for the manifest: objects, arrays, strings, numbers, literals)        */
/* ======================================================================================= */

typedef struct {
    const char *p, *end;
    int bad;
} jcur;

static void j_ws(jcur *c) {
    while (c->p < c->end && (*c->p == ' ' || *c->p == '\t' || *c->p == '\n' || *c->p == '\r')) c->p++;
}

static int j_eat(jcur *c, char ch) {
    j_ws(c);
    if (c->p < c->end && *c->p == ch) {
        c->p++;
        return 1;
    }
    return 0;
}

static int j_peek(jcur *c) {
    j_ws(c);
    return c->p < c->end ? (unsigned char)*c->p : -1;
}

static int hex4(const char *s, unsigned *out) {
    unsigned v = 0;
    for (int i = 0; i < 4; i++) {
        char ch = s[i];
        v <<= 4;
        if (ch >= '0' && ch <= '9') v |= (unsigned)(ch - '0');
        else if (ch >= 'a' && ch <= 'f') v |= (unsigned)(ch - 'a' + 10);
        else if (ch >= 'A' && ch <= 'F') v |= (unsigned)(ch - 'A' + 10);
        else return 0;
    }
    *out = v;
    return 1;
}

static size_t utf8_put(char *dst, unsigned cp) {
    if (cp < 0x80) { dst[0] = (char)cp; return 1; }
    if (cp < 0x800) { dst[0] = (char)(0xC0 | (cp >> 6)); dst[1] = (char)(0x80 | (cp & 63)); return 2; }
    if (cp < 0x10000) {
        dst[0] = (char)(0xE0 | (cp >> 12)); dst[1] = (char)(0x80 | ((cp >> 6) & 63)); dst[2] = (char)(0x80 | (cp & 63));
        return 3;
    }
    dst[0] = (char)(0xF0 | (cp >> 18)); dst[1] = (char)(0x80 | ((cp >> 12) & 63));
    dst[2] = (char)(0x80 | ((cp >> 6) & 63)); dst[3] = (char)(0x80 | (cp & 63));
    return 4;
}

/* a string -> malloc'd UTF-8 (NULL and c->bad on error); the unescaped form is never longer */
static char *j_string(jcur *c) {
    if (!j_eat(c, '"')) { c->bad = 1; return NULL; }
    const char *s = c->p;
    while (s < c->end && *s != '"') s += (*s == '\\' && s + 1 < c->end) ? 2 : 1;
    if (s >= c->end) { c->bad = 1; return NULL; }
    char *out = (char *)malloc((size_t)(s - c->p) + 1);
    if (!out) { c->bad = 1; return NULL; }
    size_t n = 0;
    const char *p = c->p;
    while (p < s) {
        if (*p != '\\') { out[n++] = *p++; continue; }
        char e = p[1];
        p += 2;
        switch (e) {
            case 'n': out[n++] = '\n'; break;
            case 't': out[n++] = '\t'; break;
            case 'r': out[n++] = '\r'; break;
            case 'b': out[n++] = '\b'; break;
            case 'f': out[n++] = '\f'; break;
            case 'u': {
                unsigned cp, lo;
                if (p + 4 > s || !hex4(p, &cp)) { free(out); c->bad = 1; return NULL; }
                p += 4;
                if (cp >= 0xD800 && cp < 0xDC00 && p + 6 <= s && p[0] == '\\' && p[1] == 'u' &&
                    hex4(p + 2, &lo) && lo >= 0xDC00 && lo < 0xE000) {
                    cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                    p += 6;
                }
                n += utf8_put(out + n, cp);
                break;
            }
            default: out[n++] = e;      /* \" \\ \/ */
        }
    }
    out[n] = 0;
    c->p = s + 1;
    return out;
}

static double j_number(jcur *c) {
    j_ws(c);
    char buf[64];
    size_t n = 0;
    while (c->p < c->end && n + 1 < sizeof buf &&
           ((*c->p >= '0' && *c->p <= '9') || *c->p == '-' || *c->p == '+' || *c->p == '.' || *c->p == 'e' || *c->p == 'E'))
        buf[n++] = *c->p++;
    buf[n] = 0;
    if (!n) { c->bad = 1; return 0; }
    char *e;
    double v = strtod(buf, &e);
    if (*e) c->bad = 1;
    return v;
}

/* a number that must be an integer in [lo, hi] (a double holds every file offset below 2^53
 * exactly); anything else makes the manifest bad instead of being converted */
static int64_t j_int(jcur *c, double lo, double hi) {
    const double v = j_number(c);
    if (!(v >= lo && v <= hi) || v != (double)(int64_t)v) { c->bad = 1; return 0; }
    return (int64_t)v;
}

static void j_skip(jcur *c, int depth) {
    if (c->bad || depth > 64) { c->bad = 1; return; }
    int ch = j_peek(c);
    if (ch == '"') {
        free(j_string(c));
    } else if (ch == '{' || ch == '[') {
        const char close = ch == '{' ? '}' : ']';
        c->p++;
        if (j_eat(c, close)) return;
        do {
            if (ch == '{') {
                free(j_string(c));
                if (!j_eat(c, ':')) c->bad = 1;
            }
            j_skip(c, depth + 1);
        } while (!c->bad && j_eat(c, ','));
        if (!j_eat(c, close)) c->bad = 1;
    } else if (ch == 't' && c->end - c->p >= 4 && !memcmp(c->p, "true", 4)) {
        c->p += 4;
    } else if (ch == 'f' && c->end - c->p >= 5 && !memcmp(c->p, "false", 5)) {
        c->p += 5;
    } else if (ch == 'n' && c->end - c->p >= 4 && !memcmp(c->p, "null", 4)) {
        c->p += 4;
    } else {
        (void)j_number(c);
    }
}

/* ======================================================================================= */
/* model_weights_quant.bin + manifest                                                      */
/* ======================================================================================= */

typedef struct {
    char *name;
    uint64_t offset, size;
    int ndim;
    int64_t shape[4];
    char dtype[8];
    int bits, group_size;
} dense_ent;

struct finch_dense {
    fmap map;
    char *model;
    dense_ent *ent;
    int n, cap;
    int *ht;             /* open addressing over ent indices, -1 = free */
    int ht_size;
};

static uint32_t fnv1a(const char *s) {
    uint32_t h = 2166136261u;
    for (; *s; s++) h = (h ^ (unsigned char)*s) * 16777619u;
    return h;
}

static int ht_build(int **ht_out, int *size_out, int n, const char *(*name_at)(const void *, int),
                    const void *owner) {
    int size = 64;
    while (size < 4 * n) size <<= 1;
    int *ht = (int *)malloc(sizeof(int) * (size_t)size);
    if (!ht) return 0;
    for (int i = 0; i < size; i++) ht[i] = -1;
    for (int i = 0; i < n; i++) {
        uint32_t h = fnv1a(name_at(owner, i)) & (uint32_t)(size - 1);
        while (ht[h] >= 0) h = (h + 1) & (uint32_t)(size - 1);
        ht[h] = i;
    }
    *ht_out = ht;
    *size_out = size;
    return 1;
}

static int ht_find(const int *ht, int size, const char *name, const char *(*name_at)(const void *, int),
                   const void *owner) {
    if (!ht || !name) return -1;
    uint32_t h = fnv1a(name) & (uint32_t)(size - 1);
    while (ht[h] >= 0) {
        if (!strcmp(name_at(owner, ht[h]), name)) return ht[h];
        h = (h + 1) & (uint32_t)(size - 1);
    }
    return -1;
}

static const char *dense_name_at(const void *o, int i) { return ((const finch_dense *)o)->ent[i].name; }

/* one manifest entry: {"offset":..,"size":..,"shape":[..],"dtype":"..", "bits":.., "group_size":..} */
static void parse_entry(jcur *c, dense_ent *e) {
    int have = 0;
    if (!j_eat(c, '{')) { c->bad = 1; return; }
    if (j_eat(c, '}')) { c->bad = 1; return; }
    do {
        char *k = j_string(c);
        if (!k || !j_eat(c, ':')) { free(k); c->bad = 1; return; }
        if (!strcmp(k, "offset")) { e->offset = (uint64_t)j_int(c, 0.0, 9007199254740992.0); have |= 1; }
        else if (!strcmp(k, "size")) { e->size = (uint64_t)j_int(c, 0.0, 9007199254740992.0); have |= 2; }
        else if (!strcmp(k, "bits") && j_peek(c) != 'n') e->bits = (int)j_int(c, -2147483648.0, 2147483647.0);
        else if (!strcmp(k, "group_size") && j_peek(c) != 'n') e->group_size = (int)j_int(c, -2147483648.0, 2147483647.0);
        else if (!strcmp(k, "dtype")) {
            char *d = j_string(c);
            if (d) { strncpy(e->dtype, d, sizeof e->dtype - 1); have |= 4; }
            free(d);
        } else if (!strcmp(k, "shape")) {
            if (!j_eat(c, '[')) c->bad = 1;
            else if (!j_eat(c, ']')) {
                do {
                    const int64_t v = j_int(c, -9007199254740992.0, 9007199254740992.0);
                    if (e->ndim < 4) e->shape[e->ndim] = v;
                    e->ndim++;
                } while (!c->bad && j_eat(c, ','));
                if (!j_eat(c, ']')) c->bad = 1;
            }
            have |= 8;
        } else j_skip(c, 0);
        free(k);
    } while (!c->bad && j_eat(c, ','));
    if (!j_eat(c, '}')) c->bad = 1;
    if ((have & 7) != 7) c->bad = 1;       /* offset, size and dtype are read unconditionally by the reference */
    if (e->ndim > 4) e->ndim = 4;
}

static int parse_manifest(finch_dense *d, const char *txt, size_t n, const char *json_path) {
    jcur c = {txt, txt + n, 0};
    int have_tensors = 0;
    if (!j_eat(&c, '{')) return ffail(FM_ERR_ARG, "%s: not a JSON object", json_path);
    if (!j_eat(&c, '}')) {
        do {
            char *k = j_string(&c);
            if (!k || !j_eat(&c, ':')) { free(k); c.bad = 1; break; }
            if (!strcmp(k, "model") && j_peek(&c) == '"') {
                free(d->model);
                d->model = j_string(&c);
            } else if (!strcmp(k, "tensors") && j_peek(&c) == '{') {
                have_tensors = 1;
                c.p++;
                if (!j_eat(&c, '}')) {
                    do {
                        if (d->n == d->cap) {
                            int cap = d->cap ? 2 * d->cap : 256;
                            dense_ent *ne = (dense_ent *)realloc(d->ent, sizeof(dense_ent) * (size_t)cap);
                            if (!ne) { free(k); return ffail(FM_ERR_NOMEM, "%s: out of memory", json_path); }
                            d->ent = ne;
                            d->cap = cap;
                        }
                        dense_ent *e = &d->ent[d->n];
                        memset(e, 0, sizeof *e);
                        e->name = j_string(&c);
                        if (!e->name || !j_eat(&c, ':')) { free(e->name); c.bad = 1; break; }
                        d->n++;
                        parse_entry(&c, e);
                    } while (!c.bad && j_eat(&c, ','));
                    if (!c.bad && !j_eat(&c, '}')) c.bad = 1;
                }
            } else j_skip(&c, 0);
            free(k);
        } while (!c.bad && j_eat(&c, ','));
        if (!c.bad && !j_eat(&c, '}')) c.bad = 1;
    }
    if (c.bad) return ffail(FM_ERR_ARG, "%s: JSON parse failed near byte %zu", json_path, (size_t)(c.p - txt));
    if (!have_tensors) return ffail(FM_ERR_ARG, "%s: no 'tensors' key", json_path);   /* infer.m:747-750 */
    return FM_OK;
}

finch_dense *finch_ops_open_dense(const char *bin_path, const char *json_path) {
    if (!bin_path) { ffail(FM_ERR_ARG, "finch_ops_open_dense: no path"); return NULL; }
    char auto_json[1024];
    if (!json_path) {
        const char *dot = strrchr(bin_path, '.'), *slash = strrchr(bin_path, '/');
        size_t stem = dot && (!slash || dot > slash) ? (size_t)(dot - bin_path) : strlen(bin_path);
        if (stem + 6 > sizeof auto_json) { ffail(FM_ERR_ARG, "finch_ops_open_dense: path too long"); return NULL; }
        memcpy(auto_json, bin_path, stem);
        strcpy(auto_json + stem, ".json");
        json_path = auto_json;
    }
    finch_dense *d = (finch_dense *)calloc(1, sizeof *d);
    if (!d) { ffail(FM_ERR_NOMEM, "finch_ops_open_dense: out of memory"); return NULL; }
    fmap js;
    if (map_file(json_path, &js)) { free(d); return NULL; }
    int rc = parse_manifest(d, (const char *)js.p, js.n, json_path);
    unmap_file(&js);
    if (!rc) rc = map_file(bin_path, &d->map);
    for (int i = 0; !rc && i < d->n; i++)
        if (d->ent[i].offset > d->map.n || d->ent[i].size > d->map.n - d->ent[i].offset)
            rc = ffail(FM_ERR_ARG, "%s: %s ends past the file", bin_path, d->ent[i].name);
    if (!rc && !ht_build(&d->ht, &d->ht_size, d->n, dense_name_at, d))
        rc = ffail(FM_ERR_NOMEM, "finch_ops_open_dense: out of memory");
    if (rc) { finch_ops_close_dense(d); return NULL; }
    return d;
}

void finch_ops_close_dense(finch_dense *d) {
    if (!d) return;
    /* resident copies keyed by addresses inside the mapping must not outlive it */
    for (int i = 0; i < d->n; i++) {
        /* (an entry that ends past the file made the open fail: its offset is not an address) */
        if (d->map.p && d->ent[i].offset <= d->map.n && !strcmp(d->ent[i].dtype, "U32"))
            finch_ops_forget_tensor(d->map.p + d->ent[i].offset);
        free(d->ent[i].name);
    }
    unmap_file(&d->map);
    free(d->ent);
    free(d->ht);
    free(d->model);
    free(d);
}

int finch_dense_count(const finch_dense *d) { return d ? d->n : 0; }
const char *finch_dense_model(const finch_dense *d) { return d ? d->model : NULL; }

int finch_dense_entry_at(const finch_dense *d, int i, finch_dense_entry *out) {
    if (!d || !out || i < 0 || i >= d->n) return ffail(FM_ERR_ARG, "finch_dense_entry_at: index %d", i);
    const dense_ent *e = &d->ent[i];
    memset(out, 0, sizeof *out);
    out->name = e->name;
    out->data = d->map.p + e->offset;
    out->offset = e->offset;
    out->size = (size_t)e->size;
    out->ndim = e->ndim;
    memcpy(out->shape, e->shape, sizeof out->shape);
    memcpy(out->dtype, e->dtype, sizeof out->dtype);
    out->bits = e->bits;
    out->group_size = e->group_size;
    return FM_OK;
}

int finch_dense_find(const finch_dense *d, const char *name, finch_dense_entry *out) {
    int i = d ? ht_find(d->ht, d->ht_size, name, dense_name_at, d) : -1;
    if (i < 0) return ffail(FM_ERR_ARG, "no tensor named %s", name ? name : "(null)");
    return finch_dense_entry_at(d, i, out);
}

int finch_dense_quantized(const finch_dense *d, const char *weight_name, const void **W,
                          const uint16_t **S, const uint16_t **B, int *out_dim, int *in_dim,
                          int *bits, int *group_size) {
    finch_dense_entry w, s, b;
    int rc = finch_dense_find(d, weight_name, &w);
    if (rc) return rc;
    if (strcmp(w.dtype, "U32")) return ffail(FM_ERR_ARG, "%s is %s, not a packed tensor", weight_name, w.dtype);
    if (w.ndim != 2 || w.bits <= 0 || w.group_size <= 0 || 32 % w.bits)
        return ffail(FM_ERR_ARG, "%s: %d-d, bits %d, group %d", weight_name, w.ndim, w.bits, w.group_size);
    const int64_t od = w.shape[0], id = w.shape[1] * 32 / w.bits;
    if (od <= 0 || id <= 0 || od > INT32_MAX || id > INT32_MAX || id % w.group_size)
        return ffail(FM_ERR_ARG, "%s: in_dim %lld is not a multiple of the group size %d", weight_name,
                     (long long)id, w.group_size);
    size_t nl = strlen(weight_name), stem = nl > 7 && !strcmp(weight_name + nl - 7, ".weight") ? nl - 7 : nl;
    char name[1024];
    if (stem + 8 > sizeof name) return ffail(FM_ERR_ARG, "%s: name too long", weight_name);
    memcpy(name, weight_name, stem);
    strcpy(name + stem, ".scales");
    if ((rc = finch_dense_find(d, name, &s))) return rc;
    strcpy(name + stem, ".biases");
    if ((rc = finch_dense_find(d, name, &b))) return rc;
    const size_t sb = (size_t)od * (size_t)(id / w.group_size) * 2;
    if (w.size != (size_t)od * (size_t)w.shape[1] * 4 || s.size != sb || b.size != sb)
        return ffail(FM_ERR_ARG, "%s: entry sizes do not match its shape", weight_name);
    if (W) *W = w.data;
    if (S) *S = (const uint16_t *)s.data;
    if (B) *B = (const uint16_t *)b.data;
    if (out_dim) *out_dim = (int)od;
    if (in_dim) *in_dim = (int)id;
    if (bits) *bits = w.bits;
    if (group_size) *group_size = w.group_size;
    return FM_OK;
}

int finch_ops_load_dense_tensor(const finch_dense *d, const char *weight_name) {
    const void *W;
    const uint16_t *S, *B;
    int od, id, bits, gs;
    int rc = finch_dense_quantized(d, weight_name, &W, &S, &B, &od, &id, &bits, &gs);
    if (rc) return rc;
    rc = finch_ops_make_resident(W, S, B, od, id, gs, bits);
    return rc ? ffail(rc, "%s: %s", weight_name, finch_ops_last_error()) : FM_OK;
}

/* ======================================================================================= */
/* GGUF                                                                                    */
/* ======================================================================================= */

typedef struct {
    char *name;
    int type, ndim;
    uint64_t dims[4], off;
    size_t nbytes;
} gguf_ent;

struct finch_gguf {
    fmap map;
    uint32_t version, alignment;
    uint64_t data_off;
    gguf_ent *ent;
    int n;
    int *ht;
    int ht_size;
};

int finch_ggml_block(int type, int *elems, int *bytes) {
    int e = 0, b = 0;
    switch (type) {           /* infer.m:934-948, plus Q8_0 and BF16 */
        case 0: e = 1, b = 4; break;        /* F32  */
        case 1: e = 1, b = 2; break;        /* F16  */
        case 8: e = 32, b = 34; break;      /* Q8_0 */
        case 12: e = 256, b = 144; break;   /* Q4_K */
        case 14: e = 256, b = 210; break;   /* Q6_K */
        case 30: e = 1, b = 2; break;       /* BF16 */
        default: break;
    }
    if (elems) *elems = e;
    if (bytes) *bytes = b;
    return e;
}

typedef struct {
    const uint8_t *p, *end;
    int bad;
} gcur;

static uint64_t g_int(gcur *c, int n) {
    if ((size_t)(c->end - c->p) < (size_t)n) { c->bad = 1; c->p = c->end; return 0; }
    uint64_t v = 0;
    for (int i = 0; i < n; i++) v |= (uint64_t)c->p[i] << (8 * i);
    c->p += n;
    return v;
}

static void g_skip(gcur *c, uint64_t n) {
    if ((uint64_t)(c->end - c->p) < n) { c->bad = 1; c->p = c->end; return; }
    c->p += n;
}

static const size_t GGUF_SCALAR[13] = {1, 1, 2, 2, 4, 4, 4, 1, 0, 0, 8, 8, 8};

/* skips one value of type vt; *as_u64 receives it when it is an integer scalar */
static void g_value(gcur *c, uint32_t vt, uint64_t *as_u64, int depth) {
    if (vt == 8) {
        g_skip(c, g_int(c, 8));
    } else if (vt == 9) {
        uint32_t at = (uint32_t)g_int(c, 4);
        uint64_t n = g_int(c, 8);
        if (at == 8 || at == 9) {
            if (depth > 4) { c->bad = 1; return; }
            for (uint64_t j = 0; j < n && !c->bad; j++) g_value(c, at, NULL, depth + 1);
        } else if (at < 13) {
            if (n > (uint64_t)(c->end - c->p)) c->bad = 1;
            else g_skip(c, n * GGUF_SCALAR[at]);
        } else c->bad = 1;
    } else if (vt < 13) {
        uint64_t v = g_int(c, (int)GGUF_SCALAR[vt]);
        if (as_u64 && vt != 6 && vt != 12) *as_u64 = v;
    } else c->bad = 1;
}

static const char *gguf_name_at(const void *o, int i) { return ((const finch_gguf *)o)->ent[i].name; }

finch_gguf *finch_ops_open_gguf(const char *path) {
    if (!path) { ffail(FM_ERR_ARG, "finch_ops_open_gguf: no path"); return NULL; }
    finch_gguf *g = (finch_gguf *)calloc(1, sizeof *g);
    if (!g) { ffail(FM_ERR_NOMEM, "finch_ops_open_gguf: out of memory"); return NULL; }
    if (map_file(path, &g->map)) { free(g); return NULL; }
    gcur c = {g->map.p, g->map.p + g->map.n, 0};
    int rc = FM_OK;
    if (g->map.n < 24 || g_int(&c, 4) != 0x46554747u) {               /* infer.m:1040-1041 */
        rc = ffail(FM_ERR_ARG, "%s is not a GGUF file", path);
        goto done;
    }
    g->version = (uint32_t)g_int(&c, 4);
    const uint64_t n_tensors = g_int(&c, 8), n_kv = g_int(&c, 8);
    if (g->version < 2 || n_tensors > (1u << 24) || n_kv > (1u << 24)) {
        rc = ffail(FM_ERR_UNSUPPORTED, "%s: GGUF version %u with %llu tensors", path, g->version,
                   (unsigned long long)n_tensors);
        goto done;
    }
    g->alignment = 32;
    for (uint64_t i = 0; i < n_kv && !c.bad; i++) {
        const uint64_t klen = g_int(&c, 8);
        const uint8_t *key = c.p;
        g_skip(&c, klen);
        const uint32_t vt = (uint32_t)g_int(&c, 4);
        uint64_t v = 0;
        g_value(&c, vt, &v, 0);
        if (!c.bad && klen == 17 && !memcmp(key, "general.alignment", 17) && v && !(v & (v - 1)) && v <= (1u << 20))
            g->alignment = (uint32_t)v;
    }
    if (c.bad) { rc = ffail(FM_ERR_ARG, "%s: key/value section runs past the file", path); goto done; }
    g->ent = (gguf_ent *)calloc(n_tensors ? (size_t)n_tensors : 1, sizeof(gguf_ent));
    if (!g->ent) { rc = ffail(FM_ERR_NOMEM, "finch_ops_open_gguf: out of memory"); goto done; }
    for (uint64_t i = 0; i < n_tensors; i++) {
        const uint64_t nlen = g_int(&c, 8);
        const uint8_t *nm = c.p;
        g_skip(&c, nlen);
        if (c.bad || nlen > 4096) { rc = ffail(FM_ERR_ARG, "%s: tensor infos overrun", path); goto done; }
        gguf_ent *e = &g->ent[g->n];
        e->name = (char *)malloc((size_t)nlen + 1);
        if (!e->name) { rc = ffail(FM_ERR_NOMEM, "finch_ops_open_gguf: out of memory"); goto done; }
        memcpy(e->name, nm, (size_t)nlen);
        e->name[nlen] = 0;
        g->n++;
        const uint32_t nd = (uint32_t)g_int(&c, 4);
        if (nd > 8) { rc = ffail(FM_ERR_ARG, "%s: %s has %u dimensions", path, e->name, nd); goto done; }
        e->ndim = nd < 4 ? (int)nd : 4;
        for (uint32_t k = 0; k < nd; k++) {
            uint64_t v = g_int(&c, 8);
            if (k < 4) e->dims[k] = v;
        }
        e->type = (int)(uint32_t)g_int(&c, 4);
        e->off = g_int(&c, 8);
        if (c.bad) { rc = ffail(FM_ERR_ARG, "%s: tensor infos overrun", path); goto done; }
    }
    g->data_off = ((uint64_t)(c.p - g->map.p) + g->alignment - 1) / g->alignment * g->alignment;
    for (int i = 0; i < g->n; i++) {
        gguf_ent *e = &g->ent[i];
        int be, bs;
        if (!finch_ggml_block(e->type, &be, &bs) || e->ndim < 1 || e->dims[0] % (uint64_t)be) continue;   /* size unknown: data stays NULL */
        uint64_t nb = e->dims[0] / (uint64_t)be * (uint64_t)bs;                          /* infer.m:1141-1143 */
        int over = 0;
        for (int k = 1; k < e->ndim; k++) {
            if (e->dims[k] && nb > UINT64_MAX / e->dims[k]) over = 1;
            nb *= e->dims[k];
        }
        if (over || g->data_off > g->map.n || e->off > g->map.n - g->data_off || nb > g->map.n - g->data_off - e->off) {
            rc = ffail(FM_ERR_ARG, "%s: %s ends past the file", path, e->name);
            goto done;
        }
        e->nbytes = (size_t)nb;
    }
    if (!ht_build(&g->ht, &g->ht_size, g->n, gguf_name_at, g)) rc = ffail(FM_ERR_NOMEM, "finch_ops_open_gguf: out of memory");
done:
    if (rc) { finch_ops_close_gguf(g); return NULL; }
    return g;
}

void finch_ops_close_gguf(finch_gguf *g) {
    if (!g) return;
    for (int i = 0; i < g->n; i++) free(g->ent[i].name);
    free(g->ent);
    free(g->ht);
    unmap_file(&g->map);
    free(g);
}

int finch_gguf_version(const finch_gguf *g) { return g ? (int)g->version : 0; }
int finch_gguf_alignment(const finch_gguf *g) { return g ? (int)g->alignment : 0; }
uint64_t finch_gguf_data_offset(const finch_gguf *g) { return g ? g->data_off : 0; }
int finch_gguf_count(const finch_gguf *g) { return g ? g->n : 0; }

int finch_gguf_tensor_at(const finch_gguf *g, int i, finch_gguf_tensor *out) {
    if (!g || !out || i < 0 || i >= g->n) return ffail(FM_ERR_ARG, "finch_gguf_tensor_at: index %d", i);
    const gguf_ent *e = &g->ent[i];
    memset(out, 0, sizeof *out);
    out->name = e->name;
    out->type = e->type;
    out->ndim = e->ndim;
    memcpy(out->dims, e->dims, sizeof out->dims);
    out->data = e->nbytes ? g->map.p + g->data_off + e->off : NULL;
    out->nbytes = e->nbytes;
    return FM_OK;
}

int finch_gguf_find(const finch_gguf *g, const char *name, finch_gguf_tensor *out) {
    int i = g ? ht_find(g->ht, g->ht_size, name, gguf_name_at, g) : -1;
    if (i < 0) return ffail(FM_ERR_ARG, "no tensor named %s", name ? name : "(null)");
    return finch_gguf_tensor_at(g, i, out);
}

static int expert_tensors(const finch_gguf *g, int layer, finch_gguf_tensor t[3]) {
    static const char *const part[3] = {"gate", "up", "down"};
    for (int k = 0; k < 3; k++) {
        char name[96];
        snprintf(name, sizeof name, "blk.%d.ffn_%s_exps.weight", layer, part[k]);   /* infer.m:1017-1022 */
        int i = ht_find(g->ht, g->ht_size, name, gguf_name_at, g);
        if (i < 0) return 0;
        finch_gguf_tensor_at(g, i, &t[k]);
    }
    return 1;
}

int finch_gguf_has_expert_layer(const finch_gguf *g, int layer) {
    finch_gguf_tensor t[3];
    return g && layer >= 0 && expert_tensors(g, layer, t);
}

int finch_gguf_expert_geometry(const finch_gguf *g, int layer, int *n_experts, int *hidden,
                               int *inter, int types[3]) {
    if (!g) return ffail(FM_ERR_ARG, "finch_gguf_expert_geometry: no file");
    finch_gguf_tensor t[3];
    if (layer < 0) {
        for (int i = 0; i < g->n; i++) {      /* the lowest layer that is complete */
            int l = -1, used = 0;
            if (sscanf(g->ent[i].name, "blk.%d.%n", &l, &used) == 1 && l >= 0 && (layer < 0 || l < layer) &&
                !strcmp(g->ent[i].name + used, "ffn_gate_exps.weight") && expert_tensors(g, l, t))
                layer = l;
        }
        if (layer < 0) return ffail(FM_ERR_STATE, "the file has no stacked expert tensors");
    } else if (!expert_tensors(g, layer, t)) {
        return ffail(FM_ERR_STATE, "layer %d has no stacked expert tensors", layer);
    }
    expert_tensors(g, layer, t);
    const uint64_t H = t[0].dims[0], I = t[0].dims[1], E = t[0].dims[2];
    if (t[0].ndim != 3 || t[1].ndim != 3 || t[2].ndim != 3 || memcmp(t[0].dims, t[1].dims, 3 * sizeof(uint64_t)) ||
        t[2].dims[0] != I || t[2].dims[1] != H || t[2].dims[2] != E || H > INT32_MAX || I > INT32_MAX || E > INT32_MAX)
        return ffail(FM_ERR_ARG, "expert tensors of layer %d disagree on their shapes", layer);
    if (n_experts) *n_experts = (int)E;
    if (hidden) *hidden = (int)H;
    if (inter) *inter = (int)I;
    if (types) for (int k = 0; k < 3; k++) types[k] = t[k].type;
    return FM_OK;
}

int finch_ops_load_gguf_experts(const finch_gguf *g, int n_layers) {
    if (!g || n_layers <= 0) return ffail(FM_ERR_ARG, "finch_ops_load_gguf_experts: bad argument");
    int loaded = 0;
    for (int l = 0; l < n_layers; l++) {
        finch_gguf_tensor t[3];
        if (!expert_tensors(g, l, t)) continue;
        if (!t[0].data || !t[1].data || !t[2].data)
            return ffail(FM_ERR_UNSUPPORTED, "layer %d: expert tensors of a type this library does not read", l);
        int rc = finch_ops_load_gguf_layer(l, t[0].data, t[0].nbytes, t[1].data, t[1].nbytes, t[2].data, t[2].nbytes);
        if (rc) return ffail(rc, "layer %d: %s", l, finch_ops_last_error());
        loaded++;
    }
    return loaded;
}
