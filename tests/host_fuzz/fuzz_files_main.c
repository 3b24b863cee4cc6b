/* Driver for tests/test_host_fuzz.py: runs the readers of finch_files.c over every file of a
 * directory, built with -fsanitize=address,undefined (host code only, no GPU).  The readers
 * take files that somebody else wrote; a damaged manifest or GGUF directory must end in an
 * error code, never in a read outside the mapping.  Every tensor that a reader accepts is
 * read first to last byte, so that a data pointer or size that leaves the mapping faults
 * here.  The upload functions of the host layer are replaced by the counting doubles below:
 * they are not what is under test and would need a GPU.
 *
 *   fuzz_files_main dense <dir>    every *.json in <dir> with the same-named .bin
 *   fuzz_files_main gguf  <dir>    every *.gguf in <dir>
 *   fuzz_files_main quant -        the quantizer on tensors salted with NaN, infinities, the largest
 *                                  and the smallest floats and constant groups: error codes or codes,
 *                                  never a conversion the C standard leaves undefined
 * Prints one line per file before it is opened, and a summary; exit code 0 unless a
 * sanitizer aborts the process. */
#include <dirent.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "finch_files.h"
#include "finch_ops.h"

/* ---- doubles for what finch_files.c calls in finch_ops.c ---- */
static unsigned long g_touched;
static void touch(const void *p, size_t n) {
    const volatile unsigned char *b = (const volatile unsigned char *)p;
    unsigned long s = 0;
    for (size_t i = 0; i < n; i += 61) s += b[i];
    if (n) s += b[n - 1];
    g_touched += s;
}
int finch_ops_load_expert_layer(int layer, const void *blob, size_t nbytes) {
    (void)layer;
    touch(blob, nbytes);
    return 0;
}
int finch_ops_load_gguf_layer(int layer, const void *gate, size_t gb, const void *up, size_t ub,
                              const void *down, size_t db) {
    (void)layer;
    touch(gate, gb);
    touch(up, ub);
    touch(down, db);
    return 0;
}
int finch_ops_make_resident(const void *W, const uint16_t *S, const uint16_t *B, int out_dim,
                            int in_dim, int group_size, int bits) {
    const size_t wb = (size_t)out_dim * in_dim * (size_t)(bits == 16 ? 16 : bits) / 8;
    touch(W, wb);
    if (S) touch(S, (size_t)out_dim * (in_dim / group_size) * 2);
    if (B) touch(B, (size_t)out_dim * (in_dim / group_size) * 2);
    return 0;
}
void finch_ops_forget_tensor(const void *W) { (void)W; }
const char *finch_ops_last_error(void) { return ""; }

static int ends_with(const char *s, const char *suf) {
    const size_t n = strlen(s), m = strlen(suf);
    return n >= m && strcmp(s + n - m, suf) == 0;
}

static int run_dense(const char *json_path) {
    char bin[4096];
    snprintf(bin, sizeof bin, "%.*s.bin", (int)(strlen(json_path) - 5), json_path);
    finch_dense *d = finch_ops_open_dense(bin, json_path);
    if (!d) return 0;
    const int n = finch_dense_count(d);
    (void)finch_dense_model(d);
    for (int i = 0; i < n; i++) {
        finch_dense_entry e;
        if (finch_dense_entry_at(d, i, &e)) continue;
        touch(e.data, e.size);
        finch_dense_entry f;
        (void)finch_dense_find(d, e.name, &f);
        const void *W;
        const uint16_t *S, *B;
        int od, id, bits, gs;
        if (finch_dense_quantized(d, e.name, &W, &S, &B, &od, &id, &bits, &gs) == 0) {
            touch(W, (size_t)od * id * bits / 8);
            touch(S, (size_t)od * (id / gs) * 2);
            touch(B, (size_t)od * (id / gs) * 2);
            (void)finch_ops_load_dense_tensor(d, e.name);
        }
    }
    (void)finch_dense_entry_at(d, n, &(finch_dense_entry){0});
    (void)finch_dense_entry_at(d, -1, &(finch_dense_entry){0});
    finch_ops_close_dense(d);
    return 1;
}

static int run_gguf(const char *path) {
    finch_gguf *g = finch_ops_open_gguf(path);
    if (!g) return 0;
    const int n = finch_gguf_count(g);
    (void)finch_gguf_version(g);
    (void)finch_gguf_alignment(g);
    (void)finch_gguf_data_offset(g);
    for (int i = 0; i < n; i++) {
        finch_gguf_tensor t;
        if (finch_gguf_tensor_at(g, i, &t)) continue;
        touch(t.data, t.nbytes);
        finch_gguf_tensor u;
        (void)finch_gguf_find(g, t.name, &u);
    }
    int ne, h, in, types[3];
    (void)finch_gguf_expert_geometry(g, -1, &ne, &h, &in, types);
    for (int l = 0; l < 4; l++) {
        (void)finch_gguf_has_expert_layer(g, l);
        (void)finch_gguf_expert_geometry(g, l, &ne, &h, &in, types);
    }
    (void)finch_ops_load_gguf_experts(g, 4);
    finch_ops_close_gguf(g);
    return 1;
}

static int run_quant(void) {
    enum { OD = 4, ID = 128 };
    static float w[OD * ID];
    static uint8_t packed[OD * ID];
    uint16_t s[OD * ID / 64], b[OD * ID / 64];
    const float specials[] = {NAN, INFINITY, -INFINITY, 3.4e38f, -3.4e38f, 1e-45f, 0.0f, -0.0f};
    const int widths[] = {2, 3, 4, 8};
    unsigned seed = 1;
    int calls = 0;
    for (int bi = 0; bi < 4; bi++)
        for (int t = 0; t < 2000; t++) {
            for (int i = 0; i < OD * ID; i++) {
                seed = seed * 1664525u + 1013904223u;
                w[i] = (float)((int)((seed >> 8) % 2001u) - 1000) / 500.0f;
            }
            for (int k = 0; k < t % 7; k++) {
                seed = seed * 1664525u + 1013904223u;
                w[(seed >> 8) % (OD * ID)] = specials[(seed >> 20) % 8];
            }
            if (t % 11 == 0)
                for (int i = 0; i < 64; i++) w[i] = 1.5f;            /* a constant group: the scale clamps */
            if (finch_quantize_affine_pack(w, OD, ID, 64, widths[bi], packed, s, b) == 0) calls++;
            touch(packed, (size_t)OD * ID * (size_t)widths[bi] / 8);
        }
    printf("done files=%d accepted=%d touched=%lu\n", 8000, calls, g_touched);
    return 0;
}

int main(int argc, char **argv) {
    if (argc != 3) return 2;
    if (strcmp(argv[1], "quant") == 0) return run_quant();
    const int dense = strcmp(argv[1], "dense") == 0;
    DIR *dir = opendir(argv[2]);
    if (!dir) return 2;
    int files = 0, accepted = 0;
    struct dirent *de;
    while ((de = readdir(dir))) {
        if (!ends_with(de->d_name, dense ? ".json" : ".gguf")) continue;
        char path[4096];
        snprintf(path, sizeof path, "%s/%s", argv[2], de->d_name);
        printf("file %s\n", de->d_name);
        fflush(stdout);
        files++;
        accepted += dense ? run_dense(path) : run_gguf(path);
    }
    closedir(dir);
    printf("done files=%d accepted=%d touched=%lu\n", files, accepted, g_touched);
    return 0;
}
