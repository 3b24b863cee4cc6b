/*
 * finch_files.h — the reference's weight files and its quantizer in C, beside the operator
 * layer of finch_ops.h (same library, libfinchops.so).
 *
 *   quantizer        finchmoe/repack_experts.py:232-333, finchmoe/quantize_model.py:13-47,
 *                    finchmoe/quantize_non_experts.py:30-69 (one arithmetic, three packings)
 *   expert files     packed_experts*\/layer_%02d.bin, finchmoe/infer.m:15405-15440
 *   dense weights    model_weights_quant.bin + .json, finchmoe/infer.m:727-786
 *   GGUF             finchmoe/infer.m:1017-1250
 *
 * Files are mapped read-only and handed to the upload calls in place.  Nothing here needs a
 * GPU except the three finch_ops_load_* calls, which upload through the context of
 * finch_ops_init().  Every function returns 0 / a valid handle on success; on failure it
 * returns a negative FM_ERR_* code or NULL and finch_files_last_error() names the cause.
 */
#ifndef FINCH_FILES_H
#define FINCH_FILES_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *finch_files_last_error(void);

/* ---- quantizer ------------------------------------------------------------------------ */
/* Group-wise affine quantisation of w [out_dim][in_dim] (fp32, row-major) to `bits` in
 * {2,3,4,8} with groups of `group_size` along in_dim:
 *   scale = max((max - min) / (2^bits - 1), 1e-8), bias = min, q = clip(round_half_even((w - bias) / scale))
 * in fp32, then scale and bias cut to BF16 by truncation — the codes come from the fp32 values,
 * as in the reference.  packed: bits 3 -> byte triplets of 8 codes (pack_3bit,
 * repack_experts.py:242-257), in_dim*3/8 bytes a row; otherwise LSB-first fields of
 * little-endian u32 words (quantize_model.py:35-43), in_dim*bits/8 bytes a row.
 * scales, biases: [out_dim][in_dim/group_size] BF16 bits. */
int finch_quantize_affine_pack(const float *w, int out_dim, int in_dim, int group_size, int bits,
                               void *packed, uint16_t *scales, uint16_t *biases);
/* bytes of one expert in a layer file: gate, up, down, each as packed|scales|biases
 * (repack_experts.py:336-392); 0 if the geometry is not representable */
size_t finch_expert_blob_size(int hidden, int inter, int group_size, int bits);
/* quantise one expert's three fp32 matrices (gate, up [inter][hidden]; down [hidden][inter])
 * into its blob */
int finch_quantize_expert(const float *gate, const float *up, const float *down, int hidden,
                          int inter, int group_size, int bits, void *blob);

/* ---- mappings ---------------------------------------------------------------------------- */
/* A whole file mapped read-only (for upload calls that take host pointers); an empty file is
 * an error. */
int finch_file_map(const char *path, const void **data, size_t *nbytes);
void finch_file_unmap(const void *data, size_t nbytes);

/* ---- expert layer files ---------------------------------------------------------------- */
/* Path of a layer file, as the reference builds it (infer.m:15412). */
int finch_expert_layer_path(const char *dir, int layer, char *out, size_t out_size);
/* Map `dir`/layer_%02d.bin for layers [0, n_layers) and upload each; the store must have been
 * configured (finch_ops_config_experts).  A missing file is skipped, as in the reference
 * (infer.m:15427-15430); a file of the wrong size is an error.  Returns the number of layers
 * loaded, or a negative code. */
int finch_ops_load_expert_dir(const char *dir, int n_layers);

/* ---- model_weights_quant.bin + manifest ------------------------------------------------ */
typedef struct finch_dense finch_dense;

typedef struct {
    const char *name;      /* owned by the handle */
    const void *data;      /* inside the mapping */
    uint64_t offset;       /* of data in the .bin file */
    size_t size;
    int ndim;
    int64_t shape[4];
    char dtype[8];         /* "U32", "BF16", "F32", ... */
    int bits, group_size;  /* 0 when the manifest has none */
} finch_dense_entry;

/* json_path NULL: bin_path with its extension replaced by ".json" */
finch_dense *finch_ops_open_dense(const char *bin_path, const char *json_path);
void finch_ops_close_dense(finch_dense *d);
int finch_dense_count(const finch_dense *d);
const char *finch_dense_model(const finch_dense *d);      /* the manifest's "model", or NULL */
int finch_dense_entry_at(const finch_dense *d, int i, finch_dense_entry *out);
int finch_dense_find(const finch_dense *d, const char *name, finch_dense_entry *out);
/* The three entries of a quantized tensor from its NAME.weight entry: W (U32), NAME.scales,
 * NAME.biases; in_dim = packed columns * 32 / bits. */
int finch_dense_quantized(const finch_dense *d, const char *weight_name, const void **W,
                          const uint16_t **S, const uint16_t **B, int *out_dim, int *in_dim,
                          int *bits, int *group_size);
/* Upload one tensor now (instead of on its first use by fast_dequant_matvec). */
int finch_ops_load_dense_tensor(const finch_dense *d, const char *weight_name);

/* ---- GGUF ------------------------------------------------------------------------------ */
typedef struct finch_gguf finch_gguf;

typedef struct {
    const char *name;      /* owned by the handle */
    int type;              /* ggml type */
    int ndim;
    uint64_t dims[4];      /* as stored: [in, out, experts] for the stacked tensors */
    const void *data;
    size_t nbytes;
} finch_gguf_tensor;

finch_gguf *finch_ops_open_gguf(const char *path);
void finch_ops_close_gguf(finch_gguf *g);
int finch_gguf_version(const finch_gguf *g);
int finch_gguf_alignment(const finch_gguf *g);
uint64_t finch_gguf_data_offset(const finch_gguf *g);
int finch_gguf_count(const finch_gguf *g);
int finch_gguf_tensor_at(const finch_gguf *g, int i, finch_gguf_tensor *out);
int finch_gguf_find(const finch_gguf *g, const char *name, finch_gguf_tensor *out);
/* (elements, bytes) of a block of a ggml type; 0 for a type this library does not read */
int finch_ggml_block(int type, int *elems, int *bytes);
/* Geometry of blk.<layer>.ffn_{gate,up,down}_exps.weight, dims [in, out, experts]
 * (infer.m:1138-1146); layer < 0: the lowest layer that has all three. */
int finch_gguf_expert_geometry(const finch_gguf *g, int layer, int *n_experts, int *hidden,
                               int *inter, int types[3]);
/* 1 if the layer has all three stacked expert tensors */
int finch_gguf_has_expert_layer(const finch_gguf *g, int layer);
/* Upload every layer in [0, n_layers) that has its expert tensors; the GGUF store must have been
 * configured (finch_ops_config_gguf_experts).  Returns the number of layers loaded. */
int finch_ops_load_gguf_experts(const finch_gguf *g, int n_layers);

#ifdef __cplusplus
}
#endif
#endif
