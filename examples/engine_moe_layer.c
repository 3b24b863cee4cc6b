/* The MoE half of one layer as the reference's C core calls it (finchmoe/infer.m:9285-9289 routing,
 * 9556-9738 experts), written against include/finch_ops.h and include/finch_files.h: what a
 * maintainer's call sites look like once the static Metal-backed functions are replaced by
 * libfinchops.so.  Not part of the library; tests/test_cabi.py compiles and links it so that the
 * headers stay self-contained C99 and every name used here stays exported.
 *
 *   gcc -std=c99 -Iinclude examples/engine_moe_layer.c -Lfinchmoe_amd -lfinchops -lfinchhip -lm
 *
 * usage: engine_moe_layer <model dir with packed_experts_3bit/ and model_weights_quant.{bin,json}> */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "finch_files.h"
#include "finch_ops.h"

enum { NUM_LAYERS = 40, NUM_EXPERTS = 256, HIDDEN_DIM = 2048, MOE_INTERMEDIATE = 512, K = 8, GROUP_SIZE = 64 };

static void die(const char *what) {
    fprintf(stderr, "%s: %s / %s\n", what, finch_ops_last_error(), finch_files_last_error());
    exit(1);
}

int main(int argc, char **argv) {
    if (argc != 2) return 2;
    char path[1024], json[1024];
    if (finch_ops_init(0)) die("finch_ops_init");                       /* was: metal_setup() */

    /* experts: resident once instead of pread per token (infer.m:9556, 15405-15440) */
    if (finch_ops_config_experts(NUM_LAYERS, NUM_EXPERTS, HIDDEN_DIM, MOE_INTERMEDIATE, 3)) die("config");
    snprintf(path, sizeof path, "%s/packed_experts_3bit", argv[1]);
    const int loaded = finch_ops_load_expert_dir(path, NUM_LAYERS);
    if (loaded < 0) die("expert files");
    fprintf(stderr, "%d expert layers resident\n", loaded);

    /* non-expert tensors: the manifest and its data file (infer.m:727-786) */
    snprintf(path, sizeof path, "%s/model_weights_quant.bin", argv[1]);
    snprintf(json, sizeof json, "%s/model_weights_quant.json", argv[1]);
    finch_dense *wf = finch_ops_open_dense(path, json);
    if (!wf) die("manifest");
    const void *gate_w;
    const uint16_t *gate_s, *gate_b;
    int out_dim, in_dim, bits, gs;
    if (finch_dense_quantized(wf, "model.layers.0.mlp.gate.weight", &gate_w, &gate_s, &gate_b, &out_dim,
                              &in_dim, &bits, &gs))
        die("mlp.gate");

    /* one token through the MoE half of layer 0: call sites as in fused_layer_forward */
    static float h_post[HIDDEN_DIM], gate_scores[NUM_EXPERTS], moe_out[HIDDEN_DIM], expert_weights[K];
    int expert_indices[K];
    for (int i = 0; i < HIDDEN_DIM; i++) h_post[i] = (float)((i * 37) % 17 - 8) / 8.0f;
    fast_dequant_matvec((const uint32_t *)gate_w, gate_s, gate_b, h_post, gate_scores, out_dim, in_dim,
                        gs, bits);                                       /* infer.m:3369 */
    if (finch_ops_last_status()) die("gate matvec");
    cpu_softmax(gate_scores, NUM_EXPERTS);                               /* infer.m:9285-9289 */
    cpu_topk(gate_scores, NUM_EXPERTS, K, expert_indices, expert_weights);
    cpu_normalize_weights(expert_weights, K);
    memset(moe_out, 0, sizeof moe_out);
    if (!moe_experts_forward(0, h_post, expert_indices, expert_weights, K, moe_out))   /* infer.m:10109-10204 */
        die("experts");
    printf("moe_out[0..3] = %g %g %g %g\n", moe_out[0], moe_out[1], moe_out[2], moe_out[3]);

    finch_ops_close_dense(wf);
    finch_ops_shutdown();
    return 0;
}
