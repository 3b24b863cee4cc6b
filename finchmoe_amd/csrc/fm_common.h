// fm_common.h — shared declarations of libfinchhip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/finch_hip.h"

#define FM_MAX_K 8
#define FM_WAVE 64

// Geometry of one affine expert blob, passed to kernels by value.
// Layout: finchmoe/repack_experts.py:76-163, finchmoe/infer.m:174-234.
struct FmExpertGeom {
    int hidden, inter, group_size, bits, scale_fp16, n_experts;
    uint32_t gate_w, gate_s, gate_b, up_w, up_s, up_b, down_w, down_s, down_b;
    uint64_t expert_size;
};

// Host-side state of the dependency counters of the fused decode kernel: two
// sets of `cap` counters that alternate between launches (a launch counts in
// set[parity] and clears the used[parity ^ 1] entries the launch before it left
// in the other set), and the device word a timed-out wait raises.  A launch that is being
// captured into a graph is replayed without the host code that alternates the sets: it counts
// in `graph_set`, which a fill kernel recorded in front of it clears on every replay.
struct FmDecodeFlags {
    unsigned int *set[2];
    unsigned int *graph_set;
    unsigned int used[2];
    unsigned int cap;
    int parity;
    unsigned int *err;
    unsigned int spin_limit;
    int always_graph_set;   // count in graph_set behind a clearing kernel even when not capturing
    // Activation sets of the launch form that keeps the per-expert vectors in LDS
    // (fm_moe_fused_rows): elements not yet produced hold a marker, so a set must be all
    // markers when a launch starts.  Two sets alternate like the counters (a launch fills
    // act_set[act_parity] and re-marks the act_used[act_parity ^ 1] floats the launch before it
    // filled); act_graph belongs to captured launches, re-marked by a kernel recorded in front.
    float *act_set[2];
    float *act_graph;
    unsigned int act_used[2];
    unsigned int act_cap;   // floats per set; 0: this launch form is not available
    int act_parity;
};

// What an element of an activation set holds until its producer has stored it (a NaN that no
// arithmetic yields), and the part of a launch's arguments that concerns the sets.
#define FM_ACT_EMPTY 0xFFC5A3E1u
struct Fm2Sync {
    float *act_other;        // the activation set of the previous and of the next launch
    unsigned int clear_n;    // floats of it to mark empty
    unsigned int *err;       // host memory
    unsigned int spin_limit;
};

// internal launch flag (above the public FM_* bits): the caller has no use for the per-expert
// vectors
#define FM_INT_NO_EXPERT_OUT (1 << 16)

// One tensor of a dense GEMV launch (fm_dense.hip).
struct FmDenseSpec {
    const uint8_t *W, *S, *B;
    float *out;
    int out_dim;
    int first_item;   // first workgroup of this tensor
    int bits;         // code width (read by the launch of tensors of different widths only)
};

// Geometry of the GGUF slabs of one layer (finchmoe/infer.m:1017-1022).
struct FmGgufGeom {
    int hidden, inter, n_experts;
    int gate_type, up_type, down_type;
    uint64_t gate_slab, up_slab, down_slab;   // bytes per expert
    uint32_t gu_row_bytes, down_row_bytes;
};

// Operands of the layer tail (fm_tail.hip): shared expert's down projection W/S/B
// [hidden][inter], the vectors it combines, and the scratch of the norm's reduction.
struct FmTailArgs {
    const uint8_t *W, *S, *B;
    int hidden, inter, K;
    const float *h_mid, *expert_out, *params, *shared_gate, *shared_up;
    const uint16_t *norm_w;
    float eps;
    float *hidden_out, *next_in;
    float *partial;
    unsigned int *counter;
    int scale_fp16;          // scale type of W's groups (the launch with the experts in front only)
    // the launch with the experts in front, optionally: the token's routing at its start (every
    // workgroup runs it on the gate logits a launch before it left in memory) instead of expert
    // indices and weights handed in; the results also go to route_idx / route_w / route_params
    const float *route_logits;
    int route_n;
    const float *route_seg;
    int32_t *route_idx;
    float *route_w, *route_params;
};

// ---------------------------------------------------------------- device helpers
#if defined(__HIPCC__)

// 16-bit scale / bias widening.  BF16: finchmoe/infer.m:690-695.
// FP16: IEEE half -> float (finchmoe/infer.m:1579-1593 computes the same value).
__device__ __forceinline__ float fm_bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float fm_bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xFFFF0000u); }
__device__ __forceinline__ float fm_fp16_bits(uint32_t h) {
    _Float16 v = __builtin_bit_cast(_Float16, (unsigned short)h);
    return (float)v;
}
template <bool FP16>
__device__ __forceinline__ float fm_widen_lo(uint32_t pair) {
    if constexpr (FP16) return fm_fp16_bits(pair & 0xFFFFu);
    else return fm_bf16_lo(pair);
}
template <bool FP16>
__device__ __forceinline__ float fm_widen_hi(uint32_t pair) {
    if constexpr (FP16) return fm_fp16_bits(pair >> 16);
    else return fm_bf16_hi(pair);
}

// Sum over aligned groups of N lanes (N a power of two <= 64); every lane of
// the group receives the sum.  N <= 16 stays inside a DPP row.
template <int CTRL>
__device__ __forceinline__ float fm_dpp(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
template <int N>
__device__ __forceinline__ float fm_group_sum(float v) {
    if constexpr (N >= 2) v += fm_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
    if constexpr (N >= 4) v += fm_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
    // once every lane of a quad holds the quad's sum, mirroring within 8 (then
    // 16) lanes fetches the neighbouring quad's (half row's) sum
    if constexpr (N >= 8) v += fm_dpp<0x141>(v);   // row_half_mirror
    if constexpr (N >= 16) v += fm_dpp<0x140>(v);  // row_mirror
    if constexpr (N >= 32) v += __shfl_xor(v, 16);
    if constexpr (N >= 64) v += __shfl_xor(v, 32);
    return v;
}

__device__ __forceinline__ float fm_silu_mul(float g, float u) {
    return (g / (1.0f + expf(-g))) * u;   // finchmoe/infer.m:1780-1786
}

#endif  // __HIPCC__

// Which form of a kernel the launchers pick where two exist (fm_set_kernel_forms): 0 = the
// default choice.  Process-wide; read by the launchers on the host only.
extern unsigned int fm_kernel_forms;
