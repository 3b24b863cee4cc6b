// fm_tail.hip — what the reference appends to a layer's expert command buffer
// after the routed experts (finchmoe/infer.m:9608-9760), in one launch:
//   shared expert   act = SwiGLU(shared_gate, shared_up)          (shaders.metal:1056-1068)
//                   shared_out = down_proj(act), affine 4-bit      (infer.m:9629-9634)
//   combine         hidden = h_mid + sum_k params[k] * expert_out[k]   (or the sum, ready-made)
//                            + sigmoid(params[8]) * shared_out     (shaders.metal:2196-2231)
//   next input      rms_norm(hidden) * bf16 weights of the next layer's input norm
//                                                                  (shaders.metal:1134-1205)
// — five dispatches there.  The down projection is a [hidden, shared_inter] GEMV
// (0.56 MB at 2048 x 512): one workgroup of four waves per 4 * 64/LPR rows, same
// lane map and vector-ALU unpack as fm_dense_gemv.  The norm needs sum(hidden^2)
// over all rows: every workgroup leaves its partial sum in memory and takes a
// ticket; the one that draws the last ticket adds the partials in workgroup
// order (so the result does not depend on which one that is) and writes the
// normalised vector.  Nothing waits for anything.
#include "fm_unpack.h"

namespace {

__device__ __forceinline__ void tail_st(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float tail_ld(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int BITS, int LPR, bool FP16>
__global__ __launch_bounds__(256) void fm_layer_tail(FmTailArgs a) {
    constexpr int RPS = FM_WAVE / LPR;
    constexpr int BPL = FmLaneBytes<BITS>::value;
    extern __shared__ __attribute__((aligned(16))) float tail_act[];   // [inter]
    __shared__ float red[4];
    __shared__ unsigned int ticket;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = lane % LPR, r = lane / LPR;
    const int row = (blockIdx.x * 4 + wave) * RPS + r;
    const int row_bytes = a.inter * BITS / 8, sb_row_bytes = (a.inter / 64) * 2;

    // everything that depends on nothing is fetched first, so that the loads overlap: the
    // row's codes, and what the combine adds to the row (all lanes of a row load the same)
    FmRowSlice<BITS> ws;
    fm_load_slice<BITS>(ws, a.W + (size_t)row * row_bytes + (size_t)c * BPL,
                        a.S + (size_t)row * sb_row_bytes + (size_t)c * 4,
                        a.B + (size_t)row * sb_row_bytes + (size_t)c * 4);
    float eo[FM_MAX_K], pw[FM_MAX_K];
#pragma unroll
    for (int k = 0; k < FM_MAX_K; k++) {
        eo[k] = k < a.K ? a.expert_out[(size_t)k * a.hidden + row] : 0.0f;
        pw[k] = k < a.K ? a.params[k] : 0.0f;
    }
    // K == 0 with a vector: the routed experts' sum is there already (fm_moe_decode_dev without
    // a buffer for the per-expert vectors adds them up in the same slot order)
    const float pre = (a.K == 0 && a.expert_out) ? a.expert_out[row] : 0.0f;
    const float hm = a.h_mid[row], score = a.params[8];
    for (int j = threadIdx.x; j < a.inter; j += blockDim.x)
        tail_act[j] = fm_silu_mul(a.shared_gate[j], a.shared_up[j]);
    __syncthreads();
    float xs[FM_CPL], xsum0, xsum1;
    fm_load_x<BITS>(tail_act + c * FM_CPL, xs, xsum0, xsum1);
    const float shared_out = fm_group_sum<LPR>(fm_lane_dot<BITS, FP16>(ws, xs, xsum0, xsum1));

    float sq = 0.0f;
    if (c == 0) {
        float moe = pre;
#pragma unroll
        for (int k = 0; k < FM_MAX_K; k++)
            if (k < a.K) moe += pw[k] * eo[k];
        const float shared_gate = 1.0f / (1.0f + expf(-score));
        const float hv = hm + moe + shared_gate * shared_out;
        tail_st(a.hidden_out + row, hv);
        sq = hv * hv;
    }
    if (!a.next_in) return;

    sq = fm_group_sum<64>(sq);
    if (lane == 0) red[wave] = sq;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // this wave's rows are in memory
    __syncthreads();
    if (threadIdx.x == 0) {
        tail_st(a.partial + blockIdx.x, ((red[0] + red[1]) + red[2]) + red[3]);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        ticket = __hip_atomic_fetch_add(a.counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (ticket != gridDim.x - 1) return;
    // The loads below read what other workgroups stored before they drew their tickets.  They
    // are relaxed device-scope accesses, which the compiler may move: keep them behind the
    // ticket (the hardware side: a device-scope store that has left the wave under vmcnt(0)
    // has been performed at the memory side of the L2s, where device-scope loads look).
    __atomic_signal_fence(__ATOMIC_ACQUIRE);

    // last workgroup: every other one has stored its rows and its partial sum.  The partials
    // are fetched side by side and added in workgroup order.
    __shared__ float parts[1024];
    for (unsigned int i = threadIdx.x; i < gridDim.x; i += blockDim.x) parts[i] = tail_ld(a.partial + i);
    __syncthreads();
    float sum_sq = 0.0f;
    for (unsigned int i = 0; i < gridDim.x; i++) sum_sq += parts[i];
    const float inv_rms = 1.0f / sqrtf(sum_sq / (float)a.hidden + a.eps);   // infer.m:1771-1772
    for (int j = threadIdx.x; j < a.hidden; j += blockDim.x)
        a.next_in[j] = tail_ld(a.hidden_out + j) * inv_rms * __uint_as_float((uint32_t)a.norm_w[j] << 16);
    if (threadIdx.x == 0)
        __hip_atomic_store(a.counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int BITS, bool FP16>
int launch_tail_t(const FmTailArgs &a, hipStream_t st) {
    const int lpr = a.inter / FM_CPL;
    const size_t sh = (size_t)a.inter * sizeof(float);
#define FM_T(L)                                                                                  \
    do {                                                                                         \
        const int rows = 4 * (FM_WAVE / L);                                                      \
        if (a.hidden % rows || a.hidden / rows > 1024) return FM_ERR_UNSUPPORTED;                \
        hipLaunchKernelGGL((fm_layer_tail<BITS, L, FP16>), dim3(a.hidden / rows), dim3(256), sh, \
                           st, a);                                                               \
    } while (0)
    switch (lpr) {
        case 1: FM_T(1); break;
        case 2: FM_T(2); break;
        case 4: FM_T(4); break;
        case 8: FM_T(8); break;
        case 16: FM_T(16); break;
        default: return FM_ERR_UNSUPPORTED;
    }
#undef FM_T
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}

}  // namespace

// a.partial must hold hidden / 4 floats at least (one per workgroup), *a.counter is 0
// between launches
extern "C" int fm_launch_layer_tail(const FmTailArgs *a, int bits, int scale_fp16, hipStream_t st) {
    if (a->inter % FM_CPL || a->inter > 2048 || a->K < 0 || a->K > FM_MAX_K) return FM_ERR_UNSUPPORTED;
    switch (bits) {
        case 3: return scale_fp16 ? launch_tail_t<3, true>(*a, st) : launch_tail_t<3, false>(*a, st);
        case 4: return scale_fp16 ? launch_tail_t<4, true>(*a, st) : launch_tail_t<4, false>(*a, st);
        case 8: return scale_fp16 ? launch_tail_t<8, true>(*a, st) : launch_tail_t<8, false>(*a, st);
        default: return FM_ERR_UNSUPPORTED;
    }
}
