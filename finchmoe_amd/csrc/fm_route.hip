// fm_route.hip — expert routing on the device: softmax over the gate logits, top-K,
// renormalised weights.  Replaces cpu_softmax / cpu_topk / cpu_normalize_weights
// (finchmoe/infer.m:1794-1840) between the routing GEMVs and the expert launch
// (infer.m:9285-9289), so that indices and weights never leave the device.
//
// The reference's top-K is a sequential scan that overwrites the slot holding the
// smallest kept value whenever a larger score arrives (strict comparisons, lowest
// slot wins among equal minima), so the ORDER of the K slots is part of its result
// and the weighted sum downstream runs in that order.  One wave reproduces the scan
// exactly without visiting every element in sequence: lane k < K holds slot k, the
// wave looks at 64 scores at a time, and only scores above the current minimum —
// found by ballot, taken in index order — cost a slot update (a few dozen per call).
#include "fm_common.h"

namespace {

struct RouteArgs {
    const float *logits;
    int n, K;
    const float *seg_score;      // shared expert's gate score, or null
    int32_t *idx;
    float *w;
    float *params;               // [10] or null: weights, zeros, score at [8]
};

// max / min over the wave's 64 lanes, the result in a scalar register: DPP inside each row
// of 16 lanes, then the four row results read lane by lane (no LDS round trips)
template <bool MAX>
__device__ __forceinline__ float pick(float a, float b) { return MAX ? fmaxf(a, b) : fminf(a, b); }
template <bool MAX>
__device__ __forceinline__ float row_reduce(float v) {
    v = pick<MAX>(v, fm_dpp<0xB1>(v));     // quad_perm [1,0,3,2]
    v = pick<MAX>(v, fm_dpp<0x4E>(v));     // quad_perm [2,3,0,1]
    v = pick<MAX>(v, fm_dpp<0x141>(v));    // row_half_mirror: 8 lanes
    return v;
}
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ float wave_max(float v) {
    v = row_reduce<true>(v);
    v = fmaxf(v, fm_dpp<0x140>(v));        // row_mirror: 16 lanes
    return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}
// min over lanes 0..7 (the K slots; lanes K.. hold +inf)
__device__ __forceinline__ float slots_min(float v) { return lane_value(row_reduce<false>(v), 0); }

#define FM_ROUTE_MAX 4096

__global__ __launch_bounds__(64) void fm_route(RouteArgs a) {
    __shared__ float p[FM_ROUTE_MAX];
    const int lane = threadIdx.x;
    // softmax (infer.m:1794-1808): max, exp, sum, scale
    float mx = -INFINITY;
    for (int i = lane; i < a.n; i += 64) {
        const float v = a.logits[i];
        p[i] = v;
        mx = fmaxf(mx, v);
    }
    mx = wave_max(mx);
    float sum = 0.0f;
    for (int i = lane; i < a.n; i += 64) {
        const float e = expf(p[i] - mx);
        p[i] = e;
        sum += e;
    }
    sum = fm_group_sum<64>(sum);
    const float inv_sum = 1.0f / sum;
    for (int i = lane; i < a.n; i += 64) p[i] *= inv_sum;
    __syncthreads();

    // top-K (infer.m:1810-1831)
    float val = lane < a.K ? -1e30f : INFINITY;    // lanes >= K never hold the minimum
    int ind = 0;
    float min_val = -1e30f;
    int min_k = 0;
    for (int base = 0; base < a.n; base += 64) {
        const int i = base + lane;
        const float s = i < a.n ? p[i] : -INFINITY;
        uint64_t pending = __ballot(s > min_val);
        while (pending) {
            const int src = __ffsll((unsigned long long)pending) - 1;
            const float sv = lane_value(s, src);
            if (lane == min_k) {
                val = sv;
                ind = base + src;
            }
            min_val = slots_min(val);
            min_k = __ffsll((unsigned long long)__ballot(val == min_val)) - 1;
            // scores after src that still beat the new minimum
            const uint64_t later = src == 63 ? 0ull : ~0ull << (src + 1);
            pending = __ballot(s > min_val) & later;
        }
    }
    // renormalise in slot order (infer.m:1833-1840)
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < FM_MAX_K; k++)
        if (k < a.K) total += lane_value(val, k);
    float wk = val;
    if (total > 0.0f) wk = val * (1.0f / total);
    if (lane < a.K) {
        a.idx[lane] = ind;
        a.w[lane] = wk;
    }
    if (a.params && lane < 10) {
        float v = 0.0f;
        if (lane < a.K) v = wk;
        if (lane == 8 && a.seg_score) v = *a.seg_score;
        a.params[lane] = v;
    }
}

}  // namespace

extern "C" int fm_launch_route(const float *d_logits, int n, int K, const float *d_seg_score,
                               int32_t *d_idx, float *d_w, float *d_params, hipStream_t st) {
    if (n < 1 || n > FM_ROUTE_MAX || K < 1 || K > FM_MAX_K || K > n) return FM_ERR_UNSUPPORTED;
    RouteArgs a{d_logits, n, K, d_seg_score, d_idx, d_w, d_params};
    hipLaunchKernelGGL(fm_route, dim3(1), dim3(64), 0, st, a);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}
