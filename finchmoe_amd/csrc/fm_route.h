// fm_route.h — the routing of one token as a device function of ONE wave (see fm_route.hip),
// so that the kernel that produces the gate logits can run it in its last workgroup.
#pragma once

#include "fm_common.h"

#if defined(__HIPCC__)

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

// p: FM_ROUTE_MAX floats of LDS.  SHARED: the logits (and the shared expert's score) were
// written earlier in this launch by other workgroups and are read at device scope.
template <bool SHARED>
__device__ __forceinline__ void fm_route_wave(const RouteArgs &a, float *p) {
    const int lane = threadIdx.x & 63;
    // softmax (infer.m:1794-1808): max, exp, sum, scale
    float mx = -INFINITY;
    for (int i = lane; i < a.n; i += 64) {
        const float v = SHARED ? __hip_atomic_load(a.logits + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : a.logits[i];
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
    // one wave: its LDS instructions execute in order, no workgroup barrier is needed (and
    // none may be used: inside another kernel only this wave is here)
    __builtin_amdgcn_wave_barrier();

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
        if (lane == 8 && a.seg_score)
            v = SHARED ? __hip_atomic_load(a.seg_score, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *a.seg_score;
        a.params[lane] = v;
    }
}

#endif
