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
#include "fm_route.h"

namespace {

__global__ __launch_bounds__(64) void fm_route(RouteArgs a) {
    __shared__ float p[FM_ROUTE_MAX];
    fm_route_wave<false>(a, p);
}

}  // namespace

extern "C" int fm_launch_route(const float *d_logits, int n, int K, const float *d_seg_score,
                               int32_t *d_idx, float *d_w, float *d_params, hipStream_t st) {
    if (n < 1 || n > FM_ROUTE_MAX || K < 1 || K > FM_MAX_K || K > n) return FM_ERR_UNSUPPORTED;
    RouteArgs a{d_logits, n, K, d_seg_score, d_idx, d_w, d_params};
    hipLaunchKernelGGL(fm_route, dim3(1), dim3(64), 0, st, a);
    return hipGetLastError() == hipSuccess ? FM_OK : FM_ERR_HIP;
}
