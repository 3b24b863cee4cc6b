// fm_prefill.hip — grouped chunked-prefill expert GEMM (placeholder: reports no
// workspace, so the caller runs the per-position path).
#include "fm_common.h"

extern "C" size_t fm_prefill_affine_ws_bytes(const FmExpertGeom *, int, int) { return 0; }
extern "C" int fm_launch_prefill_affine(const uint8_t *, const FmExpertGeom *, const float *,
                                        const int32_t *, const float *, int, int, float *, void *,
                                        size_t, int, int, hipStream_t) {
    return FM_ERR_UNSUPPORTED;
}
