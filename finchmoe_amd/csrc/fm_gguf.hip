// fm_gguf.hip — GGUF Q4_K / Q6_K expert kernels (placeholder launchers until the
// kernels land: every call reports FM_ERR_UNSUPPORTED, nothing falls back).
#include "fm_common.h"

extern "C" int fm_launch_decode_gguf(const uint8_t *const *, const uint8_t *const *,
                                     const uint8_t *const *, const FmGgufGeom *, int, int, int,
                                     const float *, const int32_t *, const float *, int, float *,
                                     float *, float *, unsigned int *, int, int, hipStream_t,
                                     hipEvent_t *) {
    return FM_ERR_UNSUPPORTED;
}
extern "C" int fm_launch_gguf_matvec(const uint8_t *, int, const float *, float *, int, int, int,
                                     hipStream_t) {
    return FM_ERR_UNSUPPORTED;
}
