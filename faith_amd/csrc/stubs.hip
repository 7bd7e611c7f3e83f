// Placeholders until the contraction kernels land.
#include "common.h"
extern "C" int faith_dot_product_verification_QK(float *, float *, float *, float *, const float *, const float *,
                                                 const float *, const float *, const float *, const float *,
                                                 const float *, const float *, float *, float *, float *, float *,
                                                 int, int, int, int, int, float, int, int, void *) {
    faith::set_error("faith_dot_product_verification_QK: not built yet");
    return FAITH_ERR_UNSUPPORTED;
}
extern "C" int faith_convolution_verification(const float *, const float *, const float *, const float *,
                                              const float *, const float *, float *, float *, float *, float *, int,
                                              int, int, int, int, int, int, int, int, void *) {
    faith::set_error("faith_convolution_verification: not built yet");
    return FAITH_ERR_UNSUPPORTED;
}
