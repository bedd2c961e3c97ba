// Temporary: entry points that are declared but not built yet report TMQ_ERR_UNSUPPORTED.
#include "tmq_hip.h"
extern "C" {
int tmq_conv2d_out_hw(const tmq_conv_shape *s, int32_t *ho, int32_t *wo) {
    if (!s || !ho || !wo || s->sy <= 0 || s->sx <= 0) return TMQ_ERR_INVALID_ARG;
    *ho = (s->H + 2 * s->py - s->dy * (s->ky - 1) - 1) / s->sy + 1;
    *wo = (s->W + 2 * s->px - s->dx * (s->kx - 1) - 1) / s->sx + 1;
    return TMQ_OK;
}
int tmq_ternary_conv2d(const void *, int, const tmq_conv_shape *, const uint32_t *, const float *, const float *,
                       const void *, int, void *, int, void *) { return TMQ_ERR_UNSUPPORTED; }
}
