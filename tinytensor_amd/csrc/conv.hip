// conv.hip — conv2d forward/backward as implicit GEMM (placeholder entry points while the kernels land).
#include "common.h"
using namespace ttamd;
extern "C" {
ttamd_status ttamd_conv2d_forward(int, ttamd_dtype, const ttamd_view4 *, const ttamd_view4 *, const void *, void *, int,
                                  int, int, int, int, int, int, int, void *) {
    set_error("conv2d_forward: not implemented yet");
    return TTAMD_ERR_INVALID_ARGUMENT;
}
ttamd_status ttamd_conv2d_backward_workspace(ttamd_dtype, int, int, int, int, int, int, int, int, size_t *bytes) {
    if (bytes) *bytes = 0;
    return TTAMD_OK;
}
ttamd_status ttamd_conv2d_backward(int, ttamd_dtype, const void *, const ttamd_view4 *, const ttamd_view4 *, void *,
                                   void *, void *, int, int, int, int, int, int, int, int, void *, size_t, void *) {
    set_error("conv2d_backward: not implemented yet");
    return TTAMD_ERR_INVALID_ARGUMENT;
}
}
