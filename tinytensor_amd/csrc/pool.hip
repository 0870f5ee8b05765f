// pool.hip — 2-D max / min / average pooling, forward and backward (gfx950).
//
// Stands where BackendBase::{max,min,avg}_pool2d and their *_backward do
// (tinytensor/tensor/backend_base.h:286-311; CPU form tinytensor/tensor/backend/cpu/conv.cpp:296-426 over the
// kernels of tinytensor/tensor/backend/cpu/kernel/conv.hpp:121-275, functors
// tinytensor/tensor/backend/common/kernel/reduce.hpp:28-140).  Both directions are bandwidth-bound streaming
// kernels: one lane per output element forward, one lane per input element backward.
//
// Forward visits the window in the reference's (p, q) order with the reference's arithmetic
//   max: out = (x > out) ? x : out from lowest();  min: out = (x < out) ? x : out from max();
//   avg: out = (x / n) + out from 0 with n = k*k (padding contributes 0 / n), integer inputs give f32,
// so results are bit-identical.  The input is read through its strides (the reference copies a non-dense input).
//
// Backward is the gather form of the reference's scatter-add: the lane that owns input (y, x) walks the outputs
// whose window contains it in increasing (h, w) — the order in which the reference's loop adds to that
// element — so the sums are bit-identical too, and nothing is written twice (no atomics, no zero-fill pass).
#include "common.h"

#include <cfloat>
#include <climits>
#include <type_traits>

namespace ttamd {
namespace {

enum { POOL_MAX = 0, POOL_MIN = 1, POOL_AVG = 2 };

struct PoolGeom {
    int B, C, H, W, K, S, P, Ho, Wo;
    int64_t xs_b, xs_c, xs_h, xs_w;  // input strides (elements)
};

template <typename R, int OP>
__device__ __forceinline__ R pool_init() {
    if constexpr (OP == POOL_AVG) return R(0);
    else if constexpr (std::is_floating_point_v<R>) {
        constexpr R big = std::is_same_v<R, float> ? R(FLT_MAX) : R(DBL_MAX);
        return OP == POOL_MAX ? -big : big;
    } else if constexpr (std::is_unsigned_v<R>) {
        return OP == POOL_MAX ? R(0) : static_cast<R>(~R(0));
    } else {
        constexpr R lo = static_cast<R>(R(1) << (sizeof(R) * 8 - 1));
        return OP == POOL_MAX ? lo : static_cast<R>(~lo);
    }
}

template <typename T, typename R, int OP>
__global__ void __launch_bounds__(256) pool_forward_kernel(PoolGeom g, const T *__restrict__ x, R *__restrict__ out, int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int w = static_cast<int>(idx % g.Wo);
    const int h = static_cast<int>((idx / g.Wo) % g.Ho);
    const int64_t bc = idx / (static_cast<int64_t>(g.Wo) * g.Ho);
    const int c = static_cast<int>(bc % g.C);
    const int64_t b = bc / g.C;
    const T *plane = x + b * g.xs_b + c * g.xs_c;
    const R n = static_cast<R>(g.K * g.K);
    R acc = pool_init<R, OP>();
    for (int p = 0; p < g.K; ++p) {
        const int hi = g.S * h + p - g.P;
        for (int q = 0; q < g.K; ++q) {
            const int wi = g.S * w + q - g.P;
            const bool in = !(hi < 0 || wi < 0 || hi >= g.H || wi >= g.W);
            const R v = in ? static_cast<R>(plane[hi * g.xs_h + wi * g.xs_w]) : pool_init<R, OP>();
            if constexpr (OP == POOL_MAX) acc = (v > acc) ? v : acc;
            else if constexpr (OP == POOL_MIN) acc = (v < acc) ? v : acc;
            else acc = (v / n) + acc;
        }
    }
    out[idx] = acc;
}

// floor(a / b) for b > 0 and any a
__device__ __forceinline__ int floor_div(int a, int b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

template <typename R, bool SELECT>
__global__ void __launch_bounds__(256)
pool_backward_kernel(PoolGeom g, const R *__restrict__ gout, const R *__restrict__ x, const R *__restrict__ res, R *__restrict__ gin,
                     int64_t total) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int xw = static_cast<int>(idx % g.W);
    const int yh = static_cast<int>((idx / g.W) % g.H);
    const int64_t bc = idx / (static_cast<int64_t>(g.W) * g.H);
    const int c = static_cast<int>(bc % g.C);
    const int64_t b = bc / g.C;
    const R *plane = x + b * g.xs_b + c * g.xs_c;
    const R *gplane = gout + bc * g.Ho * g.Wo;
    const R *rplane = res + bc * g.Ho * g.Wo;
    const R mine = plane[yh * g.xs_h + xw * g.xs_w];
    // outputs h with 0 <= yh + P - S*h < K
    int h_lo = floor_div(yh + g.P - g.K, g.S) + 1, h_hi = floor_div(yh + g.P, g.S);
    int w_lo = floor_div(xw + g.P - g.K, g.S) + 1, w_hi = floor_div(xw + g.P, g.S);
    h_lo = h_lo < 0 ? 0 : h_lo;
    w_lo = w_lo < 0 ? 0 : w_lo;
    h_hi = h_hi >= g.Ho ? g.Ho - 1 : h_hi;
    w_hi = w_hi >= g.Wo ? g.Wo - 1 : w_hi;
    R acc = R(0);
    for (int h = h_lo; h <= h_hi; ++h)
        for (int w = w_lo; w <= w_hi; ++w) {
            const R go = gplane[h * g.Wo + w];
            if constexpr (SELECT) {
                const R target = rplane[h * g.Wo + w];
                if (!(mine == target)) continue;
                R count = R(0);
                for (int p = 0; p < g.K; ++p)
                    for (int q = 0; q < g.K; ++q) {
                        const int hi = g.S * h + p - g.P, wi = g.S * w + q - g.P;
                        const bool in = !(hi < 0 || wi < 0 || hi >= g.H || wi >= g.W);
                        count += (in && plane[hi * g.xs_h + wi * g.xs_w] == target) ? R(1) : R(0);
                    }
                acc += go / count;
            } else {
                acc += go / static_cast<R>(g.K * g.K);
            }
        }
    gin[idx] = acc;
}

ttamd_status make_pool_geom(const char *who, int op, const ttamd_view4 *input, int B, int C, int H, int W, int k, int stride,
                            int padding, PoolGeom *g) {
    if (op < POOL_MAX || op > POOL_AVG) {
        set_error("%s: unknown pooling op code %d", who, op);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (!input) {
        set_error("%s: NULL input view", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (B < 0 || C <= 0 || H <= 0 || W <= 0 || k <= 0 || stride <= 0 || padding < 0) {
        set_error("%s: invalid geometry (B=%d C=%d H=%d W=%d k=%d stride=%d padding=%d)", who, B, C, H, W, k, stride, padding);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (H + 2 * padding < k || W + 2 * padding < k) {
        set_error("%s: kernel %d does not fit the padded input %dx%d", who, k, H + 2 * padding, W + 2 * padding);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    if (input->offset < 0 || input->stride[0] < 0 || input->stride[1] < 0 || input->stride[2] < 0 || input->stride[3] < 0) {
        set_error("%s: negative strides or offset are not supported", who);
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    *g = PoolGeom{};
    g->B = B; g->C = C; g->H = H; g->W = W; g->K = k; g->S = stride; g->P = padding;
    g->Ho = (H + 2 * padding - k) / stride + 1;
    g->Wo = (W + 2 * padding - k) / stride + 1;
    g->xs_b = input->stride[0]; g->xs_c = input->stride[1]; g->xs_h = input->stride[2]; g->xs_w = input->stride[3];
    return TTAMD_OK;
}

template <typename T, typename R, int OP>
ttamd_status launch_forward(const PoolGeom &g, const void *x, void *out, hipStream_t st) {
    const int64_t total = static_cast<int64_t>(g.B) * g.C * g.Ho * g.Wo;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffff) {
        set_error("pool2d: too many workgroups");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    pool_forward_kernel<T, R, OP><<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st>>>(g, static_cast<const T *>(x), static_cast<R *>(out), total);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

template <typename T>
ttamd_status forward_typed(int op, const PoolGeom &g, const void *x, void *out, hipStream_t st) {
    using Avg = std::conditional_t<std::is_floating_point_v<T>, T, float>;
    if (op == POOL_MAX) return launch_forward<T, T, POOL_MAX>(g, x, out, st);
    if (op == POOL_MIN) return launch_forward<T, T, POOL_MIN>(g, x, out, st);
    return launch_forward<T, Avg, POOL_AVG>(g, x, out, st);
}

template <typename R>
ttamd_status backward_typed(int op, const PoolGeom &g, const void *gout, const void *x, const void *res, void *gin, hipStream_t st) {
    const int64_t total = static_cast<int64_t>(g.B) * g.C * g.H * g.W;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7fffffff) {
        set_error("pool2d_backward: too many workgroups");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    if (op == POOL_AVG)
        pool_backward_kernel<R, false><<<grid, block, 0, st>>>(g, static_cast<const R *>(gout), static_cast<const R *>(x),
                                                               static_cast<const R *>(res), static_cast<R *>(gin), total);
    else
        pool_backward_kernel<R, true><<<grid, block, 0, st>>>(g, static_cast<const R *>(gout), static_cast<const R *>(x),
                                                              static_cast<const R *>(res), static_cast<R *>(gin), total);
    TTAMD_HIP_CHECK(hipGetLastError());
    return TTAMD_OK;
}

}  // namespace
}  // namespace ttamd

using namespace ttamd;

extern "C" {

ttamd_status ttamd_pool2d_forward(int device, ttamd_dtype dtype, int op, const ttamd_view4 *input, void *out, int B, int C, int H,
                                  int W, int k, int stride, int padding, void *stream) {
    if (dtype <= TTAMD_BOOL || dtype > TTAMD_F64) {
        set_error("pool2d does not support dtype code %d", static_cast<int>(dtype));
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    PoolGeom g;
    if (ttamd_status s = make_pool_geom("pool2d", op, input, B, C, H, W, k, stride, padding, &g)) return s;
    if (ttamd_status s = use_device(device)) return s;
    if (B == 0) return TTAMD_OK;
    if (!input->data || !out) {
        set_error("pool2d: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const void *x = static_cast<const char *>(input->data) + input->offset * static_cast<int64_t>(dtype_size(dtype));
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case TTAMD_U8: return forward_typed<uint8_t>(op, g, x, out, st);
    case TTAMD_I16: return forward_typed<int16_t>(op, g, x, out, st);
    case TTAMD_I32: return forward_typed<int32_t>(op, g, x, out, st);
    case TTAMD_I64: return forward_typed<int64_t>(op, g, x, out, st);
    case TTAMD_F32: return forward_typed<float>(op, g, x, out, st);
    default: return forward_typed<double>(op, g, x, out, st);
    }
}

ttamd_status ttamd_pool2d_backward(int device, ttamd_dtype dtype, int op, const void *grad_out, const ttamd_view4 *input,
                                   const void *result, void *grad_input, int B, int C, int H, int W, int k, int stride,
                                   int padding, void *stream) {
    if (dtype != TTAMD_F32 && dtype != TTAMD_F64) {
        set_error("pool2d_backward supports f32 and f64 only (autograd never differentiates integer tensors)");
        return TTAMD_ERR_UNSUPPORTED_DTYPE;
    }
    PoolGeom g;
    if (ttamd_status s = make_pool_geom("pool2d_backward", op, input, B, C, H, W, k, stride, padding, &g)) return s;
    if (ttamd_status s = use_device(device)) return s;
    if (B == 0) return TTAMD_OK;
    if (!input->data || !grad_out || !result || !grad_input) {
        set_error("pool2d_backward: NULL data pointer");
        return TTAMD_ERR_INVALID_ARGUMENT;
    }
    const void *x = static_cast<const char *>(input->data) + input->offset * static_cast<int64_t>(dtype_size(dtype));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == TTAMD_F32) return backward_typed<float>(op, g, grad_out, x, result, grad_input, st);
    return backward_typed<double>(op, g, grad_out, x, result, grad_input, st);
}

}  // extern "C"
