/*
 * tt_oracle_pool.c — CPU restatement of tinytensor's 2-D pooling (plain C).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP pooling kernels; never linked into the product.
 *
 * Follows tinytensor/tensor/backend/cpu/kernel/conv.hpp:121-275 (pool_kernel and the two
 * pool_backward_kernel overloads), driven as tinytensor/tensor/backend/cpu/conv.cpp:296-426 drives them,
 * with the reduction functors of tinytensor/tensor/backend/common/kernel/reduce.hpp:28-140:
 *   max:  out = (x > out) ? x : out,  padding = lowest();   min: out = (x < out) ? x : out, padding = max()
 *   avg:  out = (x / n) + out with n = k*k, padding = 0, result type float for integer inputs
 *         (tinytensor/tensor/backend/common/reduce.h:63-69)
 * Backward (floating types): the gradient of an output is divided by the number of in-bounds window elements
 * equal to the result (max/min) or by k*k (avg) and added to those elements, outputs visited in (h, w) order.
 */
#include "tt_oracle.h"

#include <float.h>
#include <limits.h>
#include <string.h>

#define POOL_FORWARD(NAME, T, R, INIT, COMBINE)                                                                   \
    static void NAME(const T *X, R *res, int B, int C, int H, int W, int K, int S, int P) {                        \
        const int Ho = (H + 2 * P - K) / S + 1, Wo = (W + 2 * P - K) / S + 1;                                      \
        const R n = (R)(K * K);                                                                                    \
        (void)n;                                                                                                   \
        for (int b = 0; b < B; ++b)                                                                                \
            for (int c = 0; c < C; ++c)                                                                            \
                for (int h = 0; h < Ho; ++h)                                                                       \
                    for (int w = 0; w < Wo; ++w) {                                                                 \
                        R out = (INIT);                                                                            \
                        for (int p = 0; p < K; ++p)                                                                \
                            for (int q = 0; q < K; ++q) {                                                          \
                                const int hi = S * h + p - P, wi = S * w + q - P;                                  \
                                const R x = (hi < 0 || wi < 0 || hi >= H || wi >= W)                               \
                                                ? (INIT)                                                           \
                                                : (R)X[((size_t)(b * C + c) * H + hi) * W + wi];                   \
                                out = COMBINE;                                                                     \
                            }                                                                                      \
                        res[((size_t)(b * C + c) * Ho + h) * Wo + w] = out;                                        \
                    }                                                                                              \
    }

#define MAX_OF ((x > out) ? x : out)
#define MIN_OF ((x < out) ? x : out)
#define AVG_OF ((x / n) + out)

POOL_FORWARD(pool_max_f32, float, float, -FLT_MAX, MAX_OF)
POOL_FORWARD(pool_max_f64, double, double, -DBL_MAX, MAX_OF)
POOL_FORWARD(pool_max_u8, uint8_t, uint8_t, 0, MAX_OF)
POOL_FORWARD(pool_max_i16, int16_t, int16_t, INT16_MIN, MAX_OF)
POOL_FORWARD(pool_max_i32, int32_t, int32_t, INT32_MIN, MAX_OF)
POOL_FORWARD(pool_max_i64, int64_t, int64_t, INT64_MIN, MAX_OF)
POOL_FORWARD(pool_min_f32, float, float, FLT_MAX, MIN_OF)
POOL_FORWARD(pool_min_f64, double, double, DBL_MAX, MIN_OF)
POOL_FORWARD(pool_min_u8, uint8_t, uint8_t, UINT8_MAX, MIN_OF)
POOL_FORWARD(pool_min_i16, int16_t, int16_t, INT16_MAX, MIN_OF)
POOL_FORWARD(pool_min_i32, int32_t, int32_t, INT32_MAX, MIN_OF)
POOL_FORWARD(pool_min_i64, int64_t, int64_t, INT64_MAX, MIN_OF)
POOL_FORWARD(pool_avg_f32, float, float, 0, AVG_OF)
POOL_FORWARD(pool_avg_f64, double, double, 0, AVG_OF)
POOL_FORWARD(pool_avg_u8, uint8_t, float, 0, AVG_OF)
POOL_FORWARD(pool_avg_i16, int16_t, float, 0, AVG_OF)
POOL_FORWARD(pool_avg_i32, int32_t, float, 0, AVG_OF)
POOL_FORWARD(pool_avg_i64, int64_t, float, 0, AVG_OF)

int tto_pool2d_forward(int dtype, int op, const void *input, void *out, int B, int C, int H, int W, int k, int stride,
                       int padding) {
#define CASE(OPN, DT, SUF, T, R)                                                           \
    if (op == OPN && dtype == DT) {                                                        \
        pool_##SUF((const T *)input, (R *)out, B, C, H, W, k, stride, padding);            \
        return 0;                                                                          \
    }
    CASE(0, TTO_F32, max_f32, float, float)
    CASE(0, TTO_F64, max_f64, double, double)
    CASE(0, TTO_U8, max_u8, uint8_t, uint8_t)
    CASE(0, TTO_I16, max_i16, int16_t, int16_t)
    CASE(0, TTO_I32, max_i32, int32_t, int32_t)
    CASE(0, TTO_I64, max_i64, int64_t, int64_t)
    CASE(1, TTO_F32, min_f32, float, float)
    CASE(1, TTO_F64, min_f64, double, double)
    CASE(1, TTO_U8, min_u8, uint8_t, uint8_t)
    CASE(1, TTO_I16, min_i16, int16_t, int16_t)
    CASE(1, TTO_I32, min_i32, int32_t, int32_t)
    CASE(1, TTO_I64, min_i64, int64_t, int64_t)
    CASE(2, TTO_F32, avg_f32, float, float)
    CASE(2, TTO_F64, avg_f64, double, double)
    CASE(2, TTO_U8, avg_u8, uint8_t, float)
    CASE(2, TTO_I16, avg_i16, int16_t, float)
    CASE(2, TTO_I32, avg_i32, int32_t, float)
    CASE(2, TTO_I64, avg_i64, int64_t, float)
#undef CASE
    return -1;
}

/* conv.hpp:171-275.  select = 1: max/min (gradient to the elements equal to the result), 0: avg. */
#define POOL_BACKWARD(NAME, R)                                                                                     \
    static void NAME(int select, const R *gout, R *gin, const R *X, const R *res, int B, int C, int H, int W,      \
                     int K, int S, int P) {                                                                        \
        const int Ho = (H + 2 * P - K) / S + 1, Wo = (W + 2 * P - K) / S + 1;                                      \
        memset(gin, 0, sizeof(R) * (size_t)B * C * H * W);                                                         \
        for (int b = 0; b < B; ++b)                                                                                \
            for (int c = 0; c < C; ++c) {                                                                          \
                const R *Xp = X + (size_t)(b * C + c) * H * W;                                                     \
                R *Gp = gin + (size_t)(b * C + c) * H * W;                                                         \
                for (int h = 0; h < Ho; ++h)                                                                       \
                    for (int w = 0; w < Wo; ++w) {                                                                 \
                        const size_t ir = ((size_t)(b * C + c) * Ho + h) * Wo + w;                                 \
                        R N = 0;                                                                                   \
                        const R target = res[ir];                                                                  \
                        if (select) {                                                                              \
                            for (int p = 0; p < K; ++p)                                                            \
                                for (int q = 0; q < K; ++q) {                                                      \
                                    const int hi = S * h + p - P, wi = S * w + q - P;                              \
                                    const int in = !(hi < 0 || wi < 0 || hi >= H || wi >= W);                      \
                                    N += (in && Xp[hi * W + wi] == target) ? (R)1 : (R)0;                          \
                                }                                                                                  \
                        } else {                                                                                   \
                            N = (R)(K * K);                                                                        \
                        }                                                                                          \
                        const R g = gout[ir] / N;                                                                  \
                        for (int p = 0; p < K; ++p)                                                                \
                            for (int q = 0; q < K; ++q) {                                                          \
                                const int hi = S * h + p - P, wi = S * w + q - P;                                  \
                                const int in = !(hi < 0 || wi < 0 || hi >= H || wi >= W);                          \
                                if (in && (!select || Xp[hi * W + wi] == target)) Gp[hi * W + wi] += g;            \
                            }                                                                                      \
                    }                                                                                              \
            }                                                                                                      \
    }

POOL_BACKWARD(pool_bwd_f32, float)
POOL_BACKWARD(pool_bwd_f64, double)

int tto_pool2d_backward(int dtype, int op, const void *grad_out, const void *input, const void *result, void *grad_input,
                        int B, int C, int H, int W, int k, int stride, int padding) {
    if (op < 0 || op > 2) return -1;
    if (dtype == TTO_F32) {
        pool_bwd_f32(op != 2, (const float *)grad_out, (float *)grad_input, (const float *)input, (const float *)result, B, C,
                     H, W, k, stride, padding);
        return 0;
    }
    if (dtype == TTO_F64) {
        pool_bwd_f64(op != 2, (const double *)grad_out, (double *)grad_input, (const double *)input, (const double *)result,
                     B, C, H, W, k, stride, padding);
        return 0;
    }
    return -1;
}
