/*
 * tt_oracle.c — CPU restatement of tinytensor's GEMM / conv2d-as-GEMM path (plain C).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels and the single-core CPU
 * baseline.  See tt_oracle.h for scope, citations and pinning status.
 *
 * Build flavours (oracle/Makefile):
 *   -DTTO_CONTRACT=1 -ffp-contract=fast : a*b+c contracts to fma, as g++ does for the
 *                                          reference kernel under -O2 -march=native.
 *   -DTTO_CONTRACT=0 -ffp-contract=off  : separate multiply and add, as clang emits.
 */
#include "tt_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifndef TTO_CONTRACT
#define TTO_CONTRACT 1
#endif

#define TTO_MAX_STORAGE (1200 * 1200) /* matmul.hpp:26 */
#define TTO_TILE 64                   /* matmul.hpp:27 */

static inline int round_up_i(int n, int b) { return ((n + b - 1) / b) * b; } /* matmul.hpp:104-106 */
static inline int min_i(int a, int b) { return a < b ? a : b; }

static void *zeroed_aligned(size_t bytes) {
    const size_t rounded = (bytes + 63) & ~(size_t)63;
    void *p = aligned_alloc(64, rounded ? rounded : 64);
    memset(p, 0, rounded);
    return p;
}

int tto_uses_fma(void) { return TTO_CONTRACT; }

/* ------------------------------------------------------------------ RNG */
/* random.cpp:26-31 */
uint64_t tto_splitmix64(uint64_t seed) {
    uint64_t r = seed + 0x9E3779B97f4A7C15ull;
    r = (r ^ (r >> 30)) * 0xBF58476D1CE4E5B9ull;
    r = (r ^ (r >> 27)) * 0x94D049BB133111EBull;
    return r ^ (r >> 31);
}
/* random.cpp:36-43 */
uint64_t tto_xorshift64(uint64_t *state) {
    uint64_t x = *state;
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    *state = x;
    return x;
}
uint64_t tto_generator_seed(uint64_t seed) { return tto_splitmix64(seed); }

/* common/kernel/distribution.hpp:92-99 with float_bits (:46-60) */
static inline float uniform_sample_f32(float low, float high, uint64_t *st) {
    union {
        uint32_t u;
        float f;
    } v;
    v.u = ((uint32_t)tto_xorshift64(st) >> 9) | ((uint32_t)127 << 23);
    const float r = v.f - 1.0f;
    return r * (high - low) + low;
}
static inline double uniform_sample_f64(double low, double high, uint64_t *st) {
    union {
        uint64_t u;
        double f;
    } v;
    v.u = (tto_xorshift64(st) >> 12) | ((uint64_t)1023 << 52);
    const double r = v.f - 1.0;
    return r * (high - low) + low;
}

/* Element i gets its own generator whose state is the i-th output of the master generator
 * (cpu/distribution.cpp:31-38, cpu/kernel/distribution.hpp:28-32). */
void tto_uniform_real_f32(uint64_t *state, float low, float high, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        uint64_t st = tto_xorshift64(state);
        out[i] = uniform_sample_f32(low, high, &st);
    }
}
void tto_uniform_real_f64(uint64_t *state, double low, double high, double *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        uint64_t st = tto_xorshift64(state);
        out[i] = uniform_sample_f64(low, high, &st);
    }
}
/* Box-Muller, common/kernel/distribution.hpp:232-246 */
void tto_normal_f32(uint64_t *state, float mu, float std, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        uint64_t st = tto_xorshift64(state);
        const float u1 = uniform_sample_f32(0.0f, 1.0f, &st);
        const float u2 = uniform_sample_f32(0.0f, 1.0f, &st);
        const float r = sqrtf(-2.0f * log1pf(-u1));
        const float theta = 2.0f * 3.14159265358979323846f * u2;
        out[i] = std * (r * sinf(theta)) + mu;
    }
}
void tto_normal_f64(uint64_t *state, double mu, double std, double *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        uint64_t st = tto_xorshift64(state);
        const double u1 = uniform_sample_f64(0.0, 1.0, &st);
        const double u2 = uniform_sample_f64(0.0, 1.0, &st);
        const double r = sqrt(-2.0 * log1p(-u1));
        const double theta = 2.0 * 3.14159265358979323846 * u2;
        out[i] = std * (r * sin(theta)) + mu;
    }
}

/* ------------------------------------------------------------------ contiguous() */
/* common/util.h:18-34 */
static inline int to_flat_index(int rank, int ndim, const int *shape, const int *stride, int offset) {
    int flat = offset;
    for (int i = ndim - 1; i >= 0; --i) {
        flat += (rank % shape[i]) * stride[i];
        rank /= shape[i];
    }
    return flat;
}

/* In-place draws through a strided view (cpu/distribution.cpp:96-139 with cpu/kernel/distribution.hpp:28-32):
 * element i of the view (row-major rank over `shape`) takes master output i as its state and is written at
 * to_flat_index(i).  nn::Conv2d initialises its weight through weight->permute({1,0,2,3}) (nn/conv2d.cpp:56). */
void tto_uniform_real_view_f32(uint64_t *state, float low, float high, float *data, int ndim, const int *shape,
                               const int *stride, int offset) {
    int n = 1;
    for (int d = 0; d < ndim; ++d) n *= shape[d];
    for (int i = 0; i < n; ++i) {
        uint64_t st = tto_xorshift64(state);
        data[to_flat_index(i, ndim, shape, stride, offset)] = uniform_sample_f32(low, high, &st);
    }
}
void tto_uniform_real_view_f64(uint64_t *state, double low, double high, double *data, int ndim, const int *shape,
                               const int *stride, int offset) {
    int n = 1;
    for (int d = 0; d < ndim; ++d) n *= shape[d];
    for (int i = 0; i < n; ++i) {
        uint64_t st = tto_xorshift64(state);
        data[to_flat_index(i, ndim, shape, stride, offset)] = uniform_sample_f64(low, high, &st);
    }
}
/* Draws with a parameter pair per element (the tensor forms, backend_base.h:83-103; cpu/distribution.cpp:42-139):
 * the parameters are made contiguous first, so element i reads p0[i], p1[i]; the result is written through the view
 * (dense: stride of a row-major tensor, offset 0).  dist 0 = uniform_real(low, high), 1 = normal(mu, std). */
#define TTO_DRAW_PARAMS(NAME, T, SAMPLE, SQRT, LOG1P, SIN, PI)                                                                \
    void NAME(uint64_t *state, int dist, const T *p0, const T *p1, T *data, int ndim, const int *shape, const int *stride, \
              int offset) {                                                                                                 \
        int n = 1;                                                                                                          \
        for (int d = 0; d < ndim; ++d) n *= shape[d];                                                                       \
        for (int i = 0; i < n; ++i) {                                                                                       \
            uint64_t st = tto_xorshift64(state);                                                                            \
            T value;                                                                                                        \
            if (dist == 0) {                                                                                                \
                value = SAMPLE(p0[i], p1[i], &st);                                                                          \
            } else {                                                                                                        \
                const T u1 = SAMPLE((T)0, (T)1, &st);                                                                       \
                const T u2 = SAMPLE((T)0, (T)1, &st);                                                                       \
                const T r = SQRT((T)-2 * LOG1P(-u1));                                                                       \
                const T theta = (T)2 * PI * u2;                                                                             \
                value = p1[i] * (r * SIN(theta)) + p0[i];                                                                   \
            }                                                                                                               \
            data[to_flat_index(i, ndim, shape, stride, offset)] = value;                                                    \
        }                                                                                                                   \
    }
TTO_DRAW_PARAMS(tto_draw_params_f32, float, uniform_sample_f32, sqrtf, log1pf, sinf, 3.14159265358979323846f)
TTO_DRAW_PARAMS(tto_draw_params_f64, double, uniform_sample_f64, sqrt, log1p, sin, 3.14159265358979323846)
#undef TTO_DRAW_PARAMS

/* identity op into a dense result (cpu/unary.cpp:26-58) */
void tto_contiguous(const void *src, void *dst, int elem_size, int ndim, const int *shape, const int *stride,
                    int offset) {
    int numel = 1;
    for (int i = 0; i < ndim; ++i) numel *= shape[i];
    const char *s = (const char *)src;
    char *d = (char *)dst;
    for (int i = 0; i < numel; ++i) {
        const int idx = to_flat_index(i, ndim, shape, stride, offset);
        memcpy(d + (size_t)i * elem_size, s + (size_t)idx * elem_size, (size_t)elem_size);
    }
}

/* ------------------------------------------------------------------ per-dtype kernels */
typedef float v_f32 __attribute__((vector_size(16)));
typedef double v_f64 __attribute__((vector_size(16)));
typedef uint8_t v_u8 __attribute__((vector_size(16)));
typedef int16_t v_i16 __attribute__((vector_size(16)));
typedef int32_t v_i32 __attribute__((vector_size(16)));
typedef int64_t v_i64 __attribute__((vector_size(16)));

#if TTO_CONTRACT
#define MULADD_F32(a, b, t) __builtin_fmaf((a), (b), (t))
#define MULADD_F64(a, b, t) __builtin_fma((a), (b), (t))
#else
#define MULADD_F32(a, b, t) ((t) + (a) * (b))
#define MULADD_F64(a, b, t) ((t) + (a) * (b))
#endif

#define T float
#define SUF f32
#define VT v_f32
#define VN 4
#define MULADD(a, b, t) MULADD_F32(a, b, t)
#include "tt_oracle_kernels.inc"
#undef T
#undef SUF
#undef VT
#undef VN
#undef MULADD

#define T double
#define SUF f64
#define VT v_f64
#define VN 2
#define MULADD(a, b, t) MULADD_F64(a, b, t)
#include "tt_oracle_kernels.inc"
#undef T
#undef SUF
#undef VT
#undef VN
#undef MULADD

/* Integer dtypes wrap modulo 2^n like the SIMD lanes of cpu/kernel/simd.h:120-127;
 * arithmetic is done unsigned to keep the wrap defined in C. */
#define T uint8_t
#define SUF u8
#define VT v_u8
#define VN 16
#define MULADD(a, b, t) ((uint8_t)((t) + (uint8_t)((a) * (b))))
#include "tt_oracle_kernels.inc"
#undef T
#undef SUF
#undef VT
#undef VN
#undef MULADD

#define T int16_t
#define SUF i16
#define VT v_i16
#define VN 8
#define MULADD(a, b, t) ((int16_t)((uint16_t)(t) + (uint16_t)((uint16_t)(a) * (uint16_t)(b))))
#include "tt_oracle_kernels.inc"
#undef T
#undef SUF
#undef VT
#undef VN
#undef MULADD

#define T int32_t
#define SUF i32
#define VT v_i32
#define VN 4
#define MULADD(a, b, t) ((int32_t)((uint32_t)(t) + (uint32_t)(a) * (uint32_t)(b)))
#include "tt_oracle_kernels.inc"
#undef T
#undef SUF
#undef VT
#undef VN
#undef MULADD

#define T int64_t
#define SUF i64
#define VT v_i64
#define VN 2
#define MULADD(a, b, t) ((int64_t)((uint64_t)(t) + (uint64_t)(a) * (uint64_t)(b)))
#include "tt_oracle_kernels.inc"
#undef T
#undef SUF
#undef VT
#undef VN
#undef MULADD

/* ------------------------------------------------------------------ dtype dispatch */
#define DISPATCH(dtype, CALL)                    \
    switch (dtype) {                             \
    case TTO_U8: { typedef uint8_t T_; CALL(u8); return 0; }   \
    case TTO_I16: { typedef int16_t T_; CALL(i16); return 0; } \
    case TTO_I32: { typedef int32_t T_; CALL(i32); return 0; } \
    case TTO_I64: { typedef int64_t T_; CALL(i64); return 0; } \
    case TTO_F32: { typedef float T_; CALL(f32); return 0; }   \
    case TTO_F64: { typedef double T_; CALL(f64); return 0; }  \
    default: return -1;                          \
    }

int tto_batched_matmul(int dtype, int B, int N, int K, int M, const void *lhs, int lhs_offset,
                       const int *lhs_stride, const void *rhs, int rhs_offset, const int *rhs_stride, void *out) {
#define CALL(S) \
    batched_matmul_##S(B, N, K, M, (const T_ *)lhs, lhs_offset, lhs_stride, (const T_ *)rhs, rhs_offset, rhs_stride, (T_ *)out)
    DISPATCH(dtype, CALL)
#undef CALL
}

int tto_conv2d_forward(int dtype, const void *input, const void *weight, const void *bias, void *out, int B, int C,
                       int H, int W, int O, int k, int stride, int padding) {
#define CALL(S) \
    conv2d_forward_##S((const T_ *)input, (const T_ *)weight, (const T_ *)bias, (T_ *)out, B, C, H, W, O, k, stride, padding)
    DISPATCH(dtype, CALL)
#undef CALL
}

int tto_conv2d_backward(int dtype, const void *grad_out, const void *input, const void *weight, void *grad_input,
                        void *grad_weight, void *grad_bias, int B, int C, int H, int W, int O, int k, int stride,
                        int padding) {
#define CALL(S)                                                                                              \
    conv2d_backward_##S((const T_ *)grad_out, (const T_ *)input, (const T_ *)weight, (T_ *)grad_input,      \
                        (T_ *)grad_weight, (T_ *)grad_bias, B, C, H, W, O, k, stride, padding)
    DISPATCH(dtype, CALL)
#undef CALL
}

int tto_conv2d_naive(int dtype, const void *input, const void *weight, void *out, int B, int C, int H, int W, int O,
                     int k, int stride, int padding) {
#define CALL(S) conv2d_naive_##S((const T_ *)input, (const T_ *)weight, (T_ *)out, B, C, H, W, O, k, stride, padding)
    DISPATCH(dtype, CALL)
#undef CALL
}

void tto_unroll_f64(const double *X, double *Xu, int b, int C, int H, int W, int k, int S, int P) {
    unroll_f64(X, Xu, b, C, H, W, k, S, P);
}
void tto_unroll_transpose_f64(const double *X, double *Xu, int b, int C, int H, int W, int k, int S, int P) {
    unroll_transpose_f64(X, Xu, b, C, H, W, k, S, P);
}
void tto_col2im_f64(double *X, const double *Xu, int b, int C, int H, int W, int k, int S, int P) {
    col2im_f64(X, Xu, b, C, H, W, k, S, P);
}
