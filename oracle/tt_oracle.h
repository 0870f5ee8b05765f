/*
 * tt_oracle.h — CPU restatement of tinytensor's GEMM / conv2d-as-GEMM path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP kernels are
 * compared against and the single-core CPU baseline that the benchmark times
 * beside the GPU.  Nothing in the shipped package (tinytensor_amd/, include/)
 * may link, load or call it; the product path has no CPU fallback.
 *
 * Every function cites the reference file:line whose behaviour it restates
 * (paths relative to the tinytensor source tree, v1.0.6).
 *
 * Pinning status (what independent evidence fixes each function):
 *   tto_matmul_kernel_*   exact vs the reference test's naive triple loop on the
 *                         reference's own integer patterns; bit-identical to the
 *                         independent scalar statement of the summation order
 *                         (tto_matmul_blocked_scalar_*); f64-accumulated naive
 *                         GEMM within K-scaled rounding bounds.
 *                         The *bit pattern* on non-integer f32/f64 data could only
 *                         be pinned by compiling the reference header, which needs
 *                         <format> and a cmake-generated export header that this
 *                         toolchain lacks: bit-level parity unpinned, numeric
 *                         parity is tolerance based.
 *   tto_contiguous        brute force against explicit nested-loop indexing.
 *   tto_conv2d_*          naive 7-deep loop (reference test oracle), adjoint
 *                         identities for the backward pass, and torch's CPU conv2d
 *                         and its autograd on the shapes of the reference's TT_TORCH
 *                         tests (tests/test_conv.cpp:147-184,
 *                         tests/test_conv_autograd.cpp:43-107).
 *   tto_batched_matmul backward  torch autograd on tests/test_matmul_autograd.cpp:218-262.
 *   tto_pool2d_*          torch.nn.functional max_pool2d / avg_pool2d and their autograd on
 *                         the reference tests' shapes (what tests/test_conv.cpp:186-278 and
 *                         tests/test_conv_autograd.cpp:109-230 compare with), plus a
 *                         brute-force numpy window statement incl. ties and padding.
 *   tto_splitmix64 / xorshift64  published test vectors (Vigna's splitmix64.c
 *                         seed 1234567 stream; xorshift64 13/7/17 closed form).
 *   tto_uniform_real_*    closed form from the bit construction.
 *   tto_uniform_real_view_*  the dense draw in the view's order scattered by explicit index loops
 *                         (brute force), and numpy's transposition of the dense draw for the
 *                         permuted view that nn::Conv2d's initialisation uses.
 *   tto_draw_params_*     element by element against the scalar-parameter draws above: element i equals
 *                         element i of a dense draw from the same seed with (p0[i], p1[i]) as the scalars
 *                         (brute force over every element), through dense and permuted views.
 *   tto_normal_*          closed form: every element's (u1, u2) rebuilt from the integer
 *                         generator and mu + std*sqrt(-2*log1p(-u1))*sin(2*pi*u2) evaluated
 *                         with 200-bit transcendentals, each step rounded to the type; f32
 *                         within 2 ulp, f64 within 4 ulp of std*z, with negative controls
 *                         (cos for sin, u1/u2 swapped, log(u1)) that must miss the bound.
 *                         The last bits depend on libm's log1p/sin, so inputs drawn from it
 *                         are generated once on the host and handed to both sides.
 */
#ifndef TT_ORACLE_H_
#define TT_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype codes follow tinytensor's ScalarType order (include/tt/scalar.h:21-29). */
enum tto_dtype {
    TTO_BOOL = 0,
    TTO_U8 = 1,
    TTO_I16 = 2,
    TTO_I32 = 3,
    TTO_I64 = 4,
    TTO_F32 = 5,
    TTO_F64 = 6
};

/* ---- RNG (tinytensor/tensor/random.cpp:26-63) ---- */
uint64_t tto_splitmix64(uint64_t seed);
uint64_t tto_xorshift64(uint64_t *state);
/* Generator(seed): state = splitmix64(seed) (random.cpp:47-51). */
uint64_t tto_generator_seed(uint64_t seed);

/* Tensor-level draws (cpu/distribution.cpp:31-38, cpu/kernel/distribution.hpp:28-32,
 * common/kernel/distribution.hpp:92-99, 232-246).  *state is the master
 * generator's state, advanced by n outputs. */
void tto_uniform_real_f32(uint64_t *state, float low, float high, float *out, int64_t n);
void tto_uniform_real_f64(uint64_t *state, double low, double high, double *out, int64_t n);
void tto_normal_f32(uint64_t *state, float mu, float std, float *out, int64_t n);
void tto_normal_f64(uint64_t *state, double mu, double std, double *out, int64_t n);

/* In-place uniform draws through a strided view (cpu/distribution.cpp:96-139, cpu/kernel/distribution.hpp:28-32):
 * the i-th element of the view in row-major order of `shape` takes the i-th master output as its state and lands
 * at data[offset + sum(index[d]*stride[d])].  Strides and offset in elements. */
void tto_uniform_real_view_f32(uint64_t *state, float low, float high, float *data, int ndim, const int *shape,
                               const int *stride, int offset);
void tto_uniform_real_view_f64(uint64_t *state, double low, double high, double *data, int ndim, const int *shape,
                               const int *stride, int offset);

/* Draws with a parameter pair per element (backend_base.h:83-103; cpu/distribution.cpp:42-139): dense parameter arrays
 * p0 / p1 (low / high for dist 0, mu / std for dist 1), element i of the view reads p0[i], p1[i]. */
void tto_draw_params_f32(uint64_t *state, int dist, const float *p0, const float *p1, float *data, int ndim, const int *shape,
                         const int *stride, int offset);
void tto_draw_params_f64(uint64_t *state, int dist, const double *p0, const double *p1, double *data, int ndim, const int *shape,
                         const int *stride, int offset);

/* ---- strided view -> dense copy (Tensor::contiguous via the identity op:
 * cpu/unary.cpp:26-58 with common/util.h:18-34) ---- */
void tto_contiguous(const void *src, void *dst, int elem_size, int ndim, const int *shape, const int *stride,
                    int offset);

/* ---- dense row-major GEMM C[N,M] = A[N,K] . B[K,M] ----
 * tto_matmul_kernel_*: tiled restatement of cpu/kernel/matmul.hpp:112-225
 *   (static zeroed scratch, padded copies, 64^3 tiles, 8 x 4-vector register block).
 * tto_matmul_blocked_scalar_*: the same summation order written per element
 *   (k in blocks of 64; inside a block t = muladd(a,b,t) from 0; C += t).
 * tto_matmul_naive_*: the reference test oracle (tests/test_matmul.cpp:33-46). */
#define TTO_DECL_GEMM(SUF, T)                                                                   \
    void tto_matmul_kernel_##SUF(const T *A, const T *B, T *C, int N, int K, int M);            \
    void tto_matmul_blocked_scalar_##SUF(const T *A, const T *B, T *C, int N, int K, int M);    \
    void tto_matmul_naive_##SUF(const T *A, const T *B, T *C, int N, int K, int M);
TTO_DECL_GEMM(f32, float)
TTO_DECL_GEMM(f64, double)
TTO_DECL_GEMM(u8, uint8_t)
TTO_DECL_GEMM(i16, int16_t)
TTO_DECL_GEMM(i32, int32_t)
TTO_DECL_GEMM(i64, int64_t)
#undef TTO_DECL_GEMM

/* ---- BackendBase::batched_matmul on the CPU device (cpu/matmul.cpp:25-74):
 * contiguous() both operands, then one matmul_kernel per batch.
 * Operands are 3-D strided views: element offset + (batch,row,col) strides in elements.
 * Returns 0, or -1 for an unsupported dtype. */
int tto_batched_matmul(int dtype, int B, int N, int K, int M, const void *lhs, int lhs_offset,
                       const int *lhs_stride, const void *rhs, int rhs_offset, const int *rhs_stride, void *out);

/* ---- conv2d forward/backward (cpu/conv.cpp:36-294, cpu/kernel/conv.hpp:12-118) ----
 * Dense NCHW input [B,C,H,W], weight [O,C,k,k], optional bias [O] (NULL = none).
 * backward: grad_bias may be NULL. */
int tto_conv2d_forward(int dtype, const void *input, const void *weight, const void *bias, void *out, int B, int C,
                       int H, int W, int O, int k, int stride, int padding);
int tto_conv2d_backward(int dtype, const void *grad_out, const void *input, const void *weight, void *grad_input,
                        void *grad_weight, void *grad_bias, int B, int C, int H, int W, int O, int k, int stride,
                        int padding);
/* Naive 7-deep loop (tests/test_conv.cpp:29-73). */
int tto_conv2d_naive(int dtype, const void *input, const void *weight, void *out, int B, int C, int H, int W, int O,
                     int k, int stride, int padding);

/* ---- 2-D pooling (cpu/conv.cpp:296-426, cpu/kernel/conv.hpp:121-275; tt_oracle_pool.c) ----
 * op: 0 max, 1 min, 2 avg.  Dense NCHW input; the result has the input's dtype except avg of an integer
 * input, which is f32.  backward: f32 / f64 only; grad_out, result and grad_input share the input's dtype. */
int tto_pool2d_forward(int dtype, int op, const void *input, void *out, int B, int C, int H, int W, int k, int stride,
                       int padding);
int tto_pool2d_backward(int dtype, int op, const void *grad_out, const void *input, const void *result, void *grad_input,
                        int B, int C, int H, int W, int k, int stride, int padding);

/* im2col / col2im index maps exposed for brute-force tests (conv.hpp:12-118), f64 only. */
void tto_unroll_f64(const double *X, double *Xu, int b, int C, int H, int W, int k, int S, int P);
void tto_unroll_transpose_f64(const double *X, double *Xu, int b, int C, int H, int W, int k, int S, int P);
void tto_col2im_f64(double *X, const double *Xu, int b, int C, int H, int W, int k, int S, int P);

/* 1 if this build contracts a*b+c into fma (the g++ -O2 -march=native flavour of the
 * reference), 0 for the separate mul/add flavour (clang). */
int tto_uses_fma(void);

#ifdef __cplusplus
}
#endif
#endif /* TT_ORACLE_H_ */
