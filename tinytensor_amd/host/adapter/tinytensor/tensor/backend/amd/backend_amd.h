// backend_amd.h
// AMD backend (MI355X, gfx950): tinytensor::BackendBase over the C ABI of libttamd (include/ttamd.h).
//
// Every pure virtual of BackendBase (tinytensor/tensor/backend_base.h:23-322) is overridden here.  The operations on
// the GEMM path and the callers either side of it run on the device (backend_amd.cpp lists them); every other
// operation throws TTException("... not implemented on the AMD device").  The declarations are written as lists per
// signature family: the list entries are the names (and parameter names) of backend_base.h, expanded by the macros
// right above each list, so that a new virtual in the base shows up as one missing list entry.

#ifndef TINYTENSOR_BACKEND_AMD_H_
#define TINYTENSOR_BACKEND_AMD_H_

#include <tt/random.h>
#include <tt/scalar.h>
#include <tt/tensor.h>

#include "tensor/backend_base.h"

#include <cstddef>
#include <cstdint>
#include <optional>
#include <utility>
#include <ostream>
#include <tuple>
#include <vector>

namespace tinytensor::amd {

// ---- signature families --------------------------------------------------------------------------------------
// element types of from_vec / to_vec (bool has only the const-reference from_vec: it is stored as uint8_t)
#define TT_AMD_VEC_TYPES(X) X(uint8_t) X(int16_t) X(int32_t) X(int64_t) X(float) X(double)

// Tensor f(const Tensor &tensor)
#define TT_AMD_TENSOR_TO_TENSOR(X)                                                                                     \
    X(min) X(argmin) X(max) X(argmax) X(sum)                                                                           \
    X(identity) X(negate) X(logical_not) X(abs) X(sign) X(log) X(log10) X(log2) X(log1p) X(exp) X(exp2) X(expm1)       \
    X(sqrt) X(sin) X(cos) X(tan) X(asin) X(acos) X(atan) X(sinh) X(cosh) X(tanh) X(asinh) X(acosh) X(atanh) X(erf)     \
    X(erfc) X(tgamma) X(lgamma) X(digamma) X(ceil) X(floor) X(round) X(isinf) X(isnan) X(isfinite)                     \
    X(sigmoid) X(log_sigmoid) X(hardsigmoid) X(relu) X(relu6) X(selu) X(silu) X(softsign)

// void f_(Tensor &tensor)
#define TT_AMD_TENSOR_INPLACE(X)                                                                                       \
    X(identity_) X(negate_) X(logical_not_) X(abs_) X(sign_) X(log_) X(log10_) X(log2_) X(log1p_) X(exp_) X(exp2_)     \
    X(expm1_) X(sqrt_) X(sin_) X(cos_) X(tan_) X(asin_) X(acos_) X(atan_) X(sinh_) X(cosh_) X(tanh_) X(asinh_)         \
    X(acosh_) X(atanh_) X(erf_) X(erfc_) X(tgamma_) X(lgamma_) X(digamma_) X(ceil_) X(floor_) X(round_)                \
    X(sigmoid_) X(log_sigmoid_) X(hardsigmoid_) X(relu_) X(relu6_) X(selu_) X(silu_) X(softsign_)

// Tensor f(const Tensor &lhs, const Tensor &rhs)
#define TT_AMD_BINARY(X)                                                                                               \
    X(eq) X(ne) X(lt) X(le) X(gt) X(ge) X(logical_or) X(logical_and) X(bitwise_or) X(bitwise_and) X(bitwise_xor)       \
    X(bitwise_left_shift) X(bitwise_right_shift) X(modulo) X(add) X(sub) X(mul) X(div) X(maximum) X(minimum) X(pow)    \
    X(batched_matmul)

// void f(Tensor &lhs, const Tensor &rhs)
#define TT_AMD_BINARY_INPLACE(X) X(assign) X(add_inplace) X(sub_inplace) X(mul_inplace) X(div_inplace)

// Tensor f(const Tensor &tensor, int dim)
#define TT_AMD_TENSOR_DIM(X) X(min) X(argmin) X(max) X(argmax) X(sum) X(all) X(any) X(softmax) X(log_softmax)

// distributions: Tensor f(const Tensor &a, [const Tensor &b,] Generator &gen) and the in-place forms
#define TT_AMD_DIST_ONE(X) X(bernoulli, p) X(geometric, p) X(poisson, lambda) X(exponential, lambda)
#define TT_AMD_DIST_TWO(X)                                                                                             \
    X(uniform_int, low, high) X(uniform_real, low, high) X(binomial, p, num_draws) X(normal, mu, std)                  \
    X(cauchy, loc, scale) X(lognormal, mu, std) X(weibull, scale, shape)

// pooling: Tensor f(input, kernel_size, stride, padding) and Tensor f_backward(grad_output, input, result, ...)
#define TT_AMD_POOLS(X) X(max_pool2d) X(min_pool2d) X(avg_pool2d)

class BackendAMD : public BackendBase {
public:
    // Tensor construction
    [[nodiscard]] auto from_vec(const std::vector<bool> &data, int device_id) const -> StoragePtr override;
#define X(T)                                                                                        \
    [[nodiscard]] auto from_vec(const std::vector<T> &data, int device_id) const -> StoragePtr override; \
    [[nodiscard]] auto from_vec(std::vector<T> &&data, int device_id) const -> StoragePtr override;
    TT_AMD_VEC_TYPES(X)
#undef X
    [[nodiscard]] auto from_scalar(Scalar scalar, int device_id) const -> StoragePtr override;
    [[nodiscard]] auto full(const Scalar &value, std::size_t N, int device_id) const -> StoragePtr override;
    [[nodiscard]] auto arange(std::size_t N, ScalarType dtype, int device_id) const -> StoragePtr override;

    // Conversion to vec
#define X(T) void to_vec(const Tensor &tensor, std::vector<T> &data_out) const override;
    TT_AMD_VEC_TYPES(X)
#undef X

    // Getters
    [[nodiscard]] auto item(const Tensor &tensor) const -> Scalar override;
    [[nodiscard]] auto data_ptr(const Tensor &tensor) const -> uintptr_t override;

    // Indexing
    [[nodiscard]] auto index_mask(const Tensor &input, const Tensor &mask, int N_mask) const -> Tensor override;
    [[nodiscard]] auto index_indices(const Tensor &input, const Tensor &indices) const -> Tensor override;
    void index_put_mask(Tensor &input, const Tensor &values, const Tensor &mask) const override;
    void index_put_indices(Tensor &input, const Tensor &values, const Tensor &indices) const override;
    [[nodiscard]] auto gather(const Tensor &input, const Tensor &indices, int idx) const -> Tensor override;

    // Casts, printing
    [[nodiscard]] auto to(const Tensor &tensor, ScalarType dtype) const -> Tensor override;
    auto print(std::ostream &os, const Tensor &tensor) const -> std::ostream & override;

    // Distributions
#define X(NAME, A)                                                                                 \
    [[nodiscard]] auto NAME(const Tensor &A, Generator &gen) const -> Tensor override;            \
    void NAME##_(Tensor &tensor, const Tensor &A, Generator &gen) const override;
    TT_AMD_DIST_ONE(X)
#undef X
#define X(NAME, A, B)                                                                              \
    [[nodiscard]] auto NAME(const Tensor &A, const Tensor &B, Generator &gen) const -> Tensor override; \
    void NAME##_(Tensor &tensor, const Tensor &A, const Tensor &B, Generator &gen) const override;
    TT_AMD_DIST_TWO(X)
#undef X

    // Binary operators (batched_matmul among them), their in-place forms and assign
#define X(NAME) [[nodiscard]] auto NAME(const Tensor &lhs, const Tensor &rhs) const -> Tensor override;
    TT_AMD_BINARY(X)
#undef X
#define X(NAME) void NAME(Tensor &lhs, const Tensor &rhs) const override;
    TT_AMD_BINARY_INPLACE(X)
#undef X

    // Not a virtual of BackendBase: the two products of TensorBatchedMatmul::backward (autograd/binary_ops.cpp:173-179)
    // in one call, {lhs0 . rhs0, lhs1 . rhs1}, as one grid where ttamd_batched_matmul_pair can run them so.
    [[nodiscard]] auto batched_matmul_pair(const Tensor &lhs0, const Tensor &rhs0, const Tensor &lhs1, const Tensor &rhs1) const
        -> std::pair<Tensor, Tensor>;

    // Reductions, unary operators and activations
#define X(NAME) [[nodiscard]] auto NAME(const Tensor &tensor) const -> Tensor override;
    TT_AMD_TENSOR_TO_TENSOR(X)
#undef X
#define X(NAME) [[nodiscard]] auto NAME(const Tensor &tensor, int dim) const -> Tensor override;
    TT_AMD_TENSOR_DIM(X)
#undef X
    [[nodiscard]] auto all(const Tensor &tensor) const -> bool override;
    [[nodiscard]] auto any(const Tensor &tensor) const -> bool override;
#define X(NAME) void NAME(Tensor &tensor) const override;
    TT_AMD_TENSOR_INPLACE(X)
#undef X
    [[nodiscard]] auto softplus(const Tensor &tensor, double beta, double threshold) const -> Tensor override;
    [[nodiscard]] auto leaky_relu(const Tensor &tensor, double negative_slope) const -> Tensor override;
    [[nodiscard]] auto elu(const Tensor &tensor, double alpha) const -> Tensor override;
    [[nodiscard]] auto hardtanh(const Tensor &tensor, double min, double max) const -> Tensor override;
    void softplus_(Tensor &tensor, double beta, double threshold) const override;
    void leaky_relu_(Tensor &tensor, double negative_slope) const override;
    void elu_(Tensor &tensor, double alpha) const override;
    void hardtanh_(Tensor &tensor, double min, double max) const override;
    void softmax_(Tensor &tensor, int dim) const override;
    void log_softmax_(Tensor &tensor, int dim) const override;

    // Util/misc
    [[nodiscard]] auto where(const Tensor &cond, const Tensor &lhs, const Tensor &rhs) const -> Tensor override;
    void clamp_(Tensor &tensor, const Tensor &min, const Tensor &max) const override;

    // Convolution and pooling
    [[nodiscard]] auto conv2d(
        const Tensor &input,
        const Tensor &weight,
        const std::optional<Tensor> &bias,
        int stride,
        int padding
    ) const -> Tensor override;
    [[nodiscard]] auto conv2d_backward(
        const Tensor &grad_output,
        const Tensor &input,
        const Tensor &weight,
        const std::optional<Tensor> &bias,
        int stride,
        int padding
    ) const -> std::tuple<Tensor, Tensor, std::optional<Tensor>> override;
#define X(NAME)                                                                                                    \
    [[nodiscard]] auto NAME(const Tensor &input, int kernel_size, int stride, int padding) const -> Tensor override; \
    [[nodiscard]] auto NAME##_backward(                                                                            \
        const Tensor &grad_output,                                                                                 \
        const Tensor &input,                                                                                       \
        const Tensor &result,                                                                                      \
        int kernel_size,                                                                                           \
        int stride,                                                                                                \
        int padding                                                                                                \
    ) const -> Tensor override;
    TT_AMD_POOLS(X)
#undef X

    // Memory counters and devices
    [[nodiscard]] auto current_memory_allocated(int device_id) const -> uint64_t override;
    [[nodiscard]] auto total_memory_allocated(int device_id) const -> uint64_t override;
    [[nodiscard]] auto get_device_count() const -> int override;
};

}    // namespace tinytensor::amd

#endif    // TINYTENSOR_BACKEND_AMD_H_
