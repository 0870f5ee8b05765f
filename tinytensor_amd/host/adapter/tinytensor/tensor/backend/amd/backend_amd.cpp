// backend_amd.cpp
// AMD backend (MI355X, gfx950): tinytensor::BackendBase over the C ABI of libttamd (include/ttamd.h).
//
// Implemented on the device:
//   storage        from_vec, from_scalar, full, arange, to_vec, item, data_ptr, memory counters, device count
//   the GEMM path  batched_matmul, conv2d, conv2d_backward (operands are read through their strides, no contiguous copy)
//   around it      identity (= clone / contiguous), to, assign, add/sub/mul/div/pow/maximum/minimum and their in-place
//                  forms, eq/ne/lt/le/gt/ge, negate/abs/sqrt/exp/log/sigmoid/tanh/relu and their in-place forms, where,
//                  sum, all / any of a whole tensor (the frontend's argument checks use them, e.g. CHECK_UNIFORM,
//                  tensor/tensor.cpp:1753-1759), max/min/avg pooling forward and backward, uniform_real / normal with
//                  parameter tensors (a pair per element, or one value expanded over the shape as
//                  Tensor::uniform_real_(double, double) and nn::init pass, tensor/tensor.cpp:1795-1801)
// Everything else throws TTException("<op> is not implemented on the AMD device").
//
// Status codes of the C ABI map to the reference's error model: TTException for what a caller can act on, TT_ERROR
// (print + exit, include/tt/exception.h:28-36) for a failed launch, as cuda/kernel_launch.cuh:25-28 does.

#include "tensor/backend/amd/backend_amd.h"

#include <tt/exception.h>
#include <tt/random.h>
#include <tt/scalar.h>
#include <tt/shape.h>
#include <tt/tensor.h>

#include "tensor/backend/amd/storage_amd.h"
#include "ttamd.h"

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <optional>
#include <ostream>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

namespace tinytensor::amd {

namespace {

// ---- status, dtype, views ----------------------------------------------------------------------------------------
void check(ttamd_status status) {
    if (status == TTAMD_OK) {
        return;
    }
    const std::string message = ttamd_last_error_string();
    if (status == TTAMD_ERR_LAUNCH) {
        TT_ERROR(message);
    }
    TT_EXCEPTION(message);
}

[[noreturn]] void not_implemented(const char *op) {
    TT_EXCEPTION(std::string(op) + " is not implemented on the AMD device");
}

// ScalarType and ttamd_dtype number the dtypes alike (include/tt/scalar.h:21-29)
auto code(ScalarType dtype) -> ttamd_dtype {
    return static_cast<ttamd_dtype>(static_cast<int>(dtype));
}

auto element_size(ScalarType dtype) -> std::size_t {
    switch (dtype) {
    case kBool:
    case kU8:
        return 1;
    case kI16:
        return 2;
    case kI32:
    case kF32:
        return 4;
    case kI64:
    case kF64:
        return 8;
    }
    return 0;
}

auto storage_of(const Tensor &tensor) -> StorageAMD & {
    return tensor.get_storage<StorageAMD>();
}

// A tensor as the C ABI takes it: storage pointer, element offset, shape and element strides as 64-bit arrays
struct View {
    explicit View(const Tensor &tensor)
        : data(storage_of(tensor).ptr), offset(tensor.offset()), ndim(tensor.shape().ndim()) {
        const auto &sh = tensor.shape().to_vec();
        const auto &st = tensor.stride().to_vec();
        shape.assign(sh.begin(), sh.end());
        stride.assign(st.begin(), st.end());
        if (shape.empty()) {    // rank 0: the C ABI wants non-null arrays
            shape.push_back(1);
            stride.push_back(1);
        }
    }
    void *data;
    int64_t offset;
    int ndim;
    std::vector<int64_t> shape;
    std::vector<int64_t> stride;
};

auto view3(const Tensor &tensor) -> ttamd_view3 {
    const auto &st = tensor.stride();
    return {storage_of(tensor).ptr, tensor.offset(), {st[0], st[1], st[2]}};
}

auto view4(const Tensor &tensor) -> ttamd_view4 {
    const auto &st = tensor.stride();
    return {storage_of(tensor).ptr, tensor.offset(), {st[0], st[1], st[2], st[3]}};
}

auto data_at_offset(const Tensor &tensor) -> void * {
    return static_cast<char *>(storage_of(tensor).ptr) + static_cast<std::size_t>(tensor.offset()) * element_size(tensor.dtype());
}

// A fresh dense result of `numel` elements (the internal Tensor constructor: offset 0, dense strides,
// tensor/tensor.cpp:351-358)
auto make_storage(int device_id, std::size_t numel, ScalarType dtype) -> std::shared_ptr<StorageAMD> {
    return std::make_shared<StorageAMD>(device_id, numel * element_size(dtype));
}

auto make_result(std::shared_ptr<StorageAMD> storage, ScalarType dtype, Shape shape, Device device) -> Tensor {
    return {std::move(storage), dtype, std::move(shape), device};
}

template <typename T>
auto upload(const T *data, std::size_t n, int device_id) -> BackendBase::StoragePtr {
    auto storage = std::make_unique<StorageAMD>(device_id, n * sizeof(T));
    check(ttamd_memcpy_h2d(device_id, storage->ptr, data, n * sizeof(T)));
    return storage;
}

template <typename T>
void download(const Tensor &tensor, std::vector<T> &data_out) {
    // the whole storage comes back (callers clone first, tensor/tensor.cpp:555)
    const StorageAMD &storage = storage_of(tensor);
    data_out.resize(storage.bytes / sizeof(T));
    check(ttamd_memcpy_d2h(storage.device_id, data_out.data(), storage.ptr, data_out.size() * sizeof(T)));
}

// ---- element-wise families ---------------------------------------------------------------------------------------
auto binary_op(const Tensor &lhs, const Tensor &rhs, ttamd_binary_op op) -> Tensor {
    // the frontend has broadcast both operands to one shape and promoted them to one dtype
    const ScalarType result_type = op >= TTAMD_BIN_LT ? kBool : lhs.dtype();
    auto out = make_storage(lhs.device().id, static_cast<std::size_t>(lhs.numel()), result_type);
    const View l(lhs);
    const View r(rhs);
    check(ttamd_binary(
        lhs.device().id, code(lhs.dtype()), op, l.ndim, l.shape.data(), l.data, l.offset, l.stride.data(), r.data, r.offset,
        r.stride.data(), out->ptr, nullptr
    ));
    return make_result(std::move(out), result_type, lhs.shape(), lhs.device());
}

auto unary_op(const Tensor &tensor, ttamd_unary_op op) -> Tensor {
    auto out = make_storage(tensor.device().id, static_cast<std::size_t>(tensor.numel()), tensor.dtype());
    const View v(tensor);
    check(ttamd_unary(
        tensor.device().id, code(tensor.dtype()), op, v.ndim, v.shape.data(), v.data, v.offset, v.stride.data(), out->ptr, nullptr
    ));
    return make_result(std::move(out), tensor.dtype(), tensor.shape(), tensor.device());
}

void assign_view(Tensor &lhs, const Tensor &rhs) {
    const View l(lhs);
    const View r(rhs);
    check(ttamd_assign(
        lhs.device().id, code(lhs.dtype()), l.ndim, l.shape.data(), l.data, l.offset, l.stride.data(), r.data, r.offset,
        r.stride.data(), nullptr
    ));
}

auto sum_op(const Tensor &tensor, int dim) -> Tensor {
    // bool and integer tensors sum in 64 bits into an i64 result (common/reduce.h:56-61); a reduced dimension stays
    // with extent 1 (cpu/reduce.cpp:29-32), sum(tensor) has shape {1}
    const ScalarType result_type = is_float_dtype(tensor.dtype()) ? tensor.dtype() : kI64;
    Shape result_shape = dim < 0 ? Shape({1}) : tensor.shape();
    if (dim >= 0) {
        result_shape[dim] = 1;
    }
    auto out = make_storage(tensor.device().id, static_cast<std::size_t>(result_shape.numel()), result_type);
    const View v(tensor);
    check(ttamd_sum(
        tensor.device().id, code(tensor.dtype()), v.ndim, v.shape.data(), v.data, v.offset, v.stride.data(), dim, out->ptr, nullptr
    ));
    return make_result(std::move(out), result_type, std::move(result_shape), tensor.device());
}

auto pool_forward(const Tensor &input, ttamd_pool_op op, int kernel_size, int stride, int padding) -> Tensor {
    const int B = input.size(0);
    const int C = input.size(1);
    const int H = input.size(2);
    const int W = input.size(3);
    const int H_out = (H + 2 * padding - kernel_size) / stride + 1;
    const int W_out = (W + 2 * padding - kernel_size) / stride + 1;
    // the mean of an integer tensor is computed in the default float type (common/reduce.h:63-69)
    const ScalarType result_type = (op == TTAMD_POOL_AVG && !is_float_dtype(input.dtype())) ? kDefaultFloat : input.dtype();
    Shape result_shape({B, C, H_out, W_out});
    auto out = make_storage(input.device().id, static_cast<std::size_t>(result_shape.numel()), result_type);
    const ttamd_view4 iv = view4(input);
    check(ttamd_pool2d_forward(input.device().id, code(input.dtype()), op, &iv, out->ptr, B, C, H, W, kernel_size, stride, padding, nullptr));
    return make_result(std::move(out), result_type, std::move(result_shape), input.device());
}

auto pool_backward(
    const Tensor &grad_output,
    const Tensor &input,
    const Tensor &result,
    ttamd_pool_op op,
    int kernel_size,
    int stride,
    int padding
) -> Tensor {
    const Tensor grad = grad_output.contiguous();
    const Tensor res = result.contiguous();
    auto out = make_storage(input.device().id, static_cast<std::size_t>(input.numel()), input.dtype());
    const ttamd_view4 iv = view4(input);
    check(ttamd_pool2d_backward(
        input.device().id, code(input.dtype()), op, data_at_offset(grad), &iv, data_at_offset(res), out->ptr, input.size(0),
        input.size(1), input.size(2), input.size(3), kernel_size, stride, padding, nullptr
    ));
    return make_result(std::move(out), input.dtype(), input.shape(), input.device());
}

// ---- seeded draws ------------------------------------------------------------------------------------------------
// One generator state per element, drawn from the caller's generator in order (cpu/distribution.cpp:31-38)
auto draw_states(Generator &gen, std::size_t n) -> std::vector<uint64_t> {
    std::vector<uint64_t> states;
    states.reserve(n);
    for (std::size_t i = 0; i < n; ++i) {
        states.push_back(gen());
    }
    return states;
}

// dist: 0 uniform_real(low, high), 1 normal(mu, std); written through `tensor`'s view in its row-major order.  The
// parameters are tensors of the same shape (the frontend checks it and casts them to the result's dtype,
// tensor/tensor.cpp:1783-1794); element i reads its pair at rank i of their views, whether they hold a value per element
// or one value expanded with stride 0 (what the scalar overloads build, tensor/tensor.cpp:1795-1801).
void fill_random(Tensor &tensor, int dist, const Tensor &a, const Tensor &b, Generator &gen, const char *op) {
    if (!is_float_dtype(tensor.dtype())) {
        TT_EXCEPTION(std::string(op) + " expects a floating point tensor");
    }
    if (a.dtype() != tensor.dtype() || b.dtype() != tensor.dtype() || a.numel() != tensor.numel() || b.numel() != tensor.numel()) {
        TT_EXCEPTION(std::string(op) + " expects parameters of the result's shape and dtype");
    }
    const std::vector<uint64_t> states = draw_states(gen, static_cast<std::size_t>(tensor.numel()));
    const View v(tensor);
    const View pa(a);
    const View pb(b);
    check(ttamd_random_fill_states_params(
        tensor.device().id, code(tensor.dtype()), dist, pa.data, pa.offset, pa.stride.data(), pb.data, pb.offset, pb.stride.data(),
        states.data(), v.ndim, v.shape.data(), v.stride.data(), v.data, v.offset, nullptr
    ));
}

auto new_random(int dist, const Tensor &a, const Tensor &b, Generator &gen, const char *op) -> Tensor {
    Tensor result = make_result(make_storage(a.device().id, static_cast<std::size_t>(a.numel()), a.dtype()), a.dtype(), a.shape(), a.device());
    fill_random(result, dist, a, b, gen, op);
    return result;
}

}    // namespace

// ---- storage -----------------------------------------------------------------------------------------------------
StorageAMD::StorageAMD(int _device_id, std::size_t _bytes)
    : bytes(std::max<std::size_t>(_bytes, 1)), device_id(_device_id) {
    check(ttamd_malloc(device_id, bytes, &ptr));
}

StorageAMD::~StorageAMD() {
    (void)ttamd_free(device_id, ptr, bytes);
}

auto BackendAMD::from_vec(const std::vector<bool> &data, int device_id) const -> StoragePtr {
    const std::vector<uint8_t> bytes(data.begin(), data.end());    // bool is stored as one byte holding 0 or 1
    return upload(bytes.data(), bytes.size(), device_id);
}
#define X(T)                                                                                         \
    auto BackendAMD::from_vec(const std::vector<T> &data, int device_id) const -> StoragePtr {      \
        return upload(data.data(), data.size(), device_id);                                         \
    }                                                                                                \
    auto BackendAMD::from_vec(std::vector<T> &&data, int device_id) const -> StoragePtr {           \
        return upload(data.data(), data.size(), device_id);                                         \
    }                                                                                                \
    void BackendAMD::to_vec(const Tensor &tensor, std::vector<T> &data_out) const {                 \
        download(tensor, data_out);                                                                 \
    }
TT_AMD_VEC_TYPES(X)
#undef X

auto BackendAMD::full(const Scalar &value, std::size_t N, int device_id) const -> StoragePtr {
    const ScalarType dtype = value.dtype();
    auto storage = std::make_unique<StorageAMD>(device_id, N * element_size(dtype));
    // one host element of the value's own type
    alignas(8) unsigned char host[8] = {};
    switch (dtype) {
    case kBool:
    case kU8:
        *reinterpret_cast<uint8_t *>(host) = value.to<uint8_t>();
        break;
    case kI16:
        *reinterpret_cast<int16_t *>(host) = value.to<int16_t>();
        break;
    case kI32:
        *reinterpret_cast<int32_t *>(host) = value.to<int32_t>();
        break;
    case kI64:
        *reinterpret_cast<int64_t *>(host) = value.to<int64_t>();
        break;
    case kF32:
        *reinterpret_cast<float *>(host) = value.to<float>();
        break;
    case kF64:
        *reinterpret_cast<double *>(host) = value.to<double>();
        break;
    }
    check(ttamd_full(device_id, code(dtype), host, static_cast<int64_t>(N), storage->ptr, nullptr));
    return storage;
}

auto BackendAMD::from_scalar(Scalar scalar, int device_id) const -> StoragePtr {
    return full(scalar, 1, device_id);
}

auto BackendAMD::arange(std::size_t N, ScalarType dtype, int device_id) const -> StoragePtr {
    // 0, 1, ..., N - 1 in `dtype`: built on the host and uploaded (a creation routine, not on the hot path)
    auto fill = [&]<typename T>(T) -> StoragePtr {
        std::vector<T> host(N);
        for (std::size_t i = 0; i < N; ++i) {
            host[i] = static_cast<T>(i);
        }
        return upload(host.data(), host.size(), device_id);
    };
    switch (dtype) {
    case kBool:
    case kU8:
        return fill(uint8_t{});
    case kI16:
        return fill(int16_t{});
    case kI32:
        return fill(int32_t{});
    case kI64:
        return fill(int64_t{});
    case kF32:
        return fill(float{});
    case kF64:
        return fill(double{});
    }
    TT_ERROR("Unrecoverable: Unsupported type.");
}

auto BackendAMD::item(const Tensor &tensor) const -> Scalar {
    alignas(8) unsigned char host[8] = {};
    check(ttamd_memcpy_d2h(tensor.device().id, host, data_at_offset(tensor), element_size(tensor.dtype())));
    switch (tensor.dtype()) {
    case kBool:
        return Scalar(*reinterpret_cast<const uint8_t *>(host) != 0);
    case kU8:
        return Scalar(*reinterpret_cast<const uint8_t *>(host));
    case kI16:
        return Scalar(*reinterpret_cast<const int16_t *>(host));
    case kI32:
        return Scalar(*reinterpret_cast<const int32_t *>(host));
    case kI64:
        return Scalar(*reinterpret_cast<const int64_t *>(host));
    case kF32:
        return Scalar(*reinterpret_cast<const float *>(host));
    case kF64:
        return Scalar(*reinterpret_cast<const double *>(host));
    }
    TT_ERROR("Unrecoverable: Unsupported type.");
}

auto BackendAMD::data_ptr(const Tensor &tensor) const -> uintptr_t {
    return reinterpret_cast<uintptr_t>(data_at_offset(tensor));
}

auto BackendAMD::current_memory_allocated(int device_id) const -> uint64_t {
    uint64_t current = 0;
    check(ttamd_memory_allocated(device_id, &current, nullptr));
    return current;
}

auto BackendAMD::total_memory_allocated(int device_id) const -> uint64_t {
    uint64_t total = 0;
    check(ttamd_memory_allocated(device_id, nullptr, &total));
    return total;
}

auto BackendAMD::get_device_count() const -> int {
    int count = 0;
    check(ttamd_device_count(&count));
    return count;
}

// ---- the GEMM path -----------------------------------------------------------------------------------------------
auto BackendAMD::batched_matmul(const Tensor &lhs, const Tensor &rhs) const -> Tensor {
    // lhs [B,N,K] . rhs [B,K,M] -> [B,N,M]; the frontend has checked shapes, devices and dtypes
    // (tensor/tensor.cpp:2390-2484).  Both operands are read in place through their strides.
    const int B = lhs.size(0);
    const int N = lhs.size(1);
    const int K = lhs.size(2);
    const int M = rhs.size(2);
    Shape result_shape({B, N, M});
    auto out = make_storage(lhs.device().id, static_cast<std::size_t>(result_shape.numel()), lhs.dtype());
    const ttamd_view3 l = view3(lhs);
    const ttamd_view3 r = view3(rhs);
    check(ttamd_batched_matmul(lhs.device().id, code(lhs.dtype()), B, N, K, M, &l, &r, out->ptr, nullptr, nullptr));
    return make_result(std::move(out), lhs.dtype(), std::move(result_shape), lhs.device());
}

auto BackendAMD::batched_matmul_pair(const Tensor &lhs0, const Tensor &rhs0, const Tensor &lhs1, const Tensor &rhs1) const
    -> std::pair<Tensor, Tensor> {
    if (lhs0.dtype() != lhs1.dtype() || lhs0.device().id != lhs1.device().id) {
        TT_EXCEPTION("batched_matmul_pair: both products must have one dtype and device");
    }
    const ttamd_view3 l0 = view3(lhs0), r0 = view3(rhs0), l1 = view3(lhs1), r1 = view3(rhs1);
    Shape shape0({lhs0.size(0), lhs0.size(1), rhs0.size(2)});
    Shape shape1({lhs1.size(0), lhs1.size(1), rhs1.size(2)});
    auto out0 = make_storage(lhs0.device().id, static_cast<std::size_t>(shape0.numel()), lhs0.dtype());
    auto out1 = make_storage(lhs1.device().id, static_cast<std::size_t>(shape1.numel()), lhs1.dtype());
    const ttamd_product p0{lhs0.size(0), lhs0.size(1), lhs0.size(2), rhs0.size(2), &l0, &r0, out0->ptr, nullptr};
    const ttamd_product p1{lhs1.size(0), lhs1.size(1), lhs1.size(2), rhs1.size(2), &l1, &r1, out1->ptr, nullptr};
    check(ttamd_batched_matmul_pair(lhs0.device().id, code(lhs0.dtype()), &p0, &p1, nullptr));
    return {make_result(std::move(out0), lhs0.dtype(), std::move(shape0), lhs0.device()),
            make_result(std::move(out1), lhs1.dtype(), std::move(shape1), lhs1.device())};
}

auto BackendAMD::conv2d(
    const Tensor &input,
    const Tensor &weight,
    const std::optional<Tensor> &bias,
    int stride,
    int padding
) const -> Tensor {
    const int B = input.size(0);
    const int C = input.size(1);
    const int H = input.size(2);
    const int W = input.size(3);
    const int O = weight.size(0);
    const int k = weight.size(2);
    const int H_out = (H + 2 * padding - k) / stride + 1;
    const int W_out = (W + 2 * padding - k) / stride + 1;
    // the weight is used as the matrix [O, C*k*k] (cpu/conv.cpp:69 reshapes it), the bias as a dense vector
    const Tensor w = weight.contiguous();
    const std::optional<Tensor> b = bias ? std::optional<Tensor>(bias->contiguous()) : std::nullopt;
    Shape result_shape({B, O, H_out, W_out});
    auto out = make_storage(input.device().id, static_cast<std::size_t>(result_shape.numel()), input.dtype());
    const ttamd_view4 iv = view4(input);
    const ttamd_view4 wv = view4(w);
    check(ttamd_conv2d_forward(
        input.device().id, code(input.dtype()), &iv, &wv, b ? data_at_offset(*b) : nullptr, out->ptr, B, C, H, W, O, k, stride,
        padding, nullptr
    ));
    return make_result(std::move(out), input.dtype(), std::move(result_shape), input.device());
}

auto BackendAMD::conv2d_backward(
    const Tensor &grad_output,
    const Tensor &input,
    const Tensor &weight,
    const std::optional<Tensor> &bias,
    int stride,
    int padding
) const -> std::tuple<Tensor, Tensor, std::optional<Tensor>> {
    const int B = input.size(0);
    const int C = input.size(1);
    const int H = input.size(2);
    const int W = input.size(3);
    const int O = weight.size(0);
    const int k = weight.size(2);
    const int device_id = input.device().id;
    const ScalarType dtype = input.dtype();
    const Tensor grad = grad_output.contiguous();
    const Tensor w = weight.contiguous();
    auto grad_input = make_storage(device_id, static_cast<std::size_t>(input.numel()), dtype);
    auto grad_weight = make_storage(device_id, static_cast<std::size_t>(weight.numel()), dtype);
    std::shared_ptr<StorageAMD> grad_bias = bias ? make_storage(device_id, static_cast<std::size_t>(O), dtype) : nullptr;
    std::size_t workspace_bytes = 0;
    check(ttamd_conv2d_backward_workspace(code(dtype), B, C, H, W, O, k, stride, padding, &workspace_bytes));
    // (the workspace goes back to the library's block cache when this scope ends; reuse follows stream order)
    const StorageAMD workspace(device_id, workspace_bytes);
    const ttamd_view4 iv = view4(input);
    const ttamd_view4 wv = view4(w);
    check(ttamd_conv2d_backward(
        device_id, code(dtype), data_at_offset(grad), &iv, &wv, grad_input->ptr, grad_weight->ptr,
        grad_bias ? grad_bias->ptr : nullptr, B, C, H, W, O, k, stride, padding, workspace.ptr, workspace_bytes, nullptr
    ));
    std::optional<Tensor> grad_bias_tensor;
    if (grad_bias) {
        grad_bias_tensor = make_result(std::move(grad_bias), dtype, Shape({O}), input.device());
    }
    return {
        make_result(std::move(grad_input), dtype, input.shape(), input.device()),
        make_result(std::move(grad_weight), dtype, weight.shape(), input.device()),
        std::move(grad_bias_tensor)
    };
}

#define X(NAME, OP)                                                                                                 \
    auto BackendAMD::NAME(const Tensor &input, int kernel_size, int stride, int padding) const -> Tensor {         \
        return pool_forward(input, OP, kernel_size, stride, padding);                                              \
    }                                                                                                               \
    auto BackendAMD::NAME##_backward(                                                                              \
        const Tensor &grad_output,                                                                                 \
        const Tensor &input,                                                                                       \
        const Tensor &result,                                                                                      \
        int kernel_size,                                                                                           \
        int stride,                                                                                                \
        int padding                                                                                                \
    ) const -> Tensor {                                                                                            \
        return pool_backward(grad_output, input, result, OP, kernel_size, stride, padding);                        \
    }
X(max_pool2d, TTAMD_POOL_MAX)
X(min_pool2d, TTAMD_POOL_MIN)
X(avg_pool2d, TTAMD_POOL_AVG)
#undef X

// ---- around the GEMM path ----------------------------------------------------------------------------------------
auto BackendAMD::identity(const Tensor &tensor) const -> Tensor {
    // clone of a view into dense storage: Tensor::contiguous() / clone() (tensor/tensor.cpp:583-596)
    auto out = make_storage(tensor.device().id, static_cast<std::size_t>(tensor.numel()), tensor.dtype());
    const View v(tensor);
    check(ttamd_contiguous(
        tensor.device().id, code(tensor.dtype()), v.ndim, v.shape.data(), v.stride.data(), v.data, v.offset, out->ptr, nullptr
    ));
    return make_result(std::move(out), tensor.dtype(), tensor.shape(), tensor.device());
}

auto BackendAMD::to(const Tensor &tensor, ScalarType dtype) const -> Tensor {
    auto out = make_storage(tensor.device().id, static_cast<std::size_t>(tensor.numel()), dtype);
    const View v(tensor);
    check(ttamd_cast(
        tensor.device().id, code(tensor.dtype()), code(dtype), v.ndim, v.shape.data(), v.data, v.offset, v.stride.data(), out->ptr,
        nullptr
    ));
    return make_result(std::move(out), dtype, tensor.shape(), tensor.device());
}

void BackendAMD::assign(Tensor &lhs, const Tensor &rhs) const {
    assign_view(lhs, rhs);
}

auto BackendAMD::where(const Tensor &cond, const Tensor &lhs, const Tensor &rhs) const -> Tensor {
    auto out = make_storage(lhs.device().id, static_cast<std::size_t>(lhs.numel()), lhs.dtype());
    const View c(cond);
    const View l(lhs);
    const View r(rhs);
    check(ttamd_where(
        lhs.device().id, code(lhs.dtype()), l.ndim, l.shape.data(), c.data, c.offset, c.stride.data(), l.data, l.offset,
        l.stride.data(), r.data, r.offset, r.stride.data(), out->ptr, nullptr
    ));
    return make_result(std::move(out), lhs.dtype(), lhs.shape(), lhs.device());
}

auto BackendAMD::sum(const Tensor &tensor) const -> Tensor {
    return sum_op(tensor, -1);
}

auto BackendAMD::sum(const Tensor &tensor, int dim) const -> Tensor {
    return sum_op(tensor, dim);
}

// all / any of a whole tensor: the number of non-zero elements (a cast to bool writes 0 or 1, its sum is 64-bit)
namespace {
auto count_nonzero(const BackendAMD &backend, const Tensor &tensor) -> int64_t {
    const Tensor flags = tensor.dtype() == kBool ? tensor : backend.to(tensor, kBool);
    return backend.item(sum_op(flags, -1)).to<int64_t>();
}
}    // namespace

auto BackendAMD::all(const Tensor &tensor) const -> bool {
    return count_nonzero(*this, tensor) == static_cast<int64_t>(tensor.numel());
}

auto BackendAMD::any(const Tensor &tensor) const -> bool {
    return count_nonzero(*this, tensor) != 0;
}

// binary operators on the device, and the in-place forms (result into a temporary, then written through lhs's view)
#define TT_AMD_DEVICE_BINARY(X)                                                                                        \
    X(add, TTAMD_BIN_ADD) X(sub, TTAMD_BIN_SUB) X(mul, TTAMD_BIN_MUL) X(div, TTAMD_BIN_DIV) X(pow, TTAMD_BIN_POW)      \
    X(maximum, TTAMD_BIN_MAXIMUM) X(minimum, TTAMD_BIN_MINIMUM) X(lt, TTAMD_BIN_LT) X(le, TTAMD_BIN_LE)                \
    X(gt, TTAMD_BIN_GT) X(ge, TTAMD_BIN_GE) X(eq, TTAMD_BIN_EQ) X(ne, TTAMD_BIN_NE)
#define X(NAME, OP)                                                                     \
    auto BackendAMD::NAME(const Tensor &lhs, const Tensor &rhs) const -> Tensor {      \
        return binary_op(lhs, rhs, OP);                                                \
    }
TT_AMD_DEVICE_BINARY(X)
#undef X
#define X(NAME, OP)                                                          \
    void BackendAMD::NAME##_inplace(Tensor &lhs, const Tensor &rhs) const { \
        assign_view(lhs, binary_op(lhs, rhs, OP));                          \
    }
X(add, TTAMD_BIN_ADD)
X(sub, TTAMD_BIN_SUB)
X(mul, TTAMD_BIN_MUL)
X(div, TTAMD_BIN_DIV)
#undef X

// unary operators on the device, and their in-place forms
#define TT_AMD_DEVICE_UNARY(X)                                                                                         \
    X(relu, TTAMD_UN_RELU) X(negate, TTAMD_UN_NEGATE) X(abs, TTAMD_UN_ABS) X(sqrt, TTAMD_UN_SQRT) X(exp, TTAMD_UN_EXP) \
    X(log, TTAMD_UN_LOG) X(sigmoid, TTAMD_UN_SIGMOID) X(tanh, TTAMD_UN_TANH)
#define X(NAME, OP)                                                    \
    auto BackendAMD::NAME(const Tensor &tensor) const -> Tensor {     \
        return unary_op(tensor, OP);                                  \
    }                                                                  \
    void BackendAMD::NAME##_(Tensor &tensor) const {                   \
        assign_view(tensor, unary_op(tensor, OP));                    \
    }
TT_AMD_DEVICE_UNARY(X)
#undef X

void BackendAMD::identity_(Tensor & /*tensor*/) const {}

// seeded draws: uniform_real and normal
auto BackendAMD::uniform_real(const Tensor &low, const Tensor &high, Generator &gen) const -> Tensor {
    return new_random(0, low, high, gen, "uniform_real");
}
void BackendAMD::uniform_real_(Tensor &tensor, const Tensor &low, const Tensor &high, Generator &gen) const {
    fill_random(tensor, 0, low, high, gen, "uniform_real_");
}
auto BackendAMD::normal(const Tensor &mu, const Tensor &std, Generator &gen) const -> Tensor {
    return new_random(1, mu, std, gen, "normal");
}
void BackendAMD::normal_(Tensor &tensor, const Tensor &mu, const Tensor &std, Generator &gen) const {
    fill_random(tensor, 1, mu, std, gen, "normal_");
}

auto BackendAMD::print(std::ostream &os, const Tensor &tensor) const -> std::ostream & {
    // printing formats host data: through the CPU device's printer on a host copy (Tensor::to goes through to_vec)
    return os << tensor.to(kCPU);
}

// ---- not on the GEMM path ----------------------------------------------------------------------------------------
// Tensor f(const Tensor &) with an in-place twin f_(Tensor &)
#define TT_AMD_MISSING_UNARY(X)                                                                                        \
    X(logical_not) X(sign) X(log10) X(log2) X(log1p) X(exp2) X(expm1) X(sin) X(cos) X(tan) X(asin) X(acos) X(atan)     \
    X(sinh) X(cosh) X(asinh) X(acosh) X(atanh) X(erf) X(erfc) X(tgamma) X(lgamma) X(digamma) X(ceil) X(floor) X(round) \
    X(log_sigmoid) X(hardsigmoid) X(relu6) X(selu) X(silu) X(softsign)
#define X(NAME)                                                        \
    auto BackendAMD::NAME(const Tensor & /*tensor*/) const -> Tensor { \
        not_implemented(#NAME);                                       \
    }                                                                  \
    void BackendAMD::NAME##_(Tensor & /*tensor*/) const {              \
        not_implemented(#NAME "_");                                   \
    }
TT_AMD_MISSING_UNARY(X)
#undef X

// Tensor f(const Tensor &) without an in-place form, and the reductions over one dimension
#define X(NAME)                                                        \
    auto BackendAMD::NAME(const Tensor & /*tensor*/) const -> Tensor { \
        not_implemented(#NAME);                                       \
    }
X(min) X(argmin) X(max) X(argmax) X(isinf) X(isnan) X(isfinite)
#undef X
#define X(NAME)                                                                     \
    auto BackendAMD::NAME(const Tensor & /*tensor*/, int /*dim*/) const -> Tensor { \
        not_implemented(#NAME);                                                    \
    }
X(min) X(argmin) X(max) X(argmax) X(all) X(any) X(softmax) X(log_softmax)
#undef X

// Tensor f(const Tensor &lhs, const Tensor &rhs)
#define X(NAME)                                                                            \
    auto BackendAMD::NAME(const Tensor & /*lhs*/, const Tensor & /*rhs*/) const -> Tensor { \
        not_implemented(#NAME);                                                           \
    }
X(logical_or) X(logical_and) X(bitwise_or) X(bitwise_and) X(bitwise_xor) X(bitwise_left_shift) X(bitwise_right_shift) X(modulo)
#undef X

// distributions other than uniform_real and normal
#define X(NAME, A)                                                                                  \
    auto BackendAMD::NAME(const Tensor & /*A*/, Generator & /*gen*/) const -> Tensor {             \
        not_implemented(#NAME);                                                                    \
    }                                                                                               \
    void BackendAMD::NAME##_(Tensor & /*tensor*/, const Tensor & /*A*/, Generator & /*gen*/) const { \
        not_implemented(#NAME "_");                                                                \
    }
TT_AMD_DIST_ONE(X)
#undef X
#define X(NAME)                                                                                                          \
    auto BackendAMD::NAME(const Tensor & /*a*/, const Tensor & /*b*/, Generator & /*gen*/) const -> Tensor {            \
        not_implemented(#NAME);                                                                                         \
    }                                                                                                                    \
    void BackendAMD::NAME##_(Tensor & /*tensor*/, const Tensor & /*a*/, const Tensor & /*b*/, Generator & /*gen*/) const { \
        not_implemented(#NAME "_");                                                                                     \
    }
X(uniform_int) X(binomial) X(cauchy) X(lognormal) X(weibull)
#undef X

// indexing, clamp, parameterised activations, softmax
auto BackendAMD::index_mask(const Tensor & /*input*/, const Tensor & /*mask*/, int /*N_mask*/) const -> Tensor {
    not_implemented("index_mask");
}
auto BackendAMD::index_indices(const Tensor & /*input*/, const Tensor & /*indices*/) const -> Tensor {
    not_implemented("index_indices");
}
void BackendAMD::index_put_mask(Tensor & /*input*/, const Tensor & /*values*/, const Tensor & /*mask*/) const {
    not_implemented("index_put_mask");
}
void BackendAMD::index_put_indices(Tensor & /*input*/, const Tensor & /*values*/, const Tensor & /*indices*/) const {
    not_implemented("index_put_indices");
}
auto BackendAMD::gather(const Tensor & /*input*/, const Tensor & /*indices*/, int /*idx*/) const -> Tensor {
    not_implemented("gather");
}
void BackendAMD::clamp_(Tensor & /*tensor*/, const Tensor & /*min*/, const Tensor & /*max*/) const {
    not_implemented("clamp_");
}
auto BackendAMD::softplus(const Tensor & /*tensor*/, double /*beta*/, double /*threshold*/) const -> Tensor {
    not_implemented("softplus");
}
auto BackendAMD::leaky_relu(const Tensor & /*tensor*/, double /*negative_slope*/) const -> Tensor {
    not_implemented("leaky_relu");
}
auto BackendAMD::elu(const Tensor & /*tensor*/, double /*alpha*/) const -> Tensor {
    not_implemented("elu");
}
auto BackendAMD::hardtanh(const Tensor & /*tensor*/, double /*min*/, double /*max*/) const -> Tensor {
    not_implemented("hardtanh");
}
void BackendAMD::softplus_(Tensor & /*tensor*/, double /*beta*/, double /*threshold*/) const {
    not_implemented("softplus_");
}
void BackendAMD::leaky_relu_(Tensor & /*tensor*/, double /*negative_slope*/) const {
    not_implemented("leaky_relu_");
}
void BackendAMD::elu_(Tensor & /*tensor*/, double /*alpha*/) const {
    not_implemented("elu_");
}
void BackendAMD::hardtanh_(Tensor & /*tensor*/, double /*min*/, double /*max*/) const {
    not_implemented("hardtanh_");
}
void BackendAMD::softmax_(Tensor & /*tensor*/, int /*dim*/) const {
    not_implemented("softmax_");
}
void BackendAMD::log_softmax_(Tensor & /*tensor*/, int /*dim*/) const {
    not_implemented("log_softmax_");
}

}    // namespace tinytensor::amd
