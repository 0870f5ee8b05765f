// tt_amd.h — C++20 host side of the AMD GEMM backend: the slice of tinytensor's Tensor / backend interface that
// the GEMM path needs, written over the C ABI of include/ttamd.h.  Header-only; link with libttamd.so.
//
// It mirrors the reference's names, argument meaning and error behaviour so that code (and tests) written
// against tinytensor read the same here:
//   Tensor(std::vector<T>, Shape, Device) / to_vec<T>()      include/tt/tensor.h:134-189, 370
//   shape/stride/offset/permute/reshape/expand/...           include/tt/tensor.h:245-283, 600-650 (views only
//                                                            rewrite shape/stride/offset, autograd/shape_ops.cpp:24-146)
//   matmul(lhs, rhs)                                         tinytensor/tensor/tensor.cpp:2390-2484
//   matmul backward (dA = dC.B^T, dB = A^T.dC on views)       tinytensor/autograd/binary_ops.cpp:165-179
//   conv2d / conv2d_backward                                 tinytensor/tensor/tensor.cpp:3089-3167, backend_base.h:269-284
//   nn::Linear (+ default initialisation)                    tinytensor/nn/linear.cpp:20-50, nn/init.cpp:30-52,106-112
//   add/sub/mul/div/pow/..., relu/exp/..., where, sum, full,   tinytensor/tensor/backend_base.h:51-263 (operands are
//   to(dtype), assign                                         broadcast with expand() views first, include/tt/tensor.h:600)
//   max/min/avg_pool2d (+ backward)                          tinytensor/tensor/tensor.cpp:3169-3198, backend_base.h:286-311
//   Generator, uniform_real, normal                          tinytensor/tensor/random.cpp:26-63, tensor.cpp:1773-1781
//   BackendAMD (the BackendBase methods on the path)         tinytensor/tensor/backend_base.h:23-322
//   TTException                                              include/tt/exception.h:15-25
// All arithmetic runs in libttamd.so; there is no CPU fallback.
#ifndef TT_AMD_HOST_H_
#define TT_AMD_HOST_H_

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <exception>
#include <iostream>
#include <memory>
#include <numeric>
#include <optional>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>

#include "ttamd.h"

namespace tt_amd {

class TTException : public std::exception {
public:
    explicit TTException(std::string message) : message_(std::move(message)) {}
    [[nodiscard]] auto what() const noexcept -> const char * override { return message_.c_str(); }

private:
    std::string message_;
};

// Status -> the reference's error model: TTException for user-visible problems, print + exit(1) for
// unrecoverable device failures (TT_ERROR, include/tt/exception.h:28-36).
inline void check(ttamd_status s) {
    if (s == TTAMD_OK) return;
    if (s == TTAMD_ERR_LAUNCH) {
        std::cout << ttamd_last_error_string() << std::endl;
        std::exit(1);
    }
    throw TTException(ttamd_last_error_string());
}

enum class ScalarType { bool8 = 0, u8, i16, i32, i64, f32, f64 };  // include/tt/scalar.h:21-29
constexpr ScalarType kBool = ScalarType::bool8, kU8 = ScalarType::u8, kI16 = ScalarType::i16, kI32 = ScalarType::i32,
                     kI64 = ScalarType::i64, kF32 = ScalarType::f32, kF64 = ScalarType::f64;

template <typename T>
struct to_scalar;
template <> struct to_scalar<bool> { static constexpr ScalarType type = kBool; };
template <> struct to_scalar<uint8_t> { static constexpr ScalarType type = kU8; };
template <> struct to_scalar<int16_t> { static constexpr ScalarType type = kI16; };
template <> struct to_scalar<int32_t> { static constexpr ScalarType type = kI32; };
template <> struct to_scalar<int64_t> { static constexpr ScalarType type = kI64; };
template <> struct to_scalar<float> { static constexpr ScalarType type = kF32; };
template <> struct to_scalar<double> { static constexpr ScalarType type = kF64; };

inline auto dtype_size(ScalarType t) -> std::size_t {
    switch (t) {
    case kBool: case kU8: return 1;
    case kI16: return 2;
    case kI32: case kF32: return 4;
    default: return 8;
    }
}
inline auto promote_types(ScalarType a, ScalarType b) -> ScalarType { return static_cast<int>(a) > static_cast<int>(b) ? a : b; }

enum class Backend { amd };
struct Device {
    Backend backend;
    int id;
    constexpr auto operator==(const Device &other) const -> bool { return backend == other.backend && id == other.id; }
};
constexpr Device kAMD = Device{Backend::amd, 0};

class Shape {  // include/tt/shape.h:20-123
public:
    Shape() = default;
    explicit Shape(std::vector<int> dims) : dims_(std::move(dims)) {}
    Shape(std::initializer_list<int> dims) : dims_(dims) {}
    [[nodiscard]] auto numel() const noexcept -> int {
        return std::accumulate(dims_.begin(), dims_.end(), 1, [](int a, int b) { return a * b; });
    }
    [[nodiscard]] auto ndim() const noexcept -> int { return static_cast<int>(dims_.size()); }
    [[nodiscard]] auto size() const noexcept -> int { return ndim(); }
    auto operator[](int i) -> int & { return dims_.at(static_cast<std::size_t>(i < 0 ? i + ndim() : i)); }
    auto operator[](int i) const -> int { return dims_.at(static_cast<std::size_t>(i < 0 ? i + ndim() : i)); }
    [[nodiscard]] auto to_vec() const -> const std::vector<int> & { return dims_; }
    auto operator==(const Shape &o) const -> bool { return dims_ == o.dims_; }

private:
    std::vector<int> dims_;
};

// Element count of a result, computed in 64 bits: a tensor's numel and every index the library uses fit an int
// (include/tt/shape.h:122), so anything beyond is refused instead of wrapping around into a tiny allocation.
inline auto checked_numel(std::initializer_list<int64_t> extents) -> std::size_t {
    int64_t n = 1;
    for (int64_t e : extents) {
        if (e < 0) throw TTException("negative extent");
        n *= e;
        if (n > static_cast<int64_t>(INT32_MAX)) throw TTException("tensor has more than 2^31 - 1 elements");
    }
    return static_cast<std::size_t>(n);
}

// Owning device allocation (peer of the reference's DeviceMemory<T>, cuda/data_types.cuh:28-101).
class StorageAMD {
public:
    StorageAMD(std::size_t bytes, int device_id) : bytes_(bytes ? bytes : 1), device_(device_id) {
        check(ttamd_malloc(device_, bytes_, &ptr_));
    }
    ~StorageAMD() { ttamd_free(device_, ptr_, bytes_); }
    StorageAMD(const StorageAMD &) = delete;
    StorageAMD &operator=(const StorageAMD &) = delete;
    void *ptr_ = nullptr;
    std::size_t bytes_;
    int device_;
};

class Tensor;
class BackendAMD;
inline auto get_backend(Device device) -> const BackendAMD *;

class Tensor {
public:
    Tensor() = default;
    // Tensor(std::vector<T>, Shape, Device): uploads through BackendBase::from_vec.
    template <typename T>
    Tensor(const std::vector<T> &data, Shape shape, Device device);
    template <typename T>
    Tensor(const std::vector<T> &data, Device device) : Tensor(data, Shape({static_cast<int>(data.size())}), device) {}
    // Internal constructor of backend results (tensor.cpp:351-358) and of views.
    Tensor(std::shared_ptr<StorageAMD> storage, ScalarType dtype, Shape shape, Device device)
        : storage_(std::move(storage)), dtype_(dtype), shape_(std::move(shape)), stride_(dense_stride(shape_)), device_(device) {}
    Tensor(std::shared_ptr<StorageAMD> storage, ScalarType dtype, Shape shape, Shape stride, int offset, Device device)
        : storage_(std::move(storage)), dtype_(dtype), shape_(std::move(shape)), stride_(std::move(stride)), offset_(offset),
          device_(device) {}

    [[nodiscard]] auto dtype() const -> ScalarType { return dtype_; }
    [[nodiscard]] auto device() const -> Device { return device_; }
    [[nodiscard]] auto offset() const -> int { return offset_; }
    [[nodiscard]] auto shape() const -> const Shape & { return shape_; }
    [[nodiscard]] auto stride() const -> const Shape & { return stride_; }
    [[nodiscard]] auto numel() const -> int { return shape_.numel(); }
    [[nodiscard]] auto dim() const -> int { return shape_.ndim(); }
    [[nodiscard]] auto size(int d) const -> int { return shape_[d]; }
    [[nodiscard]] auto is_contiguous() const -> bool { return stride_ == dense_stride(shape_); }
    [[nodiscard]] auto storage() const -> const std::shared_ptr<StorageAMD> & { return storage_; }
    [[nodiscard]] auto data_ptr() const -> void * {
        return static_cast<char *>(storage_->ptr_) + static_cast<std::size_t>(offset_) * dtype_size(dtype_);
    }

    [[nodiscard]] auto contiguous() const -> Tensor;  // tensor.cpp:583-591
    [[nodiscard]] auto permute(const std::vector<int> &dims) const -> Tensor {
        if (static_cast<int>(dims.size()) != dim()) throw TTException("permute: wrong number of dimensions");
        std::vector<int> sh, st, seen(dims.size(), 0);
        for (int d : dims) {
            if (d < 0 || d >= dim() || seen[static_cast<std::size_t>(d)]++) throw TTException("permute: invalid permutation");
            sh.push_back(shape_[d]);
            st.push_back(stride_[d]);
        }
        return {storage_, dtype_, Shape(sh), Shape(st), offset_, device_};
    }
    [[nodiscard]] auto unsqueeze(int d) const -> Tensor {
        if (d < 0) d += dim() + 1;
        auto sh = shape_.to_vec(), st = stride_.to_vec();
        sh.insert(sh.begin() + d, 1);
        st.insert(st.begin() + d, 0);  // a size-1 dimension is never stepped over: a pure view, no clone
        return {storage_, dtype_, Shape(sh), Shape(st), offset_, device_};
    }
    [[nodiscard]] auto squeeze(int d) const -> Tensor {
        if (shape_[d] != 1) return *this;
        auto sh = shape_.to_vec(), st = stride_.to_vec();
        if (d < 0) d += dim();
        sh.erase(sh.begin() + d);
        st.erase(st.begin() + d);
        return {storage_, dtype_, Shape(sh), Shape(st), offset_, device_};
    }
    [[nodiscard]] auto expand(const Shape &shape) const -> Tensor {
        if (shape.ndim() != dim()) throw TTException("expand: rank mismatch");
        std::vector<int> st;
        for (int i = 0; i < dim(); ++i) {
            if (shape_[i] == shape[i]) st.push_back(stride_[i]);
            else if (shape_[i] == 1) st.push_back(0);
            else throw TTException("expand: incompatible shape");
        }
        return {storage_, dtype_, shape, Shape(st), offset_, device_};
    }
    [[nodiscard]] auto reshape(const Shape &shape) const -> Tensor {  // a view when dense, a clone otherwise (tensor.cpp:1371-1387)
        if (shape.numel() != numel()) throw TTException("reshape: element counts differ");
        const Tensor base = contiguous();
        return {base.storage_, dtype_, shape, dense_stride(shape), base.offset_, device_};
    }
    [[nodiscard]] auto flatten(int start_dim = 0, int end_dim = -1) const -> Tensor {
        if (dim() == 0) return reshape(Shape({1}));
        if (start_dim < 0) start_dim += dim();
        if (end_dim < 0) end_dim += dim();
        std::vector<int> sh;
        int merged = 1;
        for (int i = 0; i < dim(); ++i) {
            if (i < start_dim || i > end_dim) sh.push_back(shape_[i]);
            else {
                merged *= shape_[i];
                if (i == end_dim) sh.push_back(merged);
            }
        }
        return reshape(Shape(sh));
    }
    template <typename T>
    [[nodiscard]] auto to_vec() const -> std::vector<T>;  // dense host copy of this view (tensor.cpp:555)
    [[nodiscard]] auto to(ScalarType dtype) const -> Tensor;  // tensor.cpp:534-540
    [[nodiscard]] auto relu() const -> Tensor;
    [[nodiscard]] auto sum() const -> Tensor;
    [[nodiscard]] auto sum(int dim) const -> Tensor;
    auto assign(const Tensor &rhs) -> Tensor &;  // writes rhs's elements through this view
    // Tensor::uniform_real_(low, high, gen) / normal_(mu, std, gen) (tensor.cpp:1783-1801): in place, through this view
    template <typename Gen> auto uniform_real_(double low, double high, Gen &gen) -> Tensor &;
    template <typename Gen> auto normal_(double mu, double std, Gen &gen) -> Tensor &;
    // an uninitialised dense tensor (the layers below overwrite every element; the reference starts from zeros())
    static auto empty(const Shape &shape, ScalarType dtype, Device device) -> Tensor {
        std::vector<int64_t> ext(shape.to_vec().begin(), shape.to_vec().end());
        int64_t n = 1;
        for (int64_t e : ext) n *= e;
        if (n < 0 || n > static_cast<int64_t>(INT32_MAX)) throw TTException("tensor has more than 2^31 - 1 elements");
        return {std::make_shared<StorageAMD>(static_cast<std::size_t>(n) * dtype_size(dtype), device.id), dtype, shape, device};
    }

    static auto dense_stride(const Shape &shape) -> Shape {
        std::vector<int> st(static_cast<std::size_t>(shape.ndim()), 1);
        for (int i = shape.ndim() - 2; i >= 0; --i) st[static_cast<std::size_t>(i)] = st[static_cast<std::size_t>(i) + 1] * shape[i + 1];
        return Shape(st);
    }

private:
    std::shared_ptr<StorageAMD> storage_;
    ScalarType dtype_ = kF32;
    Shape shape_, stride_;
    int offset_ = 0;
    Device device_ = kAMD;
};

// The BackendBase methods that the GEMM path uses (tinytensor/tensor/backend_base.h:23-322).
class BackendAMD {
public:
    template <typename T>
    [[nodiscard]] auto from_vec(const std::vector<T> &data, int device_id) const -> std::shared_ptr<StorageAMD> {
        static_assert(!std::is_same_v<T, bool>, "upload bool data as uint8_t");
        auto st = std::make_shared<StorageAMD>(data.size() * sizeof(T), device_id);
        check(ttamd_memcpy_h2d(device_id, st->ptr_, data.data(), data.size() * sizeof(T)));
        return st;
    }
    // to_vec fills the host vector with the WHOLE storage (backend_base.h:55-60).
    template <typename T>
    void to_vec(const Tensor &tensor, std::vector<T> &data_out) const {
        const auto &st = tensor.storage();
        data_out.resize(st->bytes_ / sizeof(T));
        check(ttamd_memcpy_d2h(st->device_, data_out.data(), st->ptr_, data_out.size() * sizeof(T)));
    }
    [[nodiscard]] auto identity(const Tensor &t) const -> Tensor {  // clone of a view into dense storage
        auto out = std::make_shared<StorageAMD>(static_cast<std::size_t>(t.numel()) * dtype_size(t.dtype()), t.device().id);
        std::vector<int64_t> sh(t.shape().to_vec().begin(), t.shape().to_vec().end()), st(t.stride().to_vec().begin(), t.stride().to_vec().end());
        check(ttamd_contiguous(t.device().id, static_cast<ttamd_dtype>(t.dtype()), t.dim(), sh.data(), st.data(), t.storage()->ptr_,
                               t.offset(), out->ptr_, nullptr));
        return {out, t.dtype(), t.shape(), t.device()};
    }
    // BackendBase::batched_matmul (backend_base.h:130): operands are read in place, whatever their strides.
    [[nodiscard]] auto batched_matmul(const Tensor &lhs, const Tensor &rhs, const ttamd_epilogue *epilogue = nullptr) const -> Tensor {
        const int B = lhs.size(0), N = lhs.size(1), K = lhs.size(2), M = rhs.size(2);
        const ttamd_view3 l = view3(lhs), r = view3(rhs);
        auto out = std::make_shared<StorageAMD>(checked_numel({B, N, M}) * dtype_size(lhs.dtype()), lhs.device().id);
        check(ttamd_batched_matmul(lhs.device().id, static_cast<ttamd_dtype>(lhs.dtype()), B, N, K, M, &l, &r, out->ptr_, epilogue, nullptr));
        return {out, lhs.dtype(), Shape({B, N, M}), lhs.device()};
    }
    // Two independent products in one call (ttamd_batched_matmul_pair): what TensorBatchedMatmul::backward
    // (autograd/binary_ops.cpp:173-179) asks of the backend for its two gradients.
    [[nodiscard]] auto batched_matmul_pair(const Tensor &lhs0, const Tensor &rhs0, const ttamd_epilogue *ep0, const Tensor &lhs1,
                                           const Tensor &rhs1, const ttamd_epilogue *ep1) const -> std::pair<Tensor, Tensor> {
        if (lhs0.dtype() != lhs1.dtype() || lhs0.device().id != lhs1.device().id) throw TTException("batched_matmul_pair: one dtype and device");
        const ttamd_view3 l0 = view3(lhs0), r0 = view3(rhs0), l1 = view3(lhs1), r1 = view3(rhs1);
        ttamd_product p0{lhs0.size(0), lhs0.size(1), lhs0.size(2), rhs0.size(2), &l0, &r0, nullptr, ep0};
        ttamd_product p1{lhs1.size(0), lhs1.size(1), lhs1.size(2), rhs1.size(2), &l1, &r1, nullptr, ep1};
        auto out0 = std::make_shared<StorageAMD>(checked_numel({p0.B, p0.N, p0.M}) * dtype_size(lhs0.dtype()), lhs0.device().id);
        auto out1 = std::make_shared<StorageAMD>(checked_numel({p1.B, p1.N, p1.M}) * dtype_size(lhs1.dtype()), lhs1.device().id);
        p0.out = out0->ptr_;
        p1.out = out1->ptr_;
        check(ttamd_batched_matmul_pair(lhs0.device().id, static_cast<ttamd_dtype>(lhs0.dtype()), &p0, &p1, nullptr));
        return {Tensor{out0, lhs0.dtype(), Shape({p0.B, p0.N, p0.M}), lhs0.device()}, Tensor{out1, lhs1.dtype(), Shape({p1.B, p1.N, p1.M}), lhs1.device()}};
    }
    [[nodiscard]] auto conv2d(const Tensor &input, const Tensor &weight, const std::optional<Tensor> &bias, int stride, int padding) const
        -> Tensor {
        const int B = input.size(0), C = input.size(1), H = input.size(2), W = input.size(3), O = weight.size(0), k = weight.size(2);
        const int Ho = (H + 2 * padding - k) / stride + 1, Wo = (W + 2 * padding - k) / stride + 1;
        const Tensor w = weight.contiguous();  // used as the matrix [O, C*k*k], as cpu/conv.cpp:69 reshapes it
        const std::optional<Tensor> b = bias ? std::optional<Tensor>(bias->contiguous()) : std::nullopt;
        const ttamd_view4 iv = view4(input), wv = view4(w);
        if (Ho <= 0 || Wo <= 0) throw TTException("conv2d: the kernel does not fit the padded input");
        checked_numel({B, C, H, W});
        auto out = std::make_shared<StorageAMD>(checked_numel({B, O, Ho, Wo}) * dtype_size(input.dtype()), input.device().id);
        check(ttamd_conv2d_forward(input.device().id, static_cast<ttamd_dtype>(input.dtype()), &iv, &wv, b ? b->data_ptr() : nullptr, out->ptr_,
                                   B, C, H, W, O, k, stride, padding, nullptr));
        return {out, input.dtype(), Shape({B, O, Ho, Wo}), input.device()};
    }
    [[nodiscard]] auto conv2d_backward(const Tensor &grad_output, const Tensor &input, const Tensor &weight, const std::optional<Tensor> &bias,
                                       int stride, int padding) const -> std::tuple<Tensor, Tensor, std::optional<Tensor>> {
        const int B = input.size(0), C = input.size(1), H = input.size(2), W = input.size(3), O = weight.size(0), k = weight.size(2);
        const int dev = input.device().id;
        const auto dt = static_cast<ttamd_dtype>(input.dtype());
        const std::size_t esz = dtype_size(input.dtype());
        const Tensor go = grad_output.contiguous(), w = weight.contiguous();
        auto gx = std::make_shared<StorageAMD>(checked_numel({B, C, H, W}) * esz, dev);
        auto gw = std::make_shared<StorageAMD>(checked_numel({O, C, k, k}) * esz, dev);
        std::shared_ptr<StorageAMD> gb = bias ? std::make_shared<StorageAMD>(static_cast<std::size_t>(O) * esz, dev) : nullptr;
        std::size_t ws_bytes = 0;
        check(ttamd_conv2d_backward_workspace(dt, B, C, H, W, O, k, stride, padding, &ws_bytes));
        StorageAMD ws(ws_bytes, dev);
        const ttamd_view4 iv = view4(input), wv = view4(w);
        check(ttamd_conv2d_backward(dev, dt, go.data_ptr(), &iv, &wv, gx->ptr_, gw->ptr_, gb ? gb->ptr_ : nullptr, B, C, H, W, O, k, stride,
                                    padding, ws.ptr_, ws_bytes, nullptr));
        // (no wait for the kernels: the workspace goes back to the allocator in stream order when this scope ends)
        std::optional<Tensor> grad_bias;
        if (gb) grad_bias = Tensor(gb, input.dtype(), Shape({O}), input.device());
        return {Tensor(gx, input.dtype(), input.shape(), input.device()), Tensor(gw, input.dtype(), weight.shape(), input.device()), grad_bias};
    }
    // ---- elementwise set (backend_base.h:51-263): operands share one shape; results are dense ----
    [[nodiscard]] auto binary(const Tensor &lhs, const Tensor &rhs, ttamd_binary_op op) const -> Tensor {
        if (!(lhs.shape() == rhs.shape()) || lhs.dtype() != rhs.dtype()) throw TTException("binary op: operands must share shape and dtype");
        const ScalarType rt = op >= TTAMD_BIN_LT ? kBool : lhs.dtype();
        auto out = std::make_shared<StorageAMD>(static_cast<std::size_t>(lhs.numel()) * dtype_size(rt), lhs.device().id);
        const auto sh = i64(lhs.shape()), ls = i64(lhs.stride()), rs = i64(rhs.stride());
        check(ttamd_binary(lhs.device().id, static_cast<ttamd_dtype>(lhs.dtype()), op, lhs.dim(), sh.data(), lhs.storage()->ptr_, lhs.offset(),
                           ls.data(), rhs.storage()->ptr_, rhs.offset(), rs.data(), out->ptr_, nullptr));
        return {out, rt, lhs.shape(), lhs.device()};
    }
#define TT_AMD_BINARY(NAME, CODE) \
    [[nodiscard]] auto NAME(const Tensor &lhs, const Tensor &rhs) const -> Tensor { return binary(lhs, rhs, CODE); }
    TT_AMD_BINARY(add, TTAMD_BIN_ADD)
    TT_AMD_BINARY(sub, TTAMD_BIN_SUB)
    TT_AMD_BINARY(mul, TTAMD_BIN_MUL)
    TT_AMD_BINARY(div, TTAMD_BIN_DIV)
    TT_AMD_BINARY(pow, TTAMD_BIN_POW)
    TT_AMD_BINARY(maximum, TTAMD_BIN_MAXIMUM)
    TT_AMD_BINARY(minimum, TTAMD_BIN_MINIMUM)
    TT_AMD_BINARY(lt, TTAMD_BIN_LT)
    TT_AMD_BINARY(le, TTAMD_BIN_LE)
    TT_AMD_BINARY(gt, TTAMD_BIN_GT)
    TT_AMD_BINARY(ge, TTAMD_BIN_GE)
    TT_AMD_BINARY(eq, TTAMD_BIN_EQ)
    TT_AMD_BINARY(ne, TTAMD_BIN_NE)
#undef TT_AMD_BINARY
    [[nodiscard]] auto unary(const Tensor &t, ttamd_unary_op op) const -> Tensor {
        auto out = std::make_shared<StorageAMD>(static_cast<std::size_t>(t.numel()) * dtype_size(t.dtype()), t.device().id);
        const auto sh = i64(t.shape()), st = i64(t.stride());
        check(ttamd_unary(t.device().id, static_cast<ttamd_dtype>(t.dtype()), op, t.dim(), sh.data(), t.storage()->ptr_, t.offset(), st.data(),
                          out->ptr_, nullptr));
        return {out, t.dtype(), t.shape(), t.device()};
    }
#define TT_AMD_UNARY(NAME, CODE) \
    [[nodiscard]] auto NAME(const Tensor &t) const -> Tensor { return unary(t, CODE); }
    TT_AMD_UNARY(relu, TTAMD_UN_RELU)
    TT_AMD_UNARY(negate, TTAMD_UN_NEGATE)
    TT_AMD_UNARY(abs, TTAMD_UN_ABS)
    TT_AMD_UNARY(sqrt, TTAMD_UN_SQRT)
    TT_AMD_UNARY(exp, TTAMD_UN_EXP)
    TT_AMD_UNARY(log, TTAMD_UN_LOG)
    TT_AMD_UNARY(sigmoid, TTAMD_UN_SIGMOID)
    TT_AMD_UNARY(tanh, TTAMD_UN_TANH)
#undef TT_AMD_UNARY
    [[nodiscard]] auto where(const Tensor &cond, const Tensor &lhs, const Tensor &rhs) const -> Tensor {
        if (cond.dtype() != kBool || !(cond.shape() == lhs.shape()) || !(lhs.shape() == rhs.shape()) || lhs.dtype() != rhs.dtype())
            throw TTException("where: cond must be bool and all operands must share one shape");
        auto out = std::make_shared<StorageAMD>(static_cast<std::size_t>(lhs.numel()) * dtype_size(lhs.dtype()), lhs.device().id);
        const auto sh = i64(lhs.shape()), cs = i64(cond.stride()), ls = i64(lhs.stride()), rs = i64(rhs.stride());
        check(ttamd_where(lhs.device().id, static_cast<ttamd_dtype>(lhs.dtype()), lhs.dim(), sh.data(), cond.storage()->ptr_, cond.offset(),
                          cs.data(), lhs.storage()->ptr_, lhs.offset(), ls.data(), rhs.storage()->ptr_, rhs.offset(), rs.data(), out->ptr_,
                          nullptr));
        return {out, lhs.dtype(), lhs.shape(), lhs.device()};
    }
    // sum(tensor) -> one element; sum(tensor, dim) -> that dimension removed (backend_base.h:148-149).  bool and the
    // integer dtypes are summed in 64 bits and the result is i64 (common/reduce.h:56-61).
    [[nodiscard]] auto sum(const Tensor &t, int dim = -1) const -> Tensor {
        const ScalarType rt = (t.dtype() == kF32 || t.dtype() == kF64) ? t.dtype() : kI64;
        std::vector<int> osh;
        if (dim < 0) osh = {1};
        else
            for (int d = 0; d < t.dim(); ++d)
                if (d != dim) osh.push_back(t.size(d));
        const Shape out_shape{osh};
        auto out = std::make_shared<StorageAMD>(static_cast<std::size_t>(out_shape.numel()) * dtype_size(rt), t.device().id);
        const auto sh = i64(t.shape()), st = i64(t.stride());
        check(ttamd_sum(t.device().id, static_cast<ttamd_dtype>(t.dtype()), t.dim(), sh.data(), t.storage()->ptr_, t.offset(), st.data(), dim,
                        out->ptr_, nullptr));
        return {out, rt, out_shape, t.device()};
    }
    template <typename T>
    [[nodiscard]] auto full(T value, int numel, Device device) const -> Tensor {  // backend_base.h:51
        using S = std::conditional_t<std::is_same_v<T, bool>, uint8_t, T>;
        const S v = static_cast<S>(value);
        auto out = std::make_shared<StorageAMD>(static_cast<std::size_t>(numel) * sizeof(S), device.id);
        check(ttamd_full(device.id, static_cast<ttamd_dtype>(to_scalar<T>::type), &v, numel, out->ptr_, nullptr));
        return {out, to_scalar<T>::type, Shape({numel}), device};
    }
    [[nodiscard]] auto to(const Tensor &t, ScalarType dtype) const -> Tensor {  // backend_base.h:74
        auto out = std::make_shared<StorageAMD>(static_cast<std::size_t>(t.numel()) * dtype_size(dtype), t.device().id);
        const auto sh = i64(t.shape()), st = i64(t.stride());
        check(ttamd_cast(t.device().id, static_cast<ttamd_dtype>(t.dtype()), static_cast<ttamd_dtype>(dtype), t.dim(), sh.data(),
                         t.storage()->ptr_, t.offset(), st.data(), out->ptr_, nullptr));
        return {out, dtype, t.shape(), t.device()};
    }
    void assign(Tensor &lhs, const Tensor &rhs) const {  // backend_base.h:78
        if (!(lhs.shape() == rhs.shape()) || lhs.dtype() != rhs.dtype()) throw TTException("assign: operands must share shape and dtype");
        const auto sh = i64(lhs.shape()), ls = i64(lhs.stride()), rs = i64(rhs.stride());
        check(ttamd_assign(lhs.device().id, static_cast<ttamd_dtype>(lhs.dtype()), lhs.dim(), sh.data(), lhs.storage()->ptr_, lhs.offset(),
                           ls.data(), rhs.storage()->ptr_, rhs.offset(), rs.data(), nullptr));
    }
    // ---- pooling (backend_base.h:286-311) ----
    [[nodiscard]] auto pool2d(const Tensor &input, ttamd_pool_op op, int kernel_size, int stride, int padding) const -> Tensor {
        const int B = input.size(0), C = input.size(1), H = input.size(2), W = input.size(3);
        const int Ho = (H + 2 * padding - kernel_size) / stride + 1, Wo = (W + 2 * padding - kernel_size) / stride + 1;
        const bool is_float = input.dtype() == kF32 || input.dtype() == kF64;
        const ScalarType rt = (op == TTAMD_POOL_AVG && !is_float) ? kF32 : input.dtype();  // common/reduce.h:63-69
        if (Ho <= 0 || Wo <= 0) throw TTException("pool2d: the window does not fit the padded input");
        auto out = std::make_shared<StorageAMD>(checked_numel({B, C, Ho, Wo}) * dtype_size(rt), input.device().id);
        const ttamd_view4 iv = view4(input);
        check(ttamd_pool2d_forward(input.device().id, static_cast<ttamd_dtype>(input.dtype()), op, &iv, out->ptr_, B, C, H, W, kernel_size,
                                   stride, padding, nullptr));
        return {out, rt, Shape({B, C, Ho, Wo}), input.device()};
    }
    [[nodiscard]] auto pool2d_backward(const Tensor &grad_output, const Tensor &input, const Tensor &result, ttamd_pool_op op, int kernel_size,
                                       int stride, int padding) const -> Tensor {
        const Tensor go = grad_output.contiguous(), res = result.contiguous();
        auto gx = std::make_shared<StorageAMD>(static_cast<std::size_t>(input.numel()) * dtype_size(input.dtype()), input.device().id);
        const ttamd_view4 iv = view4(input);
        check(ttamd_pool2d_backward(input.device().id, static_cast<ttamd_dtype>(input.dtype()), op, go.data_ptr(), &iv, res.data_ptr(), gx->ptr_,
                                    input.size(0), input.size(1), input.size(2), input.size(3), kernel_size, stride, padding, nullptr));
        return {gx, input.dtype(), input.shape(), input.device()};
    }
#define TT_AMD_POOL(NAME, CODE)                                                                                                    \
    [[nodiscard]] auto NAME(const Tensor &input, int kernel_size, int stride, int padding) const -> Tensor {                      \
        return pool2d(input, CODE, kernel_size, stride, padding);                                                                  \
    }                                                                                                                              \
    [[nodiscard]] auto NAME##_backward(const Tensor &grad_output, const Tensor &input, const Tensor &result, int kernel_size,     \
                                       int stride, int padding) const -> Tensor {                                                 \
        return pool2d_backward(grad_output, input, result, CODE, kernel_size, stride, padding);                                    \
    }
    TT_AMD_POOL(max_pool2d, TTAMD_POOL_MAX)
    TT_AMD_POOL(min_pool2d, TTAMD_POOL_MIN)
    TT_AMD_POOL(avg_pool2d, TTAMD_POOL_AVG)
#undef TT_AMD_POOL
    // ---- seeded draws (backend_base.h:96-103 with scalar parameters): dist 0 uniform_real(low, high), 1 normal(mu, std) ----
    [[nodiscard]] auto random_fill(int dist, double p0, double p1, const Shape &shape, uint64_t &generator_state, ScalarType dtype,
                                   Device device) const -> Tensor {
        auto out = std::make_shared<StorageAMD>(static_cast<std::size_t>(shape.numel()) * dtype_size(dtype), device.id);
        check(ttamd_random_fill(device.id, static_cast<ttamd_dtype>(dtype), dist, p0, p1, &generator_state, shape.numel(), out->ptr_, nullptr));
        return {out, dtype, shape, device};
    }
    // BackendBase::uniform_real_ / normal_ (backend_base.h:96-103), scalar parameters: written in place through the
    // view `t`; element i of the view takes the i-th draw (cpu/kernel/distribution.hpp:28-32).
    void random_fill_(const Tensor &t, int dist, double p0, double p1, uint64_t &generator_state) const {
        const auto sh = i64(t.shape()), st = i64(t.stride());
        check(ttamd_random_fill_view(t.device().id, static_cast<ttamd_dtype>(t.dtype()), dist, p0, p1, &generator_state, t.dim(), sh.data(),
                                     st.data(), t.storage()->ptr_, t.offset(), nullptr));
    }
    [[nodiscard]] auto current_memory_allocated(int device_id) const -> uint64_t {
        uint64_t cur = 0, tot = 0;
        check(ttamd_memory_allocated(device_id, &cur, &tot));
        return cur;
    }
    [[nodiscard]] auto total_memory_allocated(int device_id) const -> uint64_t {
        uint64_t cur = 0, tot = 0;
        check(ttamd_memory_allocated(device_id, &cur, &tot));
        return tot;
    }
    // Returns the blocks kept by the library's caching allocator to the driver (waits for the device).
    void empty_cache(int device_id) const { check(ttamd_empty_cache(device_id)); }
    [[nodiscard]] auto get_device_count() const -> int {
        int n = 0;
        check(ttamd_device_count(&n));
        return n;
    }

    static auto i64(const Shape &s) -> std::vector<int64_t> {
        std::vector<int64_t> v(s.to_vec().begin(), s.to_vec().end());
        if (v.empty()) v.push_back(1);  // rank 0: the C ABI wants non-NULL arrays
        return v;
    }
    static auto view3(const Tensor &t) -> ttamd_view3 {
        return {t.storage()->ptr_, t.offset(), {t.stride()[0], t.stride()[1], t.stride()[2]}};
    }
    static auto view4(const Tensor &t) -> ttamd_view4 {
        return {t.storage()->ptr_, t.offset(), {t.stride()[0], t.stride()[1], t.stride()[2], t.stride()[3]}};
    }
};

inline auto get_backend(Device) -> const BackendAMD * {  // backend_register.cpp:19-38
    static const std::unique_ptr<BackendAMD> backend = std::make_unique<BackendAMD>();
    return backend.get();
}

template <typename T>
Tensor::Tensor(const std::vector<T> &data, Shape shape, Device device) : dtype_(to_scalar<T>::type), shape_(std::move(shape)), device_(device) {
    if (shape_.numel() != static_cast<int>(data.size())) throw TTException("Tensor: data size does not match the shape");
    stride_ = dense_stride(shape_);
    if constexpr (std::is_same_v<T, bool>) {
        std::vector<uint8_t> bytes(data.begin(), data.end());  // bool is stored as uint8_t (backend_base.h:36-37)
        storage_ = get_backend(device)->from_vec(bytes, device.id);
    } else {
        storage_ = get_backend(device)->from_vec(data, device.id);
    }
}

inline auto Tensor::contiguous() const -> Tensor { return is_contiguous() ? *this : get_backend(device_)->identity(*this); }

template <typename T>
auto Tensor::to_vec() const -> std::vector<T> {
    if (to_scalar<T>::type != dtype_) throw TTException("to_vec: element type does not match the tensor dtype");
    const Tensor dense = contiguous();  // callers clone first (tensor.cpp:555), then the whole storage comes back
    std::vector<std::conditional_t<std::is_same_v<T, bool>, uint8_t, T>> whole;  // bool travels as bytes (tensor.cpp:558-564)
    get_backend(device_)->to_vec(dense, whole);
    return {whole.begin() + dense.offset(), whole.begin() + dense.offset() + dense.numel()};
}

// tinytensor::matmul (tensor.cpp:2390-2484): rank dispatch onto batched_matmul; bool is rejected.
inline auto matmul(const Tensor &lhs_, const Tensor &rhs_) -> Tensor {
    if (!(lhs_.device() == rhs_.device())) throw TTException("Expected tensors on the same device");
    const auto promoted = promote_types(lhs_.dtype(), rhs_.dtype());
    if (promoted == kBool) throw TTException("matmul does not support boolean tensors");
    const Tensor lhs = lhs_.to(promoted), rhs = rhs_.to(promoted);  // check_promote (tensor.cpp:2398-2399)
    const auto *be = get_backend(lhs.device());
    const auto &ls = lhs.shape(), &rs = rhs.shape();
    if (ls.ndim() == 1 && rs.ndim() == 1) {
        if (ls[0] != rs[0]) throw TTException("Invalid shapes for dot product. Both LHS and RHS must have same dimensions");
        return be->batched_matmul(lhs.reshape({1, 1, ls[0]}), rhs.reshape({1, rs[0], 1})).flatten();
    }
    if (ls.ndim() == 1 && rs.ndim() == 2) {
        if (ls[0] != rs[0]) throw TTException("Invalid shape for matrix multiplication. Length of LHS should equal size of RHS dimension 0");
        return be->batched_matmul(lhs.reshape({1, 1, ls[0]}), rhs.unsqueeze(0)).flatten();
    }
    if (ls.ndim() == 2 && rs.ndim() == 1) {
        if (ls[1] != rs[0]) throw TTException("Invalid shape for matrix multiplication. Length of RHS should equal size of LHS dimension 1");
        return be->batched_matmul(lhs.unsqueeze(0), rhs.reshape({1, rs[0], 1})).flatten();
    }
    if (ls.ndim() == 2 && rs.ndim() == 2) {
        if (ls[1] != rs[0]) throw TTException("Invalid shape for matrix multiplication. Size of LHS dimension 1 should equal size of RHS dimension 0");
        return be->batched_matmul(lhs.unsqueeze(0), rhs.unsqueeze(0)).squeeze(0);
    }
    if (ls.ndim() == 3 && rs.ndim() == 3) {
        if (ls[2] != rs[1] || ls[0] != rs[0]) throw TTException("Invalid shape for batched matrix multiplication");
        return be->batched_matmul(lhs, rhs);
    }
    throw TTException("Unsupported sizes. Try reshaping or broadcasting.");
}

// TensorBatchedMatmul::backward (autograd/binary_ops.cpp:173-179): both gradients, on permuted VIEWS.
inline auto matmul_backward(const Tensor &lhs, const Tensor &rhs, const Tensor &grad_output) -> std::pair<Tensor, Tensor> {
    if (lhs.dim() == 3 && rhs.dim() == 3 && grad_output.dim() == 3 && lhs.dtype() == rhs.dtype() && lhs.dtype() == grad_output.dtype() &&
        lhs.dtype() != kBool && lhs.size(0) == rhs.size(0) && lhs.size(2) == rhs.size(1) && grad_output.size(0) == lhs.size(0) &&
        grad_output.size(1) == lhs.size(1) && grad_output.size(2) == rhs.size(2))
        // what forward stored: 3-D operands of one dtype -- both products in one backend call (one grid where that pays)
        return get_backend(lhs.device())->batched_matmul_pair(grad_output, rhs.permute({0, 2, 1}), nullptr, lhs.permute({0, 2, 1}), grad_output, nullptr);
    return {matmul(grad_output, rhs.permute({0, 2, 1})), matmul(lhs.permute({0, 2, 1}), grad_output)};
}

// tinytensor::conv2d argument checks (tensor.cpp:3089-3167).
inline auto conv2d(const Tensor &input, const Tensor &weight, const std::optional<Tensor> &bias = {}, int stride = 1, int padding = 0) -> Tensor {
    if (input.dim() != 4 || weight.dim() != 4) throw TTException("conv2d expects 4-D input [B,C,H,W] and weight [O,C,k,k]");
    if (input.size(1) != weight.size(1)) throw TTException("conv2d: input channels do not match weight channels");
    if (weight.size(2) != weight.size(3)) throw TTException("conv2d: only square kernels are supported");
    if (stride <= 0 || padding < 0) throw TTException("conv2d: stride must be > 0 and padding >= 0");
    if (bias && (bias->dim() != 1 || bias->size(0) != weight.size(0))) throw TTException("conv2d: bias must have one entry per output channel");
    if (input.dtype() != weight.dtype() || input.dtype() == kBool) throw TTException("conv2d: operands must share one non-bool dtype");
    return get_backend(input.device())->conv2d(input, weight, bias, stride, padding);
}
inline auto conv2d_backward(const Tensor &grad_output, const Tensor &input, const Tensor &weight, const std::optional<Tensor> &bias = {},
                            int stride = 1, int padding = 0) {
    return get_backend(input.device())->conv2d_backward(grad_output, input, weight, bias, stride, padding);
}

inline auto Tensor::to(ScalarType dtype) const -> Tensor { return dtype == dtype_ ? *this : get_backend(device_)->to(*this, dtype); }
inline auto Tensor::relu() const -> Tensor { return get_backend(device_)->relu(*this); }
inline auto Tensor::sum() const -> Tensor { return get_backend(device_)->sum(*this); }
inline auto Tensor::sum(int dim) const -> Tensor { return get_backend(device_)->sum(*this, dim < 0 ? dim + this->dim() : dim); }
inline auto Tensor::assign(const Tensor &rhs) -> Tensor & {
    get_backend(device_)->assign(*this, rhs);
    return *this;
}

// Right-aligned broadcasting through unsqueeze + expand views (no data movement), then one shape for the backend.
inline auto broadcast_tensors(Tensor a, Tensor b) -> std::pair<Tensor, Tensor> {
    while (a.dim() < b.dim()) a = a.unsqueeze(0);
    while (b.dim() < a.dim()) b = b.unsqueeze(0);
    std::vector<int> sh;
    for (int d = 0; d < a.dim(); ++d) {
        if (a.size(d) != b.size(d) && a.size(d) != 1 && b.size(d) != 1) throw TTException("Tensors are not broadcastable");
        sh.push_back(std::max(a.size(d), b.size(d)));
    }
    return {a.expand(Shape(sh)), b.expand(Shape(sh))};
}
#define TT_AMD_FREE_BINARY(NAME)                                                                 \
    inline auto NAME(const Tensor &lhs, const Tensor &rhs) -> Tensor {                           \
        /* operands are cast to promote_types(lhs, rhs) (tensor/tensor.cpp:2272-2274) */         \
        const auto promoted = promote_types(lhs.dtype(), rhs.dtype());                           \
        const auto [l, r] = broadcast_tensors(lhs.dtype() == promoted ? lhs : lhs.to(promoted),  \
                                              rhs.dtype() == promoted ? rhs : rhs.to(promoted)); \
        return get_backend(lhs.device())->NAME(l, r);                                            \
    }
TT_AMD_FREE_BINARY(add)
TT_AMD_FREE_BINARY(sub)
TT_AMD_FREE_BINARY(mul)
TT_AMD_FREE_BINARY(div)
TT_AMD_FREE_BINARY(pow)
TT_AMD_FREE_BINARY(maximum)
TT_AMD_FREE_BINARY(minimum)
TT_AMD_FREE_BINARY(lt)
TT_AMD_FREE_BINARY(le)
TT_AMD_FREE_BINARY(gt)
TT_AMD_FREE_BINARY(ge)
TT_AMD_FREE_BINARY(eq)
TT_AMD_FREE_BINARY(ne)
#undef TT_AMD_FREE_BINARY
inline auto operator+(const Tensor &a, const Tensor &b) -> Tensor { return add(a, b); }
inline auto operator-(const Tensor &a, const Tensor &b) -> Tensor { return sub(a, b); }
inline auto operator*(const Tensor &a, const Tensor &b) -> Tensor { return mul(a, b); }
inline auto operator/(const Tensor &a, const Tensor &b) -> Tensor { return div(a, b); }
inline auto operator<(const Tensor &a, const Tensor &b) -> Tensor { return lt(a, b); }
inline auto operator>(const Tensor &a, const Tensor &b) -> Tensor { return gt(a, b); }
inline auto relu(const Tensor &t) -> Tensor { return t.relu(); }
inline auto where(const Tensor &cond, const Tensor &lhs, const Tensor &rhs) -> Tensor {
    const auto [l, r] = broadcast_tensors(lhs, rhs);
    const auto [c, l2] = broadcast_tensors(cond, l);
    const auto [c2, r2] = broadcast_tensors(c, r);
    return get_backend(lhs.device())->where(c2, l2, r2);
}
// tinytensor::full: a one-element storage expanded to `shape` (stride 0), like Tensor(Scalar).expand().
template <typename T>
inline auto full(T value, const Shape &shape, Device device = kAMD) -> Tensor {
    const Tensor one = get_backend(device)->full(value, 1, device);
    return {one.storage(), one.dtype(), shape, Shape(std::vector<int>(static_cast<std::size_t>(shape.ndim()), 0)), 0, device};
}

// tinytensor::{max,min,avg}_pool2d argument checks (tensor.cpp:3169-3198).
#define TT_AMD_FREE_POOL(NAME)                                                                                                        \
    inline auto NAME(const Tensor &input, int kernel_size, int stride, int padding) -> Tensor {                                      \
        if (input.dtype() == kBool) throw TTException(#NAME " does not support boolean tensors");                                     \
        if (input.dim() != 4) throw TTException("Input shape expected to have 4 dimensions.");                                        \
        if (stride <= 0) throw TTException("Stide is expected to be positive.");                                                      \
        if (padding < 0) throw TTException("Padding is expected to be non-negative.");                                                \
        if (input.size(2) + padding < kernel_size || input.size(3) + padding < kernel_size)                                           \
            throw TTException("Kernel size cannot be greater than input size + padding");                                            \
        return get_backend(input.device())->NAME(input, kernel_size, stride, padding);                                                \
    }                                                                                                                                 \
    inline auto NAME##_backward(const Tensor &grad_output, const Tensor &input, const Tensor &result, int kernel_size, int stride,    \
                                int padding) -> Tensor {                                                                              \
        return get_backend(input.device())->NAME##_backward(grad_output, input, result, kernel_size, stride, padding);                \
    }
TT_AMD_FREE_POOL(max_pool2d)
TT_AMD_FREE_POOL(min_pool2d)
TT_AMD_FREE_POOL(avg_pool2d)
#undef TT_AMD_FREE_POOL

// tinytensor::Generator (tensor/random.cpp:46-63): state = splitmix64(seed); the device draws advance it.
class Generator {
public:
    explicit Generator(uint64_t seed = 0) {
        uint64_t r = seed + 0x9E3779B97F4A7C15ull;
        r = (r ^ (r >> 30)) * 0xBF58476D1CE4E5B9ull;
        r = (r ^ (r >> 27)) * 0x94D049BB133111EBull;
        state = r ^ (r >> 31);
    }
    uint64_t state;
};
// tinytensor::uniform_real(low, high, shape, options, gen) (tensor.cpp:1773-1781) and normal.
inline auto uniform_real(double low, double high, const Shape &shape, Generator &gen, ScalarType dtype = kF32, Device device = kAMD) -> Tensor {
    if (!(low < high)) throw TTException("Expected low < high. At least one element violates this.");
    return get_backend(device)->random_fill(0, low, high, shape, gen.state, dtype, device);
}
inline auto normal(double mu, double std, const Shape &shape, Generator &gen, ScalarType dtype = kF32, Device device = kAMD) -> Tensor {
    return get_backend(device)->random_fill(1, mu, std, shape, gen.state, dtype, device);
}

template <typename Gen>
auto Tensor::uniform_real_(double low, double high, Gen &gen) -> Tensor & {
    if (dtype_ != kF32 && dtype_ != kF64) throw TTException("uniform_real_ expects a floating point tensor");
    if (!(low < high)) throw TTException("Expected low < high. At least one element violates this.");
    get_backend(device_)->random_fill_(*this, 0, low, high, gen.state);
    return *this;
}
template <typename Gen>
auto Tensor::normal_(double mu, double std, Gen &gen) -> Tensor & {
    if (dtype_ != kF32 && dtype_ != kF64) throw TTException("normal_ expects a floating point tensor");
    get_backend(device_)->random_fill_(*this, 1, mu, std, gen.state);
    return *this;
}

namespace nn {
// nn::calc_fan_in_out (nn/init.cpp:30-52): both fans are size(0) times the receptive field (the sizes beyond dim 1).
inline auto calc_fan_in_out(const Tensor &tensor) -> std::tuple<double, double> {
    if (tensor.dim() < 2) throw TTException("Unable to calculate fan in and fan out for tensors with dimensions fewer than 2");
    int field = 1;
    for (int i = 2; i < tensor.dim(); ++i) field *= tensor.size(i);
    const double fan = static_cast<double>(tensor.size(0) * field);
    return {fan, fan};
}
// nn::kaiming_uniform_ (nn/init.cpp:106-112), fan_in mode: U(+-sqrt(3) * gain / sqrt(fan)), drawn in place.
inline void kaiming_uniform_(Tensor tensor, Generator &gen, double gain = 1.0) {
    const auto [fan_in, fan_out] = calc_fan_in_out(tensor);
    (void)fan_out;
    const double bound = std::sqrt(3.0) * (gain / std::sqrt(fan_in));
    tensor.uniform_real_(-bound, bound, gen);
}

// nn::Conv2d (nn/conv2d.cpp:20-81, include/tt/nn/conv2d.h:35-44): weight [out, in, k, k] initialised through the view
// weight.permute({1,0,2,3}) (conv2d.cpp:56) -- the draws run in that view's row-major order and its fan is in*k*k --
// then bias ~ U(+-1/sqrt(out*k*k)) (calc_fan_in_out of the weight itself, conv2d.cpp:60-62); forward = conv2d.
class Conv2d {
public:
    Conv2d(int in_channels, int out_channels, int kernel_size, int stride, int padding, bool with_bias, Generator &gen,
           ScalarType dtype = kF32, Device device = kAMD)
        : stride_(stride), padding_(padding) {
        if (in_channels <= 0) throw TTException("Expected in_channels > 0, given in_channels=" + std::to_string(in_channels));
        if (out_channels <= 0) throw TTException("Expected out_channels > 0, given out_channels=" + std::to_string(out_channels));
        if (kernel_size <= 0) throw TTException("Expected kernel_size > 0, given kernel_size=" + std::to_string(kernel_size));
        if (stride <= 0) throw TTException("Expected stride > 0, given stride=" + std::to_string(stride));
        if (padding < 0) throw TTException("Expected padding >= 0, given padding=" + std::to_string(padding));
        weight = Tensor::empty(Shape({out_channels, in_channels, kernel_size, kernel_size}), dtype, device);
        kaiming_uniform_(weight.permute({1, 0, 2, 3}), gen);
        if (with_bias) {
            bias = Tensor::empty(Shape({out_channels}), dtype, device);
            const auto [fan_in, fan_out] = calc_fan_in_out(weight);
            (void)fan_out;
            const double bound = 1.0 / std::sqrt(fan_in);
            bias->uniform_real_(-bound, bound, gen);
        }
    }
    [[nodiscard]] auto forward(const Tensor &input) const -> Tensor {
        if (input.dim() == 4 && input.size(1) != weight.size(1))
            throw TTException("Input channels " + std::to_string(input.size(1)) + " does not match layer input channels " +
                              std::to_string(weight.size(1)));
        return conv2d(input, weight, bias, stride_, padding_);
    }
    Tensor weight;
    std::optional<Tensor> bias;

private:
    int stride_, padding_;
};

// nn::Linear (nn/linear.cpp:20-50): weight is [in_features, out_features]; forward = matmul + bias.  The bias add
// (and an optional ReLU that follows it) is fused into the GEMM's store phase.
class Linear {
public:
    Linear(Tensor weight_, std::optional<Tensor> bias_) : weight(std::move(weight_)), bias(std::move(bias_)) {
        if (weight.dim() != 2) throw TTException("Linear: weight must be [in_features, out_features]");
    }
    // Default initialisation (nn/linear.cpp:20-40): weight by kaiming_uniform_ with gain 1 and fan = weight.size(0)
    // (nn/init.cpp:30-52,106-112), then bias ~ U(+-1/sqrt(fan)), both drawn from `gen` in that order.
    Linear(int in_features, int out_features, bool with_bias, Generator &gen, ScalarType dtype = kF32, Device device = kAMD) {
        const double fan = static_cast<double>(in_features);
        const double bound_w = std::sqrt(3.0) * (1.0 / std::sqrt(fan));
        weight = uniform_real(-bound_w, bound_w, Shape({in_features, out_features}), gen, dtype, device);
        if (with_bias) {
            const double bound_b = 1.0 / std::sqrt(fan);
            bias = uniform_real(-bound_b, bound_b, Shape({out_features}), gen, dtype, device);
        }
    }
    [[nodiscard]] auto forward(const Tensor &input, bool fuse_relu = false) const -> Tensor {
        const Tensor x2 = input.dim() == 2 ? input : input.flatten(0, -2);
        if (x2.size(1) != weight.size(0)) throw TTException("Invalid shape for matrix multiplication");
        if (x2.dtype() != weight.dtype() || x2.dtype() == kBool) throw TTException("Linear: operands must share one non-bool dtype");
        ttamd_epilogue ep{};
        std::optional<Tensor> b = bias ? std::optional<Tensor>(bias->contiguous()) : std::nullopt;
        ep.bias = b ? b->data_ptr() : nullptr;
        ep.bias_mode = b ? 1 : 0;
        ep.relu = fuse_relu ? 1 : 0;
        Tensor out = get_backend(input.device())->batched_matmul(x2.unsqueeze(0), weight.unsqueeze(0), &ep);
        auto sh = input.shape().to_vec();
        sh.back() = weight.size(1);
        return out.reshape(Shape(sh));
    }
    // forward followed by relu() in ONE launch -> {z, a}: z = input . weight + bias is what autograd saves as the
    // ReLU's input (autograd/unary_ops.cpp:562-567), a = max(z, 0) what the next layer reads.
    [[nodiscard]] auto forward_relu(const Tensor &input) const -> std::pair<Tensor, Tensor> {
        const Tensor x2 = input.dim() == 2 ? input : input.flatten(0, -2);
        if (x2.size(1) != weight.size(0)) throw TTException("Invalid shape for matrix multiplication");
        if (x2.dtype() != weight.dtype() || x2.dtype() == kBool) throw TTException("Linear: operands must share one non-bool dtype");
        auto sh = input.shape().to_vec();
        sh.back() = weight.size(1);
        const Tensor act = Tensor::empty(Shape(sh), x2.dtype(), input.device());
        ttamd_epilogue ep{};
        std::optional<Tensor> b = bias ? std::optional<Tensor>(bias->contiguous()) : std::nullopt;
        ep.bias = b ? b->data_ptr() : nullptr;
        ep.bias_mode = b ? 1 : 0;
        ep.relu_out = act.data_ptr();
        const Tensor out = get_backend(input.device())->batched_matmul(x2.unsqueeze(0), weight.unsqueeze(0), &ep);
        return {out.reshape(Shape(sh)), act};
    }
    Tensor weight;
    std::optional<Tensor> bias;
};

// Backward of y = x . W (+ b) for 2-D operands, as autograd emits it (TensorBatchedMatmul::backward on permute views,
// autograd/binary_ops.cpp:173-179) with the element-wise steps that follow dx fused into its GEMM's store:
//   dx = dy . W^T;  when x = relu(*relu_input): dx *= where(relu_input < 0, 0, 1) (autograd/unary_ops.cpp:568-573);
//   BiasGrad::kPrev: db = dx.sum(0), the bias gradient of the Linear layer that produced relu_input, from the store of
//   dx's GEMM;
//   dW = x^T . dy;
//   BiasGrad::kOwn: db = dy.sum(0), this layer's own bias gradient (nn/linear.cpp:45-48), from the vectors of dy that dW's
//   GEMM stages.
enum class BiasGrad { kNone, kPrev, kOwn };
struct LinearGrads {
    Tensor dx, dW;
    std::optional<Tensor> db;
};
inline auto linear_backward(const Tensor &grad_output, const Tensor &input, const Tensor &weight, const Tensor *relu_input = nullptr,
                            BiasGrad bias_grad = BiasGrad::kNone) -> LinearGrads {
    const auto *be = get_backend(grad_output.device());
    LinearGrads g;
    ttamd_epilogue ep{}, ep_w{};
    std::optional<Tensor> z;
    if (relu_input) {
        if (!(relu_input->shape() == input.shape()) || relu_input->dtype() != input.dtype()) throw TTException("linear_backward: relu_input must match input");
        z = relu_input->contiguous();
        ep.relu_grad_input = z->data_ptr();
    }
    const Tensor dy = bias_grad == BiasGrad::kOwn ? grad_output.contiguous() : grad_output;  // (its sums need a dense operand)
    if (bias_grad == BiasGrad::kPrev) {
        g.db = Tensor::empty(Shape({input.size(1)}), input.dtype(), input.device());
        ep.colsum_out = g.db->data_ptr();
    } else if (bias_grad == BiasGrad::kOwn) {
        g.db = Tensor::empty(Shape({dy.size(1)}), dy.dtype(), dy.device());
        ep_w.rhs_colsum_out = g.db->data_ptr();
    }
    auto [dx, dW] = be->batched_matmul_pair(dy.unsqueeze(0), weight.unsqueeze(0).permute({0, 2, 1}), &ep, input.unsqueeze(0).permute({0, 2, 1}),
                                            dy.unsqueeze(0), bias_grad == BiasGrad::kOwn ? &ep_w : nullptr);
    g.dx = dx.squeeze(0);
    g.dW = dW.squeeze(0);
    return g;
}

// nn::mse_loss(input, target) with mean reduction (nn/loss.cpp:69-72) and its backward in the same pass:
// loss [1], grad_input (1 / numel) * 2 * (input - target), and (bias_grad, at most 64 columns) grad_input.sum(0).
struct MseLoss {
    Tensor loss, grad_input;
    std::optional<Tensor> grad_colsum;
};
inline auto mse_loss(const Tensor &input, const Tensor &target, bool bias_grad = false) -> MseLoss {
    if (!(input.shape() == target.shape()) || input.dtype() != target.dtype() || input.dim() != 2)
        throw TTException("mse_loss: input and target must be 2-D tensors of one shape and dtype");
    const Tensor y = input.contiguous(), t = target.contiguous();
    MseLoss r;
    r.loss = Tensor::empty(Shape({1}), y.dtype(), y.device());
    r.grad_input = Tensor::empty(y.shape(), y.dtype(), y.device());
    if (bias_grad) r.grad_colsum = Tensor::empty(Shape({y.size(1)}), y.dtype(), y.device());
    check(ttamd_mse_loss(y.device().id, static_cast<ttamd_dtype>(y.dtype()), y.size(0), y.size(1), y.data_ptr(), t.data_ptr(), r.loss.data_ptr(),
                         r.grad_input.data_ptr(), r.grad_colsum ? r.grad_colsum->data_ptr() : nullptr, nullptr));
    return r;
}

// A network's last Linear layer with the loss behind it, forward and backward in one call (ttamd_linear_mse_head):
// y = nn::Linear::forward(input) (nn/linear.cpp:42-50), loss = nn::mse_loss(y, target) (nn/loss.cpp:69-72) and what
// autograd makes of them: dx = (dy . W^T) * where(relu_input < 0, 0, 1) with dy = (1 / numel) * 2 * (y - target),
// dW = x^T . dy, db = dy.sum(0) (autograd/reduce_ops.cpp:195-205, binary_ops.cpp:153-159,173-179, unary_ops.cpp:568-573).
// 2-D operands of one float dtype, at most 64 outputs; two launches for f32 layers of at most 16 outputs.
struct HeadResult {
    Tensor output, loss, grad_output, dx, dW;
    std::optional<Tensor> db;
};
inline auto linear_mse_head(const Tensor &input, const Tensor &weight, const Tensor *bias, const Tensor &target, const Tensor *relu_input = nullptr)
    -> HeadResult {
    if (input.dim() != 2 || weight.dim() != 2 || target.dim() != 2) throw TTException("linear_mse_head: input, weight and target must be 2-D");
    const int64_t rows = input.size(0), fin = input.size(1), fout = weight.size(1);
    if (weight.size(0) != fin) throw TTException("Invalid shape for matrix multiplication");
    if (target.size(0) != rows || target.size(1) != fout || (relu_input && !(relu_input->shape() == input.shape())))
        throw TTException("linear_mse_head: target must be [rows, out_features] and relu_input [rows, in_features]");
    if (bias && bias->numel() != fout) throw TTException("linear_mse_head: bias must hold out_features elements");
    const ScalarType dt = input.dtype();
    if (weight.dtype() != dt || target.dtype() != dt || (bias && bias->dtype() != dt) || (relu_input && relu_input->dtype() != dt))
        throw TTException("linear_mse_head: operands of one dtype");
    const Tensor x = input.contiguous(), w = weight.contiguous(), t = target.contiguous();
    std::optional<Tensor> b, z;
    if (bias) b = bias->contiguous();
    if (relu_input) z = relu_input->contiguous();
    HeadResult r;
    const Device dev = x.device();
    r.output = Tensor::empty(Shape({rows, fout}), dt, dev);
    r.loss = Tensor::empty(Shape({1}), dt, dev);
    r.grad_output = Tensor::empty(Shape({rows, fout}), dt, dev);
    r.dx = Tensor::empty(Shape({rows, fin}), dt, dev);
    r.dW = Tensor::empty(Shape({fin, fout}), dt, dev);
    if (bias) r.db = Tensor::empty(Shape({fout}), dt, dev);
    check(ttamd_linear_mse_head(dev.id, static_cast<ttamd_dtype>(dt), rows, fin, fout, x.data_ptr(), w.data_ptr(), b ? b->data_ptr() : nullptr,
                                t.data_ptr(), z ? z->data_ptr() : nullptr, r.output.data_ptr(), r.loss.data_ptr(), r.grad_output.data_ptr(),
                                r.dx.data_ptr(), r.dW.data_ptr(), r.db ? r.db->data_ptr() : nullptr, nullptr));
    return r;
}
}  // namespace nn

}  // namespace tt_amd

#endif  // TT_AMD_HOST_H_
