// tt/tensor.h — TEST-SIDE STAND-IN (see tt/exception.h in this directory): a Tensor that is storage + dtype + shape
// + element strides + element offset, with the constructor backends return results through
// (tensor/tensor.cpp:351-358: dense strides, offset 0) and the few members the adapter calls (contiguous, to, numel,
// size, get_storage).  Views are built by permute / expand / narrow; there is no autograd and no broadcasting.
// Everything that touches data goes through get_backend(device), defined by the test.
#ifndef TT_STANDIN_TENSOR_H_
#define TT_STANDIN_TENSOR_H_

#include <tt/device.h>
#include <tt/exception.h>
#include <tt/scalar.h>
#include <tt/shape.h>

#include <cstdint>
#include <memory>
#include <ostream>
#include <utility>
#include <vector>

namespace tinytensor {

class StorageBase;
class BackendBase;

// the registry of tensor/backend_register.cpp:19-38, with the case that patches/backend_register.cpp.patch adds
auto get_backend(Device device) -> BackendBase *;

class Tensor {
public:
    // what a backend returns a result through
    Tensor(std::shared_ptr<StorageBase> storage, ScalarType dtype, Shape shape, Device device)
        : device_(device), dtype_(dtype), offset_(0), shape_(std::move(shape)), stride_(shape_.to_stride()),
          storage_(std::move(storage)) {}
    // host data -> device (BackendBase::from_vec)
    template <typename T>
    Tensor(const std::vector<T> &data, Shape shape, Device device);
    // one value (BackendBase::from_scalar), shape {1}
    Tensor(Scalar scalar, Device device);

    [[nodiscard]] auto dtype() const -> ScalarType { return dtype_; }
    [[nodiscard]] auto device() const -> Device { return device_; }
    [[nodiscard]] auto offset() const -> int { return offset_; }
    [[nodiscard]] auto shape() const -> const Shape & { return shape_; }
    [[nodiscard]] auto stride() const -> const Shape & { return stride_; }
    [[nodiscard]] auto numel() const -> int { return shape_.numel(); }
    [[nodiscard]] auto dim() const -> int { return shape_.ndim(); }
    [[nodiscard]] auto size(int d) const -> int { return shape_[d]; }
    [[nodiscard]] auto is_contiguous() const -> bool { return offset_ == 0 && stride_ == shape_.to_stride(); }

    // dense copy through BackendBase::identity unless already dense with offset 0
    [[nodiscard]] auto contiguous() const -> Tensor;
    [[nodiscard]] auto clone() const -> Tensor;
    [[nodiscard]] auto to(ScalarType dtype) const -> Tensor;
    // there is no CPU backend in the stand-in: only the tensor's own device is accepted
    [[nodiscard]] auto to(Device device) const -> Tensor;
    // the elements in row-major order of the view (clone, then BackendBase::to_vec of the whole storage)
    template <typename T>
    [[nodiscard]] auto to_vec() const -> std::vector<T>;
    [[nodiscard]] auto item() const -> Scalar;

    template <typename T>
    [[nodiscard]] auto get_storage() const -> T & {
        return *static_cast<T *>(storage_.get());
    }

    // views: only shape, strides and offset change
    [[nodiscard]] auto permute(const std::vector<int> &dims) const -> Tensor;
    [[nodiscard]] auto expand(const Shape &shape) const -> Tensor;
    [[nodiscard]] auto narrow(int dim, int start, int length) const -> Tensor;

    friend auto operator<<(std::ostream &os, const Tensor &tensor) -> std::ostream &;

private:
    Device device_;
    ScalarType dtype_;
    int offset_;
    Shape shape_;
    Shape stride_;
    std::shared_ptr<StorageBase> storage_;
};

}    // namespace tinytensor

#endif    // TT_STANDIN_TENSOR_H_
