// standin.cpp — the out-of-line members of the TEST-SIDE STAND-IN Tensor (tt/tensor.h in this directory) and the
// backend registry.  Compiled against the reference's own tinytensor/tensor/backend_base.h.
#include <tt/tensor.h>

#include "tensor/backend/amd/backend_amd.h"
#include "tensor/backend_base.h"

#include <memory>

namespace tinytensor {

auto get_backend(Device device) -> BackendBase * {
    if (device.backend == Backend::amd) {
        static const std::unique_ptr<amd::BackendAMD> backend_amd = std::make_unique<amd::BackendAMD>();
        return backend_amd.get();
    }
    TT_EXCEPTION("Unknown device type.");
}

template <typename T>
Tensor::Tensor(const std::vector<T> &data, Shape shape, Device device)
    : device_(device), dtype_(to_scalar<T>::type), offset_(0), shape_(std::move(shape)), stride_(shape_.to_stride()),
      storage_(get_backend(device)->from_vec(data, device.id)) {
    if (static_cast<std::size_t>(shape_.numel()) != data.size()) {
        TT_EXCEPTION("Tensor: the data does not fill the shape");
    }
}
template Tensor::Tensor(const std::vector<bool> &, Shape, Device);
template Tensor::Tensor(const std::vector<uint8_t> &, Shape, Device);
template Tensor::Tensor(const std::vector<int16_t> &, Shape, Device);
template Tensor::Tensor(const std::vector<int32_t> &, Shape, Device);
template Tensor::Tensor(const std::vector<int64_t> &, Shape, Device);
template Tensor::Tensor(const std::vector<float> &, Shape, Device);
template Tensor::Tensor(const std::vector<double> &, Shape, Device);

Tensor::Tensor(Scalar scalar, Device device)
    : device_(device), dtype_(scalar.dtype()), offset_(0), shape_({1}), stride_(shape_.to_stride()),
      storage_(get_backend(device)->from_scalar(scalar, device.id)) {}

auto Tensor::contiguous() const -> Tensor {
    return is_contiguous() ? *this : clone();
}

auto Tensor::clone() const -> Tensor {
    return get_backend(device_)->identity(*this);
}

auto Tensor::to(ScalarType dtype) const -> Tensor {
    return dtype == dtype_ ? *this : get_backend(device_)->to(*this, dtype);
}

auto Tensor::to(Device device) const -> Tensor {
    if (device == device_) {
        return *this;
    }
    TT_EXCEPTION("the stand-in Tensor has no other device to go to");
}

template <typename T>
auto Tensor::to_vec() const -> std::vector<T> {
    const Tensor dense = dtype_ == to_scalar<T>::type ? clone() : to(to_scalar<T>::type);
    std::vector<T> out;
    get_backend(device_)->to_vec(dense, out);
    return out;
}
template auto Tensor::to_vec() const -> std::vector<uint8_t>;
template auto Tensor::to_vec() const -> std::vector<int16_t>;
template auto Tensor::to_vec() const -> std::vector<int32_t>;
template auto Tensor::to_vec() const -> std::vector<int64_t>;
template auto Tensor::to_vec() const -> std::vector<float>;
template auto Tensor::to_vec() const -> std::vector<double>;

auto Tensor::item() const -> Scalar {
    return get_backend(device_)->item(*this);
}

auto Tensor::permute(const std::vector<int> &dims) const -> Tensor {
    if (static_cast<int>(dims.size()) != dim()) {
        TT_EXCEPTION("permute: one index per dimension");
    }
    Tensor view = *this;
    for (int i = 0; i < dim(); ++i) {
        view.shape_[i] = shape_[dims[static_cast<std::size_t>(i)]];
        view.stride_[i] = stride_[dims[static_cast<std::size_t>(i)]];
    }
    return view;
}

auto Tensor::expand(const Shape &shape) const -> Tensor {
    // trailing dimensions align; an extent of 1 (or a missing leading dimension) is repeated with stride 0
    Tensor view = *this;
    std::vector<int> strides(static_cast<std::size_t>(shape.ndim()), 0);
    for (int i = 0; i < dim(); ++i) {
        const int j = shape.ndim() - dim() + i;
        if (j < 0 || (shape_[i] != shape[j] && shape_[i] != 1)) {
            TT_EXCEPTION("expand: incompatible shapes");
        }
        strides[static_cast<std::size_t>(j)] = shape_[i] == shape[j] && shape_[i] != 1 ? stride_[i] : 0;
    }
    view.shape_ = shape;
    view.stride_ = Shape(std::move(strides));
    return view;
}

auto Tensor::narrow(int d, int start, int length) const -> Tensor {
    if (start < 0 || length < 0 || start + length > shape_[d]) {
        TT_EXCEPTION("narrow: range outside the dimension");
    }
    Tensor view = *this;
    view.offset_ += start * stride_[d];
    view.shape_[d] = length;
    return view;
}

auto operator<<(std::ostream &os, const Tensor &tensor) -> std::ostream & {
    return get_backend(tensor.device())->print(os, tensor);
}

}    // namespace tinytensor
