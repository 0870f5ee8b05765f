// tt/shape.h — TEST-SIDE STAND-IN (see tt/exception.h in this directory): a list of extents (or strides).
#ifndef TT_STANDIN_SHAPE_H_
#define TT_STANDIN_SHAPE_H_

#include <tt/exception.h>

#include <initializer_list>
#include <utility>
#include <vector>

namespace tinytensor {

class Shape {
public:
    Shape() = default;
    explicit Shape(const std::vector<int> &d) : dims(d) {}
    explicit Shape(std::vector<int> &&d) : dims(std::move(d)) {}
    Shape(std::initializer_list<int> d) : dims(d) {}

    [[nodiscard]] auto numel() const noexcept -> int {
        int n = 1;
        for (const int d : dims) {
            n *= d;
        }
        return n;
    }
    [[nodiscard]] auto ndim() const noexcept -> int { return static_cast<int>(dims.size()); }
    [[nodiscard]] auto size() const noexcept -> int { return ndim(); }
    auto operator[](int index) -> int & { return dims[at(index)]; }
    auto operator[](int index) const -> int { return dims[at(index)]; }
    auto operator==(const Shape &other) const noexcept -> bool { return dims == other.dims; }
    // the strides of a dense row-major tensor of this shape
    [[nodiscard]] auto to_stride() const -> Shape {
        std::vector<int> st(dims.size(), 1);
        for (int i = ndim() - 2; i >= 0; --i) {
            st[static_cast<std::size_t>(i)] = st[static_cast<std::size_t>(i) + 1] * dims[static_cast<std::size_t>(i) + 1];
        }
        return Shape(std::move(st));
    }
    [[nodiscard]] auto to_vec() const -> const std::vector<int> & { return dims; }

private:
    [[nodiscard]] auto at(int index) const -> std::size_t {
        const int i = index < 0 ? index + ndim() : index;
        if (i < 0 || i >= ndim()) {
            TT_EXCEPTION("Shape index out of range");
        }
        return static_cast<std::size_t>(i);
    }
    std::vector<int> dims;
};

}    // namespace tinytensor

#endif    // TT_STANDIN_SHAPE_H_
