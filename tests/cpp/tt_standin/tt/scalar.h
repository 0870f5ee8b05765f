// tt/scalar.h — TEST-SIDE STAND-IN (see tt/exception.h in this directory): ScalarType in the reference's order
// (include/tt/scalar.h:21-29), the ctype traits and a type-erased Scalar.
#ifndef TT_STANDIN_SCALAR_H_
#define TT_STANDIN_SCALAR_H_

#include <cstddef>
#include <cstdint>
#include <type_traits>

namespace tinytensor {

enum class ScalarType { bool8 = 0, u8, i16, i32, i64, f32, f64 };

constexpr ScalarType kBool = ScalarType::bool8;
constexpr ScalarType kU8 = ScalarType::u8;
constexpr ScalarType kI16 = ScalarType::i16;
constexpr ScalarType kI32 = ScalarType::i32;
constexpr ScalarType kI64 = ScalarType::i64;
constexpr ScalarType kF32 = ScalarType::f32;
constexpr ScalarType kF64 = ScalarType::f64;
constexpr ScalarType kDefaultInt = ScalarType::i32;
constexpr ScalarType kDefaultFloat = ScalarType::f32;

constexpr auto is_integral_dtype(ScalarType dtype) -> bool {
    return dtype == kU8 || dtype == kI16 || dtype == kI32 || dtype == kI64;
}
constexpr auto is_float_dtype(ScalarType dtype) -> bool {
    return dtype == kF32 || dtype == kF64;
}

template <typename T>
struct to_scalar;
template <> struct to_scalar<bool> { static constexpr ScalarType type = kBool; };
template <> struct to_scalar<uint8_t> { static constexpr ScalarType type = kU8; };
template <> struct to_scalar<int16_t> { static constexpr ScalarType type = kI16; };
template <> struct to_scalar<int32_t> { static constexpr ScalarType type = kI32; };
template <> struct to_scalar<int64_t> { static constexpr ScalarType type = kI64; };
template <> struct to_scalar<float> { static constexpr ScalarType type = kF32; };
template <> struct to_scalar<double> { static constexpr ScalarType type = kF64; };

// One value with its dtype; integers are kept in 64 bits, floats in a double (exact for every dtype's range but
// int64 beyond 2^53, which the test does not use).
class Scalar {
public:
    explicit Scalar(bool v) : integer(v ? 1 : 0), type(kBool) {}
    explicit Scalar(uint8_t v) : integer(v), type(kU8) {}
    explicit Scalar(int16_t v) : integer(v), type(kI16) {}
    explicit Scalar(int32_t v) : integer(v), type(kI32) {}
    explicit Scalar(int64_t v) : integer(v), type(kI64) {}
    explicit Scalar(float v) : real(v), type(kF32) {}
    explicit Scalar(double v) : real(v), type(kF64) {}
    template <typename T>
    Scalar(T v, ScalarType dtype) : type(dtype) {
        if (is_float_dtype(dtype)) {
            real = dtype == kF32 ? static_cast<double>(static_cast<float>(v)) : static_cast<double>(v);
        } else if (dtype == kBool) {
            integer = static_cast<bool>(v) ? 1 : 0;
        } else {
            integer = static_cast<int64_t>(v);
        }
    }

    [[nodiscard]] constexpr auto dtype() const -> ScalarType { return type; }

    template <typename T>
    [[nodiscard]] auto to() const -> T {
        return is_float_dtype(type) ? static_cast<T>(real) : static_cast<T>(integer);
    }

private:
    int64_t integer = 0;
    double real = 0.0;
    ScalarType type;
};

}    // namespace tinytensor

#endif    // TT_STANDIN_SCALAR_H_
