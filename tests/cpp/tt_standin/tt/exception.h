// tt/exception.h — TEST-SIDE STAND-IN for the reference's include/tt/exception.h.
// The reference's own public headers need <format> and constexpr std::string (libstdc++ 13), which this image lacks.
// The files in this directory give the names that tinytensor/tensor/backend_base.h and the AMD adapter use just
// enough behaviour for the adapter's code to RUN in tests/cpp/test_adapter_amd.cpp.  They are written for that test
// only, pin nothing about the reference's semantics and are not part of the product.
#ifndef TT_STANDIN_EXCEPTION_H_
#define TT_STANDIN_EXCEPTION_H_

#include <cstdlib>
#include <exception>
#include <iostream>
#include <string>

namespace tinytensor {

class TTException : public std::exception {
public:
    TTException(const std::string &text, const char *file, const char *function, int line)
        : message(text + " [" + file + ":" + std::to_string(line) + " " + function + "]") {}
    [[nodiscard]] auto what() const noexcept -> const char * override { return message.c_str(); }

private:
    std::string message;
};

}    // namespace tinytensor

#define TT_EXCEPTION(msg) throw tinytensor::TTException(msg, __FILE__, __PRETTY_FUNCTION__, __LINE__)
#define TT_ERROR(msg)                       \
    {                                       \
        std::cout << (msg) << std::endl;    \
        std::exit(1);                       \
    }

#endif    // TT_STANDIN_EXCEPTION_H_
