// mini_test.h — a few macros in the style of the reference's doctest usage (TEST_CASE / CHECK /
// CHECK_THROWS_AS), enough for the host-side tests; every test runs for the device list in runner_*.
#ifndef TT_AMD_MINI_TEST_H_
#define TT_AMD_MINI_TEST_H_

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

namespace mini {
struct Case {
    const char *name;
    std::function<void()> fn;
};
inline std::vector<Case> &cases() {
    static std::vector<Case> c;
    return c;
}
inline int &failures() {
    static int f = 0;
    return f;
}
struct Registrar {
    Registrar(const char *name, std::function<void()> fn) { cases().push_back({name, std::move(fn)}); }
};
inline int run_all(int argc, char **argv) {
    const bool list = argc > 1 && std::strcmp(argv[1], "--list") == 0;
    for (auto &c : cases()) {
        if (list) {
            std::printf("%s\n", c.name);
            continue;
        }
        const int before = failures();
        std::printf("[ RUN  ] %s\n", c.name);
        std::fflush(stdout);
        try {
            c.fn();
        } catch (const std::exception &e) {
            std::printf("  unexpected exception: %s\n", e.what());
            ++failures();
        }
        std::printf("[ %s ] %s\n", failures() == before ? " OK " : "FAIL", c.name);
        std::fflush(stdout);
    }
    if (!list) std::printf("%d test case(s), %d failure(s)\n", static_cast<int>(cases().size()), failures());
    return failures() == 0 ? 0 : 1;
}
}  // namespace mini

#define MINI_CAT2(a, b) a##b
#define MINI_CAT(a, b) MINI_CAT2(a, b)
#define TEST_CASE(name)                                                        \
    static void MINI_CAT(test_fn_, __LINE__)();                                \
    static mini::Registrar MINI_CAT(test_reg_, __LINE__)(name, MINI_CAT(test_fn_, __LINE__)); \
    static void MINI_CAT(test_fn_, __LINE__)()
#define CHECK(...)                                                              \
    do {                                                                        \
        if (!(__VA_ARGS__)) {                                                   \
            std::printf("  %s:%d: CHECK(%s) failed\n", __FILE__, __LINE__, #__VA_ARGS__); \
            ++mini::failures();                                                 \
        }                                                                       \
    } while (0)
#define CHECK_THROWS_AS(expr, Exc)                                              \
    do {                                                                        \
        bool caught_ = false;                                                   \
        try {                                                                   \
            expr;                                                               \
        } catch (const Exc &) {                                                 \
            caught_ = true;                                                     \
        } catch (...) {                                                         \
        }                                                                       \
        if (!caught_) {                                                         \
            std::printf("  %s:%d: CHECK_THROWS_AS(%s, %s) failed\n", __FILE__, __LINE__, #expr, #Exc); \
            ++mini::failures();                                                 \
        }                                                                       \
    } while (0)

// allclose with the reference's defaults rtol 1e-5 / atol 1e-8 (include/tt/tensor.h:3396-3398), on host vectors.
template <typename T>
bool allclose(const std::vector<T> &a, const std::vector<T> &b, double rtol = 1e-5, double atol = 1e-8) {
    if (a.size() != b.size()) return false;
    for (std::size_t i = 0; i < a.size(); ++i) {
        const double x = static_cast<double>(a[i]), y = static_cast<double>(b[i]);
        if (!(std::fabs(x - y) <= atol + rtol * std::fabs(y))) return false;
    }
    return true;
}

// (a test that brings its own Tensor defines MINI_TEST_NO_HOST_LAYER and its own fan-out)
#ifndef MINI_TEST_NO_HOST_LAYER
// Device / dtype fan-out in the style of the reference's tests/test_util.h:5-45.
#include "tt_amd.h"
template <typename T, typename F>
void runner_single_type(F &&f) {
    f.template operator()<T>(tt_amd::kAMD);
}
template <typename F>
void runner_all_except_bool(F &&f) {
    runner_single_type<uint8_t>(f);
    runner_single_type<int16_t>(f);
    runner_single_type<int32_t>(f);
    runner_single_type<int64_t>(f);
    runner_single_type<float>(f);
    runner_single_type<double>(f);
}
template <typename F>
void runner_floating_point(F &&f) {
    runner_single_type<float>(f);
    runner_single_type<double>(f);
}
template <typename F>
void runner_boolean(F &&f) {
    runner_single_type<bool>(f);
}
#endif  // MINI_TEST_NO_HOST_LAYER

#endif  // TT_AMD_MINI_TEST_H_
