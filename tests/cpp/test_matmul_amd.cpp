// test_matmul_amd.cpp — the reference's matmul tests (tests/test_matmul.cpp: dot product, vector-matrix,
// matrix-vector, matrix-matrix, batched; same shapes and data patterns, naive host loop as the oracle) run
// against the AMD device through the C++ host layer, plus the strided-operand cases the reference only
// reaches through autograd (backward GEMMs on permuted views) and nn::Linear.
#include "mini_test.h"

using namespace tt_amd;

namespace {
template <typename T>
std::vector<T> dot_product(const std::vector<T> &v1, const std::vector<T> &v2) {
    T result{};
    for (std::size_t i = 0; i < v1.size(); ++i) result += static_cast<T>(v1[i] * v2[i]);
    return {result};
}
// C[N,M] += A[N,K] . B[K,M], element type arithmetic (integers wrap)
template <typename T>
void naive(const T *A, const T *B, T *C, int N, int K, int M) {
    for (int row = 0; row < N; ++row)
        for (int col = 0; col < M; ++col)
            for (int i = 0; i < K; ++i) C[row * M + col] += static_cast<T>(A[row * K + i] * B[i * M + col]);
}
}  // namespace

TEST_CASE("Dot product") {
    auto test_bool = []<typename T>(Device device) {
        Tensor lhs(std::vector<bool>(12, true), {12}, device), rhs(std::vector<bool>(12, true), {12}, device);
        CHECK_THROWS_AS((void)matmul(lhs, rhs), TTException);
    };
    runner_boolean(test_bool);
    auto test = []<typename T>(Device device) {
        for (int n : {12, 2048}) {
            std::vector<T> a, b;
            for (int i = 0; i < n; ++i) {
                a.push_back(static_cast<T>(i));
                b.push_back(static_cast<T>(i + 10));
            }
            CHECK(allclose(matmul(Tensor(a, {n}, device), Tensor(b, {n}, device)).template to_vec<T>(), dot_product(a, b)));
        }
    };
    runner_all_except_bool(test);
}

TEST_CASE("Vector Matrix and Matrix Vector product") {
    auto test = []<typename T>(Device device) {
        constexpr int N = 256 + 123, M = 512 + 123;
        std::vector<T> v, m, mt(static_cast<std::size_t>(N) * M);
        for (int i = 0; i < N; ++i) {
            v.push_back(static_cast<T>(i % 100));
            for (int j = 0; j < M; ++j) m.push_back(static_cast<T>((i + j) % 100));
        }
        std::vector<T> expected(M, 0);
        naive(v.data(), m.data(), expected.data(), 1, N, M);
        CHECK(allclose(matmul(Tensor(v, {N}, device), Tensor(m, {N, M}, device)).template to_vec<T>(), expected));
        // matrix . vector with the matrix given as a transposed VIEW of the same storage
        CHECK(allclose(matmul(Tensor(m, {N, M}, device).permute({1, 0}), Tensor(v, {N}, device)).template to_vec<T>(), expected));
        CHECK_THROWS_AS((void)matmul(Tensor(v, {N}, device), Tensor(m, {M, N}, device)), TTException);
    };
    runner_all_except_bool(test);
}

TEST_CASE("Matrix Matrix product") {
    auto test = []<typename T>(Device device) {
        constexpr int N = 256 + 123, M = 1024 + 123, K = 512 + 123;
        std::vector<T> lhs, rhs;
        for (int i = 0; i < N; ++i)
            for (int j = 0; j < M; ++j) lhs.push_back(static_cast<T>((i + j) % 100));
        for (int i = 0; i < M; ++i)
            for (int j = 0; j < K; ++j) rhs.push_back(static_cast<T>((i + j) % 100));
        std::vector<T> expected(static_cast<std::size_t>(N) * K, 0);
        naive(lhs.data(), rhs.data(), expected.data(), N, M, K);
        const Tensor got = matmul(Tensor(lhs, {N, M}, device), Tensor(rhs, {M, K}, device));
        CHECK(got.shape() == Shape({N, K}));
        CHECK(got.template to_vec<T>() == expected);  // exact: every partial sum is an integer below 2^24 (or wraps)
    };
    runner_all_except_bool(test);
}

TEST_CASE("Batched Matrix Matrix product") {
    auto test_bool = []<typename T>(Device device) {
        Tensor lhs(std::vector<bool>(2 * 12 * 4, true), {2, 12, 4}, device), rhs(std::vector<bool>(2 * 4 * 12, true), {2, 4, 12}, device);
        CHECK_THROWS_AS((void)matmul(lhs, rhs), TTException);
    };
    runner_boolean(test_bool);
    auto test = []<typename T>(Device device) {
        constexpr int B = 4, N = 256 + 123, M = 1024 + 123, K = 512 + 123;  // tests/test_matmul.cpp:200-236, at its own size
        std::vector<T> lhs, rhs;
        for (int b = 0; b < B; ++b) {
            for (int i = 0; i < N; ++i)
                for (int j = 0; j < M; ++j) lhs.push_back(static_cast<T>((i * b + j + b) % 100));
            for (int i = 0; i < M; ++i)
                for (int j = 0; j < K; ++j) rhs.push_back(static_cast<T>((i + j + 2 * b) % 100));
        }
        std::vector<T> expected(static_cast<std::size_t>(B) * N * K, 0);
        for (int b = 0; b < B; ++b) naive(lhs.data() + b * N * M, rhs.data() + b * M * K, expected.data() + b * N * K, N, M, K);
        CHECK(matmul(Tensor(lhs, {B, N, M}, device), Tensor(rhs, {B, M, K}, device)).template to_vec<T>() == expected);
    };
    runner_all_except_bool(test);
}

TEST_CASE("Backward GEMMs on permuted views") {
    // dA = dC . B^T and dB = A^T . dC (autograd/binary_ops.cpp:173-179); integer-valued data, so exact.
    auto test = []<typename T>(Device device) {
        constexpr int B = 2, N = 70, K = 45, M = 130;
        std::vector<T> a, b, g;
        for (int i = 0; i < B * N * K; ++i) a.push_back(static_cast<T>(i % 7 - 3));
        for (int i = 0; i < B * K * M; ++i) b.push_back(static_cast<T>(i % 5 - 2));
        for (int i = 0; i < B * N * M; ++i) g.push_back(static_cast<T>(i % 3 - 1));
        const Tensor A(a, {B, N, K}, device), Bt(b, {B, K, M}, device), G(g, {B, N, M}, device);
        const auto [dA, dB] = matmul_backward(A, Bt, G);
        std::vector<T> eA(a.size(), 0), eB(b.size(), 0);
        for (int bb = 0; bb < B; ++bb)
            for (int n = 0; n < N; ++n)
                for (int m = 0; m < M; ++m) {
                    const T gv = g[(bb * N + n) * M + m];
                    for (int k = 0; k < K; ++k) {
                        eA[(bb * N + n) * K + k] += gv * b[(bb * K + k) * M + m];
                        eB[(bb * K + k) * M + m] += a[(bb * N + n) * K + k] * gv;
                    }
                }
        CHECK(dA.shape() == A.shape());
        CHECK(dB.shape() == Bt.shape());
        CHECK(dA.template to_vec<T>() == eA);
        CHECK(dB.template to_vec<T>() == eB);
    };
    runner_floating_point(test);
}

TEST_CASE("nn::Linear forward") {
    auto test = []<typename T>(Device device) {
        constexpr int R = 50, IN = 37, OUT = 21;
        std::vector<T> x, w, b;
        for (int i = 0; i < 2 * R * IN; ++i) x.push_back(static_cast<T>(i % 9 - 4));
        for (int i = 0; i < IN * OUT; ++i) w.push_back(static_cast<T>(i % 7 - 3));
        for (int i = 0; i < OUT; ++i) b.push_back(static_cast<T>(i % 5 - 2));
        nn::Linear layer(Tensor(w, {IN, OUT}, device), Tensor(b, {OUT}, device));  // weight is [in, out]
        const Tensor y = layer.forward(Tensor(x, {2, R, IN}, device));
        CHECK(y.shape() == Shape({2, R, OUT}));
        std::vector<T> expected(static_cast<std::size_t>(2) * R * OUT, 0);
        naive(x.data(), w.data(), expected.data(), 2 * R, IN, OUT);
        for (int i = 0; i < 2 * R; ++i)
            for (int j = 0; j < OUT; ++j) expected[i * OUT + j] += b[j];
        CHECK(y.template to_vec<T>() == expected);
        for (auto &v : expected) v = v > T(0) ? v : T(0);
        CHECK(layer.forward(Tensor(x, {2, R, IN}, device), true).template to_vec<T>() == expected);
    };
    runner_floating_point(test);
}

TEST_CASE("Device errors and memory counters") {
    const auto *be = get_backend(kAMD);
    CHECK(be->get_device_count() >= 1);
    const auto before = be->current_memory_allocated(0);
    {
        Tensor t(std::vector<float>(1024, 1.0f), {1024}, kAMD);
        CHECK(be->current_memory_allocated(0) == before + 4096);
    }
    CHECK(be->current_memory_allocated(0) == before);
    CHECK_THROWS_AS(Tensor(std::vector<float>(4, 0.f), {4}, Device{Backend::amd, be->get_device_count()}), TTException);
}

int main(int argc, char **argv) { return mini::run_all(argc, argv); }
