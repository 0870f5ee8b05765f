// test_adapter_amd.cpp — RUNS the reference-side adapter (tinytensor_amd/host/adapter/.../backend_amd.cpp) on the GPU.
//
// backend_amd.cpp is compiled to an object against the reference's own tinytensor/tensor/backend_base.h and
// storage_base.h and linked with libttamd.so; the <tt/...> public headers, which this image's standard library cannot
// compile, are replaced by the functional stand-ins in tests/cpp/tt_standin/ (a minimal Tensor / Shape / Scalar /
// Generator written for this test).  Every call below goes through a `const BackendBase &`, the way the reference's
// frontend calls a backend.  This executes the adapter's code (views, offsets in elements, storage lifetimes, result
// shapes, the status -> TTException mapping); it does not pin reference semantics: stand-ins pin nothing.
// Expected values are naive host loops on the patterns of the reference's tests (tests/test_matmul.cpp:163-236,
// tests/test_conv.cpp:99-143).
#define MINI_TEST_NO_HOST_LAYER
#include "mini_test.h"

#include <tt/device.h>
#include <tt/exception.h>
#include <tt/random.h>
#include <tt/scalar.h>
#include <tt/shape.h>
#include <tt/tensor.h>

#include "tensor/backend/amd/backend_amd.h"
#include "tensor/backend_base.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <optional>
#include <sstream>
#include <tuple>
#include <vector>

using namespace tinytensor;

namespace {

const BackendBase &backend() {
    return *get_backend(kAMD);
}

template <typename F>
void for_all_except_bool(F &&f) {
    f.template operator()<uint8_t>();
    f.template operator()<int16_t>();
    f.template operator()<int32_t>();
    f.template operator()<int64_t>();
    f.template operator()<float>();
    f.template operator()<double>();
}
template <typename F>
void for_floating_point(F &&f) {
    f.template operator()<float>();
    f.template operator()<double>();
}

template <typename T>
std::vector<T> pattern(int n, int mod, int shift) {
    std::vector<T> v(static_cast<std::size_t>(n));
    for (int i = 0; i < n; ++i) v[static_cast<std::size_t>(i)] = static_cast<T>(i % mod - shift);
    return v;
}

// C[N,M] += A[N,K] . B[K,M] in the element type (integers wrap)
template <typename T>
void gemm_naive(const T *A, const T *B, T *C, int N, int K, int M) {
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) {
            const T a = A[n * K + k];
            for (int m = 0; m < M; ++m) C[n * M + m] = static_cast<T>(C[n * M + m] + static_cast<T>(a * B[k * M + m]));
        }
}

// out[b,o,y,x] = sum_{c,p,q} in[b,c,y*S-P+p,x*S-P+q] * w[o,c,p,q] (+ bias[o]), zero padding
template <typename T>
std::vector<T> conv_naive(const std::vector<T> &in, const std::vector<T> &w, const std::vector<T> *bias, int B, int C, int O, int H,
                          int W, int k, int S, int P) {
    const int Ho = (H + 2 * P - k) / S + 1, Wo = (W + 2 * P - k) / S + 1;
    std::vector<T> out(static_cast<std::size_t>(B) * O * Ho * Wo, T(0));
    for (int b = 0; b < B; ++b)
        for (int o = 0; o < O; ++o)
            for (int y = 0; y < Ho; ++y)
                for (int x = 0; x < Wo; ++x) {
                    T acc = T(0);
                    for (int c = 0; c < C; ++c)
                        for (int p = 0; p < k; ++p)
                            for (int q = 0; q < k; ++q) {
                                const int iy = y * S - P + p, ix = x * S - P + q;
                                if (iy < 0 || ix < 0 || iy >= H || ix >= W) continue;
                                acc = static_cast<T>(acc + static_cast<T>(in[((static_cast<std::size_t>(b) * C + c) * H + iy) * W + ix] *
                                                                          w[((static_cast<std::size_t>(o) * C + c) * k + p) * k + q]));
                            }
                    if (bias) acc = static_cast<T>(acc + (*bias)[static_cast<std::size_t>(o)]);
                    out[((static_cast<std::size_t>(b) * O + o) * Ho + y) * Wo + x] = acc;
                }
    return out;
}

// gradients of sum(out * g) with respect to in, w and bias
template <typename T>
void conv_backward_naive(const std::vector<T> &g, const std::vector<T> &in, const std::vector<T> &w, int B, int C, int O, int H, int W, int k,
                         int S, int P, std::vector<T> &gin, std::vector<T> &gw, std::vector<T> &gb) {
    const int Ho = (H + 2 * P - k) / S + 1, Wo = (W + 2 * P - k) / S + 1;
    gin.assign(in.size(), T(0));
    gw.assign(w.size(), T(0));
    gb.assign(static_cast<std::size_t>(O), T(0));
    for (int b = 0; b < B; ++b)
        for (int o = 0; o < O; ++o)
            for (int y = 0; y < Ho; ++y)
                for (int x = 0; x < Wo; ++x) {
                    const T gv = g[((static_cast<std::size_t>(b) * O + o) * Ho + y) * Wo + x];
                    gb[static_cast<std::size_t>(o)] += gv;
                    for (int c = 0; c < C; ++c)
                        for (int p = 0; p < k; ++p)
                            for (int q = 0; q < k; ++q) {
                                const int iy = y * S - P + p, ix = x * S - P + q;
                                if (iy < 0 || ix < 0 || iy >= H || ix >= W) continue;
                                const std::size_t ii = ((static_cast<std::size_t>(b) * C + c) * H + iy) * W + ix;
                                const std::size_t wi = ((static_cast<std::size_t>(o) * C + c) * k + p) * k + q;
                                gin[ii] += gv * w[wi];
                                gw[wi] += gv * in[ii];
                            }
                }
}

template <typename T>
T unit_draw(uint64_t bits);
template <>
float unit_draw<float>(uint64_t bits) {
    const uint32_t u = (static_cast<uint32_t>(bits) >> 9U) | 0x3F800000U;
    float f;
    std::memcpy(&f, &u, sizeof(f));
    return f - 1.0F;
}
template <>
double unit_draw<double>(uint64_t bits) {
    const uint64_t u = (bits >> 12U) | 0x3FF0000000000000ULL;
    double f;
    std::memcpy(&f, &u, sizeof(f));
    return f - 1.0;
}

}  // namespace

TEST_CASE("storage: from_vec / to_vec / from_scalar / full / arange / item / data_ptr / counters") {
    const BackendBase &be = backend();
    CHECK(be.get_device_count() >= 1);
    for_all_except_bool([&]<typename T>() {
        const std::vector<T> host = pattern<T>(1000, 97, 13);
        const Tensor t(host, {10, 100}, kAMD);
        std::vector<T> back;
        be.to_vec(t, back);
        CHECK(back == host);
        std::vector<T> moved = host;
        const Tensor t2(std::shared_ptr<StorageBase>(be.from_vec(std::move(moved), 0)), to_scalar<T>::type, {1000}, kAMD);
        CHECK(t2.to_vec<T>() == host);
        // item() and data_ptr() of a view look at the element under its offset
        const Tensor third_row = t.narrow(0, 3, 1);
        CHECK(third_row.offset() == 300);
        CHECK(be.item(third_row).to<T>() == host[300]);
        CHECK(be.data_ptr(third_row) == be.data_ptr(t) + 300 * sizeof(T));
        const Tensor filled(std::shared_ptr<StorageBase>(be.full(Scalar(T(7)), 33, 0)), to_scalar<T>::type, {33}, kAMD);
        CHECK(filled.to_vec<T>() == std::vector<T>(33, T(7)));
        const Tensor counted(std::shared_ptr<StorageBase>(be.arange(50, to_scalar<T>::type, 0)), to_scalar<T>::type, {50}, kAMD);
        std::vector<T> want(50);
        for (int i = 0; i < 50; ++i) want[static_cast<std::size_t>(i)] = static_cast<T>(i);
        CHECK(counted.to_vec<T>() == want);
        CHECK(Tensor(Scalar(T(5)), kAMD).item().to<T>() == T(5));
    });
    const Tensor flags(std::vector<bool>{true, false, true, true}, {4}, kAMD);
    CHECK(flags.dtype() == kBool);
    std::vector<uint8_t> bytes;
    be.to_vec(flags, bytes);
    CHECK(bytes == std::vector<uint8_t>{1, 0, 1, 1});
    CHECK(be.any(flags));
    CHECK(!be.all(flags));
    CHECK(be.all(flags.narrow(0, 2, 2)));
    CHECK(!be.any(Tensor(std::vector<float>(9, 0.0F), {3, 3}, kAMD)));
    CHECK(be.any(Tensor(std::vector<int32_t>{0, 0, -4}, {3}, kAMD)));
    // counters follow the storages; a device id out of range throws
    const auto before = be.current_memory_allocated(0);
    {
        const Tensor t(std::vector<float>(1024, 1.0F), {1024}, kAMD);
        CHECK(be.current_memory_allocated(0) == before + 4096);
        CHECK(be.total_memory_allocated(0) >= before + 4096);
    }
    CHECK(be.current_memory_allocated(0) == before);
    CHECK_THROWS_AS((void)be.from_vec(std::vector<float>(4, 0.F), be.get_device_count()), TTException);
}

TEST_CASE("batched_matmul: the reference's batched pattern at its own size, all dtypes") {
    // tests/test_matmul.cpp:200-236: B = 4, [379 x 1147] . [1147 x 635]
    const BackendBase &be = backend();
    for_all_except_bool([&]<typename T>() {
        constexpr int B = 4, N = 256 + 123, K = 1024 + 123, M = 512 + 123;
        std::vector<T> lhs, rhs;
        lhs.reserve(static_cast<std::size_t>(B) * N * K);
        rhs.reserve(static_cast<std::size_t>(B) * K * M);
        for (int b = 0; b < B; ++b) {
            for (int i = 0; i < N; ++i)
                for (int j = 0; j < K; ++j) lhs.push_back(static_cast<T>((i * b + j + b) % 100));
            for (int i = 0; i < K; ++i)
                for (int j = 0; j < M; ++j) rhs.push_back(static_cast<T>((i + j + 2 * b) % 100));
        }
        std::vector<T> expected(static_cast<std::size_t>(B) * N * M, T(0));
        for (int b = 0; b < B; ++b)
            gemm_naive(lhs.data() + static_cast<std::size_t>(b) * N * K, rhs.data() + static_cast<std::size_t>(b) * K * M,
                       expected.data() + static_cast<std::size_t>(b) * N * M, N, K, M);
        const Tensor got = be.batched_matmul(Tensor(lhs, {B, N, K}, kAMD), Tensor(rhs, {B, K, M}, kAMD));
        CHECK(got.shape() == Shape({B, N, M}));
        CHECK(got.is_contiguous());
        CHECK(got.dtype() == to_scalar<T>::type);
        CHECK(got.to_vec<T>() == expected);  // every partial sum is an integer below 2^24, or wraps
    });
}

TEST_CASE("batched_matmul on a permuted operand with an offset, read in place") {
    const BackendBase &be = backend();
    for_all_except_bool([&]<typename T>() {
        constexpr int B = 3, N = 70, K = 45, M = 130, PAD = 3;
        // lhs: columns PAD.. of a [B, N, K + PAD] storage (offset PAD, row stride K + PAD)
        const std::vector<T> lhs_store = pattern<T>(B * N * (K + PAD), 7, 3);
        const Tensor lhs = Tensor(lhs_store, {B, N, K + PAD}, kAMD).narrow(2, PAD, K);
        // rhs: stored transposed as [B + 1, M, K]; batches 1.. (offset M * K), then permuted to [B, K, M]
        const std::vector<T> rhs_store = pattern<T>((B + 1) * M * K, 5, 2);
        const Tensor rhs = Tensor(rhs_store, {B + 1, M, K}, kAMD).narrow(0, 1, B).permute({0, 2, 1});
        CHECK(lhs.offset() == PAD);
        CHECK(rhs.offset() == M * K);
        CHECK(rhs.stride() == Shape({M * K, 1, K}));
        std::vector<T> expected(static_cast<std::size_t>(B) * N * M, T(0));
        for (int b = 0; b < B; ++b)
            for (int n = 0; n < N; ++n)
                for (int k = 0; k < K; ++k)
                    for (int m = 0; m < M; ++m) {
                        const T a = lhs_store[(static_cast<std::size_t>(b) * N + n) * (K + PAD) + PAD + k];
                        const T r = rhs_store[(static_cast<std::size_t>(b + 1) * M + m) * K + k];
                        T &c = expected[(static_cast<std::size_t>(b) * N + n) * M + m];
                        c = static_cast<T>(c + static_cast<T>(a * r));
                    }
        CHECK(be.batched_matmul(lhs, rhs).to_vec<T>() == expected);
        // an expanded operand (stride 0 over the batch): every batch multiplies the same matrix
        const Tensor shared = Tensor(rhs_store, {B + 1, M, K}, kAMD).narrow(0, 2, 1).permute({0, 2, 1}).expand({B, K, M});
        CHECK(shared.stride()[0] == 0);
        std::vector<T> expected_shared(static_cast<std::size_t>(B) * N * M, T(0));
        for (int b = 0; b < B; ++b)
            for (int n = 0; n < N; ++n)
                for (int k = 0; k < K; ++k)
                    for (int m = 0; m < M; ++m) {
                        const T a = lhs_store[(static_cast<std::size_t>(b) * N + n) * (K + PAD) + PAD + k];
                        const T r = rhs_store[(static_cast<std::size_t>(2) * M + m) * K + k];
                        T &c = expected_shared[(static_cast<std::size_t>(b) * N + n) * M + m];
                        c = static_cast<T>(c + static_cast<T>(a * r));
                    }
        CHECK(be.batched_matmul(lhs, shared).to_vec<T>() == expected_shared);
    });
}

TEST_CASE("batched_matmul_pair: the two products of TensorBatchedMatmul::backward in one call") {
    // autograd/binary_ops.cpp:173-179: {grad . rhs^T, lhs^T . grad} on permuted views.  Not a virtual of BackendBase: called
    // on the adapter's class.  float at a Linear layer's size (both products in one grid) and every dtype at a small one (two
    // calls inside); data i % 7 - 3, every sum an integer below 2^24.
    const auto &be = dynamic_cast<const tinytensor::amd::BackendAMD &>(backend());
    auto run = [&]<typename T>(int B, int N, int K, int M) {
        const std::vector<T> lhs = pattern<T>(B * N * K, 7, 3), rhs = pattern<T>(B * K * M, 5, 2), grad = pattern<T>(B * N * M, 3, 1);
        const Tensor tl(lhs, {B, N, K}, kAMD), tr(rhs, {B, K, M}, kAMD), tg(grad, {B, N, M}, kAMD);
        const auto [dl, dr] = be.batched_matmul_pair(tg, tr.permute({0, 2, 1}), tl.permute({0, 2, 1}), tg);
        std::vector<T> want_l(lhs.size(), T(0)), want_r(rhs.size(), T(0));
        for (int b = 0; b < B; ++b)
            for (int n = 0; n < N; ++n)
                for (int m = 0; m < M; ++m) {
                    const T g = grad[(static_cast<std::size_t>(b) * N + n) * M + m];
                    for (int k = 0; k < K; ++k) {
                        T &a = want_l[(static_cast<std::size_t>(b) * N + n) * K + k];
                        a = static_cast<T>(a + static_cast<T>(g * rhs[(static_cast<std::size_t>(b) * K + k) * M + m]));
                        T &c = want_r[(static_cast<std::size_t>(b) * K + k) * M + m];
                        c = static_cast<T>(c + static_cast<T>(lhs[(static_cast<std::size_t>(b) * N + n) * K + k] * g));
                    }
                }
        CHECK(dl.shape() == Shape({B, N, K}));
        CHECK(dr.shape() == Shape({B, K, M}));
        CHECK(dl.to_vec<T>() == want_l);
        CHECK(dr.to_vec<T>() == want_r);
        // the same bits as the two calls of the interface where those run the same kernels (the small size)
        if (N < 256) {
            CHECK(be.batched_matmul(tg, tr.permute({0, 2, 1})).template to_vec<T>() == dl.template to_vec<T>());
            CHECK(be.batched_matmul(tl.permute({0, 2, 1}), tg).template to_vec<T>() == dr.template to_vec<T>());
        }
    };
    for_all_except_bool([&]<typename T>() { run.template operator()<T>(2, 37, 29, 45); });
    run.template operator()<float>(1, 576, 1000, 704);  // 144 and 176 tiles of 64 x 64, reductions of 704 and 576
}

TEST_CASE("conv2d: the reference's two geometries, all dtypes") {
    // tests/test_conv.cpp:99-143: [4,3,64,64] * [128,3,3,3], (stride, padding) = (1, 0) and (2, 1), data i % 10
    const BackendBase &be = backend();
    for_all_except_bool([&]<typename T>() {
        constexpr int B = 4, C = 3, O = 128, H = 64, W = 64, k = 3;
        const std::vector<T> x = pattern<T>(B * C * H * W, 10, 0);
        const std::vector<T> w = pattern<T>(O * C * k * k, 10, 0);
        const Tensor X(x, {B, C, H, W}, kAMD), Wt(w, {O, C, k, k}, kAMD);
        for (const auto &[S, P] : {std::pair{1, 0}, std::pair{2, 1}}) {
            const Tensor got = be.conv2d(X, Wt, std::nullopt, S, P);
            const int Ho = (H + 2 * P - k) / S + 1;
            CHECK(got.shape() == Shape({B, O, Ho, Ho}));
            CHECK(got.to_vec<T>() == conv_naive(x, w, static_cast<const std::vector<T> *>(nullptr), B, C, O, H, W, k, S, P));
        }
    });
}

TEST_CASE("conv2d with a bias, on an input view and a permuted weight") {
    const BackendBase &be = backend();
    for_floating_point([&]<typename T>() {
        constexpr int B = 3, C = 8, O = 5, H = 12, W = 8, k = 3, S = 1, P = 1;
        // the input is images 1..B of a [B + 1, C, H, W] storage; the weight is stored [C, O, k, k] and permuted
        const std::vector<T> x_store = pattern<T>((B + 1) * C * H * W, 9, 4);
        const std::vector<T> w_store = pattern<T>(C * O * k * k, 5, 2);
        const std::vector<T> bias = pattern<T>(O, 4, 1);
        const Tensor X = Tensor(x_store, {B + 1, C, H, W}, kAMD).narrow(0, 1, B);
        const Tensor Wt = Tensor(w_store, {C, O, k, k}, kAMD).permute({1, 0, 2, 3});
        CHECK(!Wt.is_contiguous());
        const std::vector<T> x(x_store.begin() + C * H * W, x_store.end());
        std::vector<T> w(w_store.size());
        for (int o = 0; o < O; ++o)
            for (int c = 0; c < C; ++c)
                for (int t = 0; t < k * k; ++t) w[(static_cast<std::size_t>(o) * C + c) * k * k + t] = w_store[(static_cast<std::size_t>(c) * O + o) * k * k + t];
        const Tensor got = be.conv2d(X, Wt, Tensor(bias, {O}, kAMD), S, P);
        CHECK(got.shape() == Shape({B, O, H, W}));
        CHECK(got.to_vec<T>() == conv_naive(x, w, &bias, B, C, O, H, W, k, S, P));
    });
}

TEST_CASE("conv2d_backward with and without a bias") {
    const BackendBase &be = backend();
    for_floating_point([&]<typename T>() {
        for (const auto &[S, P, C, O, H, W] : {std::tuple{2, 1, 3, 5, 9, 8}, std::tuple{1, 1, 8, 32, 8, 8}, std::tuple{1, 0, 4, 6, 7, 5}}) {
            constexpr int B = 2, k = 3;
            const int Ho = (H + 2 * P - k) / S + 1, Wo = (W + 2 * P - k) / S + 1;
            const std::vector<T> x = pattern<T>(B * C * H * W, 7, 3);
            const std::vector<T> w = pattern<T>(O * C * k * k, 5, 2);
            // grad_output arrives as a view: rows 1.. of a taller storage
            const std::vector<T> g_store = pattern<T>(B * O * (Ho + 1) * Wo, 3, 1);
            const Tensor G = Tensor(g_store, {B, O, Ho + 1, Wo}, kAMD).narrow(2, 1, Ho);
            std::vector<T> g;
            for (int i = 0; i < B * O; ++i)
                for (int y = 1; y <= Ho; ++y)
                    for (int xx = 0; xx < Wo; ++xx) g.push_back(g_store[(static_cast<std::size_t>(i) * (Ho + 1) + y) * Wo + xx]);
            std::vector<T> gin, gw, gb;
            conv_backward_naive(g, x, w, B, C, O, H, W, k, S, P, gin, gw, gb);
            const Tensor X(x, {B, C, H, W}, kAMD), Wt(w, {O, C, k, k}, kAMD);
            const Tensor bias(pattern<T>(O, 3, 1), {O}, kAMD);
            {
                const auto [gX, gW, gB] = be.conv2d_backward(G, X, Wt, bias, S, P);
                CHECK(gX.shape() == X.shape());
                CHECK(gW.shape() == Wt.shape());
                CHECK(gB.has_value());
                CHECK(gX.template to_vec<T>() == gin);
                CHECK(gW.template to_vec<T>() == gw);
                CHECK(gB->shape() == Shape({O}));
                CHECK(gB->template to_vec<T>() == gb);
            }
            {
                const auto [gX, gW, gB] = be.conv2d_backward(G, X, Wt, std::nullopt, S, P);
                CHECK(!gB.has_value());
                CHECK(gX.template to_vec<T>() == gin);
                CHECK(gW.template to_vec<T>() == gw);
            }
        }
    });
    const Tensor xi(std::vector<int32_t>(2 * 3 * 5 * 5, 1), {2, 3, 5, 5}, kAMD), wi(std::vector<int32_t>(4 * 3 * 3 * 3, 1), {4, 3, 3, 3}, kAMD);
    const Tensor gi(std::vector<int32_t>(2 * 4 * 3 * 3, 1), {2, 4, 3, 3}, kAMD);
    CHECK_THROWS_AS((void)be.conv2d_backward(gi, xi, wi, std::nullopt, 1, 0), TTException);  // integers are not differentiated
}

TEST_CASE("sum over a dimension and over everything, through views") {
    const BackendBase &be = backend();
    constexpr int A = 6, Bd = 37, Cd = 21;
    const std::vector<int32_t> hi = pattern<int32_t>(A * Bd * Cd, 11, 5);
    const std::vector<float> hf(hi.begin(), hi.end());
    const Tensor ti = Tensor(hi, {A, Bd, Cd}, kAMD).permute({2, 0, 1}).narrow(1, 1, A - 1);   // [Cd, A - 1, Bd]
    const Tensor tf = Tensor(hf, {A, Bd, Cd}, kAMD).permute({2, 0, 1}).narrow(1, 1, A - 1);
    auto at = [&](int c, int a, int b) { return hi[(static_cast<std::size_t>(a + 1) * Bd + b) * Cd + c]; };
    for (int dim = 0; dim < 3; ++dim) {
        const Tensor si = be.sum(ti, dim), sf = be.sum(tf, dim);
        Shape want_shape = ti.shape();
        want_shape[dim] = 1;
        CHECK(si.shape() == want_shape);
        CHECK(sf.shape() == want_shape);
        CHECK(si.dtype() == kI64);  // integers sum in 64 bits
        CHECK(sf.dtype() == kF32);
        std::vector<int64_t> want;
        const int n0 = dim == 0 ? 1 : Cd, n1 = dim == 1 ? 1 : A - 1, n2 = dim == 2 ? 1 : Bd;
        for (int c = 0; c < n0; ++c)
            for (int a = 0; a < n1; ++a)
                for (int b = 0; b < n2; ++b) {
                    int64_t s = 0;
                    for (int r = 0; r < ti.size(dim); ++r) s += at(dim == 0 ? r : c, dim == 1 ? r : a, dim == 2 ? r : b);
                    want.push_back(s);
                }
        CHECK(si.to_vec<int64_t>() == want);
        const std::vector<float> gotf = sf.to_vec<float>();
        CHECK(gotf.size() == want.size());
        for (std::size_t i = 0; i < want.size() && i < gotf.size(); ++i) CHECK(gotf[i] == static_cast<float>(want[i]));
    }
    int64_t total = 0;
    for (int c = 0; c < Cd; ++c)
        for (int a = 0; a < A - 1; ++a)
            for (int b = 0; b < Bd; ++b) total += at(c, a, b);
    const Tensor all = be.sum(ti);
    CHECK(all.shape() == Shape({1}));
    CHECK(be.item(all).to<int64_t>() == total);
    CHECK(be.item(be.sum(tf)).to<float>() == static_cast<float>(total));
}

TEST_CASE("identity, assign and to(dtype) through views") {
    const BackendBase &be = backend();
    for_all_except_bool([&]<typename T>() {
        constexpr int A = 5, Bd = 7, Cd = 6;
        const std::vector<T> host = pattern<T>(A * Bd * Cd, 50, 10);
        const Tensor base(host, {A, Bd, Cd}, kAMD);
        const Tensor view = base.permute({1, 2, 0}).narrow(0, 2, 4).narrow(1, 1, 3);  // [4, 3, A] of [Bd, Cd, A]
        std::vector<T> want;
        for (int b = 2; b < 6; ++b)
            for (int c = 1; c < 4; ++c)
                for (int a = 0; a < A; ++a) want.push_back(host[(static_cast<std::size_t>(a) * Bd + b) * Cd + c]);
        const Tensor dense = be.identity(view);
        CHECK(dense.is_contiguous());
        CHECK(dense.shape() == Shape({4, 3, A}));
        std::vector<T> got;
        be.to_vec(dense, got);
        CHECK(got == want);
        // to(dtype) reads through the view too
        const std::vector<double> as_double = be.to(view, kF64).template to_vec<double>();
        CHECK(as_double.size() == want.size());
        for (std::size_t i = 0; i < want.size() && i < as_double.size(); ++i) CHECK(as_double[i] == static_cast<double>(want[i]));
        // assign writes through the view and leaves every other element of the storage alone
        Tensor target(std::vector<T>(host.size(), T(1)), {A, Bd, Cd}, kAMD);
        Tensor target_view = target.permute({1, 2, 0}).narrow(0, 2, 4).narrow(1, 1, 3);
        be.assign(target_view, dense);
        std::vector<T> expect_store(host.size(), T(1));
        for (int b = 2; b < 6; ++b)
            for (int c = 1; c < 4; ++c)
                for (int a = 0; a < A; ++a) {
                    const std::size_t i = (static_cast<std::size_t>(a) * Bd + b) * Cd + c;
                    expect_store[i] = host[i];
                }
        std::vector<T> store;
        be.to_vec(target, store);
        CHECK(store == expect_store);
    });
}

TEST_CASE("element-wise operators, comparisons, where and the in-place forms") {
    const BackendBase &be = backend();
    for_floating_point([&]<typename T>() {
        constexpr int R = 33, Cn = 20;
        const std::vector<T> a = pattern<T>(R * Cn, 13, 6), b = pattern<T>(R * Cn, 7, 3);
        const Tensor A(a, {R, Cn}, kAMD);
        const Tensor Bt = Tensor(b, {Cn, R}, kAMD).permute({1, 0});  // element (r, c) is b[c * R + r]
        auto bv = [&](int r, int c) { return b[static_cast<std::size_t>(c) * R + r]; };
        std::vector<T> add, mul, relu, picked, maxed;
        std::vector<uint8_t> lt;
        for (int r = 0; r < R; ++r)
            for (int c = 0; c < Cn; ++c) {
                const T x = a[static_cast<std::size_t>(r) * Cn + c], y = bv(r, c);
                add.push_back(x + y);
                mul.push_back(x * y);
                lt.push_back(x < y ? 1 : 0);
                relu.push_back(y < T(0) ? T(0) : y);
                picked.push_back(x < y ? x : y);
                maxed.push_back(std::max(x, y));
            }
        CHECK(be.add(A, Bt).to_vec<T>() == add);
        CHECK(be.mul(A, Bt).to_vec<T>() == mul);
        CHECK(be.maximum(A, Bt).to_vec<T>() == maxed);
        const Tensor mask = be.lt(A, Bt);
        CHECK(mask.dtype() == kBool);
        CHECK(mask.to_vec<uint8_t>() == lt);
        CHECK(be.relu(Bt).to_vec<T>() == relu);
        CHECK(be.where(mask, A, Bt).to_vec<T>() == picked);
        // in place through a view: add_inplace on the transposed view changes b's storage in its own order
        Tensor Bview = Tensor(b, {Cn, R}, kAMD).permute({1, 0});
        be.add_inplace(Bview, A);
        CHECK(Bview.to_vec<T>() == add);
        Tensor Brelu = Tensor(b, {Cn, R}, kAMD).permute({1, 0});
        be.relu_(Brelu);
        CHECK(Brelu.to_vec<T>() == relu);
        // a value expanded over the shape as the second operand (what `tensor * 2` builds)
        const Tensor two = Tensor(Scalar(T(2)), kAMD).expand({R, Cn});
        std::vector<T> doubled;
        for (const T v : a) doubled.push_back(v * T(2));
        CHECK(be.mul(A, two).to_vec<T>() == doubled);
    });
}

TEST_CASE("uniform_real_ and normal_: through a view, with expanded and with per-element parameters") {
    const BackendBase &be = backend();
    for_floating_point([&]<typename T>() {
        constexpr int A = 4, Bd = 6, Cd = 5;
        Tensor base(std::vector<T>(A * Bd * Cd, T(-7)), {A, Bd, Cd}, kAMD);
        Tensor view = base.permute({1, 0, 2}).narrow(0, 1, Bd - 1).narrow(2, 1, 3);  // [Bd - 1, A, 3], offset Cd + 1
        CHECK(view.offset() == Cd + 1);
        const int n = view.numel();
        // one value expanded over the shape, as Tensor::uniform_real_(double, double) passes it
        const T low = T(-0.5), high = T(0.25);
        const Tensor t_low = Tensor(Scalar(low), kAMD).expand(view.shape()), t_high = Tensor(Scalar(high), kAMD).expand(view.shape());
        Generator gen(17), twin(17);
        be.uniform_real_(view, t_low, t_high, gen);
        std::vector<T> expect(static_cast<std::size_t>(A) * Bd * Cd, T(-7));
        {
            int i = 0;
            for (int b = 1; b < Bd; ++b)
                for (int a = 0; a < A; ++a)
                    for (int c = 1; c < 4; ++c, ++i) {
                        Generator element = Generator::from_state(twin());
                        expect[(static_cast<std::size_t>(a) * Bd + b) * Cd + c] = std::fma(unit_draw<T>(element()), high - low, low);
                    }
            CHECK(i == n);
        }
        std::vector<T> store;
        be.to_vec(base, store);
        CHECK(store == expect);
        CHECK(gen() == twin());  // both consumed one output per element
        // a pair per element: low dense, high a permuted view, non-constant
        std::vector<T> lows(static_cast<std::size_t>(n)), highs_store(static_cast<std::size_t>(n));
        for (int i = 0; i < n; ++i) lows[static_cast<std::size_t>(i)] = static_cast<T>(-1.0 + 0.03125 * (i % 29));
        const Tensor t_lows(lows, {Bd - 1, A, 3}, kAMD);
        for (int c = 0; c < 3; ++c)
            for (int b = 0; b < Bd - 1; ++b)
                for (int a = 0; a < A; ++a)
                    highs_store[(static_cast<std::size_t>(c) * (Bd - 1) + b) * A + a] =
                        lows[(static_cast<std::size_t>(b) * A + a) * 3 + c] + static_cast<T>(0.5 + 0.25 * ((a + 2 * b + c) % 5));
        const Tensor t_highs = Tensor(highs_store, {3, Bd - 1, A}, kAMD).permute({1, 2, 0});
        Generator gen2(23), twin2(23);
        be.uniform_real_(view, t_lows, t_highs, gen2);
        {
            int i = 0;
            for (int b = 1; b < Bd; ++b)
                for (int a = 0; a < A; ++a)
                    for (int c = 1; c < 4; ++c, ++i) {
                        Generator element = Generator::from_state(twin2());
                        const T lo = lows[static_cast<std::size_t>(i)];
                        const T hi = highs_store[(static_cast<std::size_t>(c - 1) * (Bd - 1) + (b - 1)) * A + a];
                        expect[(static_cast<std::size_t>(a) * Bd + b) * Cd + c] = std::fma(unit_draw<T>(element()), hi - lo, lo);
                    }
        }
        be.to_vec(base, store);
        CHECK(store == expect);
        // the out-of-place form returns a dense tensor of the parameters' shape
        Generator gen3(23);
        const Tensor fresh = be.uniform_real(t_lows, t_highs, gen3);
        CHECK(fresh.shape() == view.shape());
        CHECK(fresh.to_vec<T>() == view.to_vec<T>());
        // normal_: mu + std * sqrt(-2 log1p(-u1)) sin(2 pi u2), within the two math libraries' rounding
        const Tensor mu = Tensor(Scalar(T(0.25)), kAMD).expand(view.shape());
        std::vector<T> stds(static_cast<std::size_t>(n));
        for (int i = 0; i < n; ++i) stds[static_cast<std::size_t>(i)] = static_cast<T>(0.1 + 0.05 * (i % 7));
        Generator gen4(5), twin4(5);
        be.normal_(view, mu, Tensor(stds, {Bd - 1, A, 3}, kAMD), gen4);
        const std::vector<T> drawn = view.to_vec<T>();
        CHECK(static_cast<int>(drawn.size()) == n);
        double worst = 0.0;
        for (int i = 0; i < n && i < static_cast<int>(drawn.size()); ++i) {
            Generator element = Generator::from_state(twin4());
            const double u1 = static_cast<double>(unit_draw<T>(element())), u2 = static_cast<double>(unit_draw<T>(element()));
            const double z = std::sqrt(-2.0 * std::log1p(-u1)) * std::sin(2.0 * 3.14159265358979323846 * u2);
            worst = std::max(worst, std::fabs(static_cast<double>(drawn[static_cast<std::size_t>(i)]) - (0.25 + static_cast<double>(stds[static_cast<std::size_t>(i)]) * z)));
        }
        CHECK(worst <= (sizeof(T) == 4 ? 2e-6 : 1e-13));
        // an integer tensor is refused
        Tensor ints(std::vector<int32_t>(4, 0), {4}, kAMD);
        const Tensor zero = Tensor(Scalar(int32_t(0)), kAMD).expand({4}), one = Tensor(Scalar(int32_t(1)), kAMD).expand({4});
        CHECK_THROWS_AS(be.uniform_real_(ints, zero, one, gen4), TTException);
    });
}

TEST_CASE("pooling forward and backward") {
    const BackendBase &be = backend();
    constexpr int B = 2, C = 3, H = 8, W = 6;
    const std::vector<float> x = pattern<float>(B * C * H * W, 17, 8);
    const Tensor X(x, {B, C, H, W}, kAMD);
    const Tensor pooled = be.max_pool2d(X, 2, 2, 0);
    CHECK(pooled.shape() == Shape({B, C, H / 2, W / 2}));
    std::vector<float> want_max, want_avg;
    for (int p = 0; p < B * C; ++p)
        for (int y = 0; y < H / 2; ++y)
            for (int xx = 0; xx < W / 2; ++xx) {
                const float *q = x.data() + (static_cast<std::size_t>(p) * H + 2 * y) * W + 2 * xx;
                want_max.push_back(std::max(std::max(q[0], q[1]), std::max(q[W], q[W + 1])));
                want_avg.push_back(q[0] / 4 + q[1] / 4 + q[W] / 4 + q[W + 1] / 4);
            }
    CHECK(pooled.to_vec<float>() == want_max);
    CHECK(be.avg_pool2d(X, 2, 2, 0).to_vec<float>() == want_avg);
    // avg backward spreads each gradient evenly over its window
    const std::vector<float> g = pattern<float>(B * C * (H / 2) * (W / 2), 5, 2);
    const Tensor G(g, {B, C, H / 2, W / 2}, kAMD);
    std::vector<float> want_grad(x.size());
    for (int p = 0; p < B * C; ++p)
        for (int y = 0; y < H; ++y)
            for (int xx = 0; xx < W; ++xx)
                want_grad[(static_cast<std::size_t>(p) * H + y) * W + xx] = g[(static_cast<std::size_t>(p) * (H / 2) + y / 2) * (W / 2) + xx / 2] / 4;
    const Tensor grad = be.avg_pool2d_backward(G, X, be.avg_pool2d(X, 2, 2, 0), 2, 2, 0);
    CHECK(grad.shape() == X.shape());
    CHECK(grad.to_vec<float>() == want_grad);
}

TEST_CASE("what is not on the path says so") {
    const BackendBase &be = backend();
    const Tensor t(std::vector<float>(12, 1.0F), {3, 4}, kAMD);
    CHECK_THROWS_AS((void)be.softmax(t, 1), TTException);
    CHECK_THROWS_AS((void)be.sin(t), TTException);
    CHECK_THROWS_AS((void)be.gather(t, t, 0), TTException);
    CHECK_THROWS_AS((void)be.argmax(t), TTException);
    Generator gen(1);
    CHECK_THROWS_AS((void)be.bernoulli(t, gen), TTException);
    try {
        (void)be.modulo(t, t);
        CHECK(false);
    } catch (const TTException &e) {
        CHECK(std::string(e.what()).find("modulo is not implemented on the AMD device") != std::string::npos);
    }
    // printing formats a host copy through the CPU device, which the stand-in Tensor does not have
    std::ostringstream os;
    CHECK_THROWS_AS(be.print(os, t), TTException);
}

int main(int argc, char **argv) {
    return mini::run_all(argc, argv);
}
