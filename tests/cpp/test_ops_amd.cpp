// test_ops_amd.cpp — the operations around the GEMMs on the AMD device, checked against plain host loops in the
// style of the reference's tests/test_binary.cpp, test_reduce.cpp, test_to.cpp and the pooling cases of
// tests/test_conv.cpp:186-278 (whose expected values come from a naive window loop here instead of libtorch):
// elementwise binary / unary with broadcasting, where, sum, full, to(dtype), assign through views, max / min / avg
// pooling forward and backward, seeded uniform draws and nn::Linear's default initialisation.
#include "mini_test.h"

#include <chrono>
#include <limits>

using namespace tt_amd;

namespace {
template <typename T>
std::vector<T> pattern(int n, int mod, int shift) {
    std::vector<T> v;
    for (int i = 0; i < n; ++i) v.push_back(static_cast<T>((i * 7 + 3) % mod + shift));
    return v;
}
template <typename T, typename R, typename F>
std::vector<R> pool_naive(const std::vector<T> &X, int B, int C, int H, int W, int K, int S, int P, R init, F fold) {
    const int Ho = (H + 2 * P - K) / S + 1, Wo = (W + 2 * P - K) / S + 1;
    std::vector<R> out(static_cast<std::size_t>(B) * C * Ho * Wo);
    for (int bc = 0; bc < B * C; ++bc)
        for (int h = 0; h < Ho; ++h)
            for (int w = 0; w < Wo; ++w) {
                R acc = init;
                for (int p = 0; p < K; ++p)
                    for (int q = 0; q < K; ++q) {
                        const int hi = S * h + p - P, wi = S * w + q - P;
                        const R x = (hi < 0 || wi < 0 || hi >= H || wi >= W) ? init : static_cast<R>(X[(static_cast<std::size_t>(bc) * H + hi) * W + wi]);
                        acc = fold(x, acc);
                    }
                out[(static_cast<std::size_t>(bc) * Ho + h) * Wo + w] = acc;
            }
    return out;
}
}  // namespace

TEST_CASE("Binary ops with broadcasting") {
    auto test = []<typename T>(Device device) {
        const int R = 37, Cn = 19;
        const auto a = pattern<T>(R * Cn, 11, 1), b = pattern<T>(Cn, 5, 1);
        const Tensor A(a, {R, Cn}, device), Bv(b, {Cn}, device);
        std::vector<T> sum_, dif, prod, quot, mx;
        std::vector<bool> less;
        for (int i = 0; i < R * Cn; ++i) {
            const T x = a[static_cast<std::size_t>(i)], y = b[static_cast<std::size_t>(i % Cn)];
            sum_.push_back(static_cast<T>(x + y));
            dif.push_back(static_cast<T>(x - y));
            prod.push_back(static_cast<T>(x * y));
            quot.push_back(static_cast<T>(x / y));
            mx.push_back(x > y ? x : y);
            less.push_back(x < y);
        }
        CHECK((A + Bv).template to_vec<T>() == sum_);
        CHECK((A - Bv).template to_vec<T>() == dif);
        CHECK((A * Bv).template to_vec<T>() == prod);
        CHECK((A / Bv).template to_vec<T>() == quot);
        CHECK(maximum(A, Bv).template to_vec<T>() == mx);
        const Tensor L = A < Bv;
        CHECK(L.dtype() == kBool);
        CHECK(L.template to_vec<bool>() == less);
        // a transposed view as the left operand
        const Tensor At = A.permute({1, 0});
        const auto t = (At + At).template to_vec<T>();
        bool ok = true;
        for (int c = 0; c < Cn; ++c)
            for (int r = 0; r < R; ++r) ok = ok && t[static_cast<std::size_t>(c * R + r)] == static_cast<T>(2 * a[static_cast<std::size_t>(r * Cn + c)]);
        CHECK(ok);
        CHECK_THROWS_AS(std::ignore = A + Tensor(pattern<T>(R, 5, 1), {R}, device), TTException);  // not broadcastable
        // mixed dtypes are promoted (tensor/tensor.cpp:2272-2274): T with f64 gives f64
        std::vector<double> bd, mixed;
        for (int i = 0; i < Cn; ++i) bd.push_back(0.5 + i);
        for (int i = 0; i < R * Cn; ++i) mixed.push_back(static_cast<double>(a[static_cast<std::size_t>(i)]) + bd[static_cast<std::size_t>(i % Cn)]);
        const Tensor M = A + Tensor(bd, {Cn}, device);
        CHECK(M.dtype() == kF64);
        CHECK(M.template to_vec<double>() == mixed);
    };
    runner_all_except_bool(test);
}

TEST_CASE("Unary ops, where, sum, full") {
    auto test = []<typename T>(Device device) {
        const int N = 1000;
        std::vector<T> a;
        for (int i = 0; i < N; ++i) a.push_back(static_cast<T>((i % 13) - 6) / T(4));
        const Tensor A(a, {10, 100}, device);
        std::vector<T> r, e;
        for (T x : a) {
            r.push_back(x > T(0) ? x : T(0));
            e.push_back(std::exp(x));
        }
        CHECK(relu(A).template to_vec<T>() == r);
        CHECK(allclose(get_backend(device)->exp(A).template to_vec<T>(), e, 1e-6, 1e-7));
        // relu backward as the reference writes it: where(input > 0, grad, 0) (autograd/unary_ops.cpp:568-573)
        const Tensor zero = full(T(0), A.shape(), device), grad = full(T(2.5), A.shape(), device);
        const auto g = where(A > zero, grad, zero).template to_vec<T>();
        bool ok = true;
        for (int i = 0; i < N; ++i) ok = ok && g[static_cast<std::size_t>(i)] == (a[static_cast<std::size_t>(i)] > T(0) ? T(2.5) : T(0));
        CHECK(ok);
        // sums of multiples of 1/4 are exact in any order
        double total = 0;
        for (T x : a) total += static_cast<double>(x);
        CHECK(A.sum().template to_vec<T>() == std::vector<T>{static_cast<T>(total)});
        std::vector<T> cols(100, T(0)), rows(10, T(0));
        for (int i = 0; i < 10; ++i)
            for (int j = 0; j < 100; ++j) {
                cols[static_cast<std::size_t>(j)] += a[static_cast<std::size_t>(i * 100 + j)];
                rows[static_cast<std::size_t>(i)] += a[static_cast<std::size_t>(i * 100 + j)];
            }
        CHECK(A.sum(0).template to_vec<T>() == cols);
        CHECK(A.sum(-1).template to_vec<T>() == rows);
    };
    runner_floating_point(test);
}

TEST_CASE("To") {
    auto test = []<typename T>(Device device) {
        const auto a = pattern<T>(300, 100, 0);
        const Tensor A(a, {3, 100}, device);
        auto expect = [&]<typename R>(R) {
            std::vector<R> e;
            for (T x : a) e.push_back(static_cast<R>(x));
            return e;
        };
        CHECK(A.to(kU8).template to_vec<uint8_t>() == expect(uint8_t{}));
        CHECK(A.to(kI16).template to_vec<int16_t>() == expect(int16_t{}));
        CHECK(A.to(kI32).template to_vec<int32_t>() == expect(int32_t{}));
        CHECK(A.to(kI64).template to_vec<int64_t>() == expect(int64_t{}));
        CHECK(A.to(kF32).template to_vec<float>() == expect(float{}));
        CHECK(A.to(kF64).template to_vec<double>() == expect(double{}));
        std::vector<bool> eb;
        for (T x : a) eb.push_back(x != T(0));
        CHECK(A.to(kBool).template to_vec<bool>() == eb);
        CHECK(A.to(A.dtype()).storage() == A.storage());  // same dtype: the tensor itself (tensor.cpp:536-538)
        // matmul promotes mixed operands (tensor.cpp:2394-2399): T x f64 -> f64
        const std::vector<double> w(100 * 2, 0.5);
        const Tensor Y = matmul(A, Tensor(w, {100, 2}, device));
        CHECK(Y.dtype() == kF64);
        std::vector<double> ey;
        for (int r = 0; r < 3; ++r) {
            double acc = 0;
            for (int k = 0; k < 100; ++k) acc += 0.5 * static_cast<double>(a[static_cast<std::size_t>(r * 100 + k)]);
            ey.push_back(acc);
            ey.push_back(acc);
        }
        CHECK(Y.template to_vec<double>() == ey);
    };
    runner_all_except_bool(test);
}

TEST_CASE("Assign through views") {
    auto test = []<typename T>(Device device) {
        auto base = pattern<T>(60, 50, 0);
        const auto rhs = pattern<T>(12, 9, 60);
        Tensor Bt(base, {6, 10}, device);
        Tensor window(Bt.storage(), Bt.dtype(), Shape({4, 3}), Shape({10, 2}), 12, device);  // rows 1..4, columns 2,4,6
        window.assign(Tensor(rhs, {3, 4}, device).permute({1, 0}));
        for (int i = 0; i < 4; ++i)
            for (int j = 0; j < 3; ++j) base[static_cast<std::size_t>((1 + i) * 10 + 2 + 2 * j)] = rhs[static_cast<std::size_t>(j * 4 + i)];
        CHECK(Bt.template to_vec<T>() == base);
        CHECK_THROWS_AS(window.assign(Tensor(rhs, {12}, device)), TTException);
    };
    runner_all_except_bool(test);
}

TEST_CASE("Pool2D Forward") {
    auto test = []<typename T>(Device device) {
        // tests/test_conv.cpp:186-278: B4 C128 68x28, k3 s2 p1
        const int B = 4, C = 128, H = 68, W = 28, K = 3, S = 2, P = 1;
        std::vector<T> x;
        for (int i = 0; i < B * C * H * W; ++i) x.push_back(static_cast<T>((i * 2654435761u >> 7) % 97) - T(40 * (std::is_signed_v<T> ? 1 : 0)));
        const Tensor X(x, {B, C, H, W}, device);
        using L = std::numeric_limits<T>;
        CHECK(max_pool2d(X, K, S, P).template to_vec<T>() ==
              pool_naive<T, T>(x, B, C, H, W, K, S, P, L::lowest(), [](T v, T acc) { return v > acc ? v : acc; }));
        CHECK(min_pool2d(X, K, S, P).template to_vec<T>() ==
              pool_naive<T, T>(x, B, C, H, W, K, S, P, L::max(), [](T v, T acc) { return v < acc ? v : acc; }));
        using R = std::conditional_t<std::is_floating_point_v<T>, T, float>;
        const R n = static_cast<R>(K * K);
        const Tensor avg = avg_pool2d(X, K, S, P);
        CHECK(avg.dtype() == to_scalar<R>::type);
        CHECK(avg.shape() == Shape({B, C, 34, 14}));
        CHECK(avg.template to_vec<R>() == pool_naive<T, R>(x, B, C, H, W, K, S, P, R(0), [n](R v, R acc) { return (v / n) + acc; }));
    };
    runner_all_except_bool(test);
    CHECK_THROWS_AS(std::ignore = max_pool2d(Tensor(std::vector<bool>(16, true), {1, 1, 4, 4}, kAMD), 2, 2, 0), TTException);
    CHECK_THROWS_AS(std::ignore = avg_pool2d(Tensor(std::vector<float>(16, 1.f), {1, 4, 4}, kAMD), 2, 2, 0), TTException);
    CHECK_THROWS_AS(std::ignore = min_pool2d(Tensor(std::vector<float>(16, 1.f), {1, 1, 4, 4}, kAMD), 6, 1, 1), TTException);
}

TEST_CASE("Pool2D Backward") {
    auto test = []<typename T>(Device device) {
        const int B = 2, C = 3, H = 9, W = 8, K = 3, S = 2, P = 1;
        const int Ho = (H + 2 * P - K) / S + 1, Wo = (W + 2 * P - K) / S + 1;
        std::vector<T> x, g;
        for (int i = 0; i < B * C * H * W; ++i) x.push_back(static_cast<T>((i * 5) % 4));  // ties
        for (int i = 0; i < B * C * Ho * Wo; ++i) g.push_back(static_cast<T>(i % 9 - 4));
        const Tensor X(x, {B, C, H, W}, device), G(g, {B, C, Ho, Wo}, device);
        for (int op = 0; op < 3; ++op) {
            const Tensor res = op == 0 ? max_pool2d(X, K, S, P) : op == 1 ? min_pool2d(X, K, S, P) : avg_pool2d(X, K, S, P);
            const Tensor gx = op == 0 ? max_pool2d_backward(G, X, res, K, S, P)
                              : op == 1 ? min_pool2d_backward(G, X, res, K, S, P)
                                        : avg_pool2d_backward(G, X, res, K, S, P);
            const auto r = res.template to_vec<T>();
            std::vector<T> want(x.size(), T(0));  // the reference's scatter loop (cpu/kernel/conv.hpp:171-275)
            for (int bc = 0; bc < B * C; ++bc)
                for (int h = 0; h < Ho; ++h)
                    for (int w = 0; w < Wo; ++w) {
                        const std::size_t ir = (static_cast<std::size_t>(bc) * Ho + h) * Wo + w;
                        T count = op == 2 ? static_cast<T>(K * K) : T(0);
                        auto each = [&](auto &&f) {
                            for (int p = 0; p < K; ++p)
                                for (int q = 0; q < K; ++q) {
                                    const int hi = S * h + p - P, wi = S * w + q - P;
                                    if (hi < 0 || wi < 0 || hi >= H || wi >= W) continue;
                                    const std::size_t ii = (static_cast<std::size_t>(bc) * H + hi) * W + wi;
                                    if (op == 2 || x[ii] == r[ir]) f(ii);
                                }
                        };
                        if (op != 2) each([&](std::size_t) { count += T(1); });
                        const T share = g[ir] / count;
                        each([&](std::size_t ii) { want[ii] += share; });
                    }
            CHECK(gx.template to_vec<T>() == want);
        }
    };
    runner_floating_point(test);
}

TEST_CASE("Seeded draws and Linear default init") {
    Generator g1(42), g2(42), g3(43);
    const Tensor a = uniform_real(-2.0, 3.0, {1000, 7}, g1), b = uniform_real(-2.0, 3.0, {1000, 7}, g2), c = uniform_real(-2.0, 3.0, {1000, 7}, g3);
    const auto va = a.to_vec<float>(), vb = b.to_vec<float>(), vc = c.to_vec<float>();
    CHECK(va == vb);
    CHECK(va != vc);
    CHECK(g1.state == g2.state);
    double mean = 0;
    bool in_range = true;
    for (float v : va) {
        mean += v;
        in_range = in_range && v >= -2.0f && v < 3.0f;
    }
    CHECK(in_range);
    CHECK(std::abs(mean / static_cast<double>(va.size()) - 0.5) < 0.06);
    CHECK_THROWS_AS(std::ignore = uniform_real(1.0, 1.0, {4}, g1), TTException);
    // nn::Linear(in, out): weight [in,out] ~ U(+-sqrt(3/in)), bias ~ U(+-1/sqrt(in)), drawn in that order
    Generator gl(7), gr(7);
    const nn::Linear layer(256, 64, true, gl);
    CHECK(layer.weight.shape() == Shape({256, 64}));
    CHECK(layer.bias->shape() == Shape({64}));
    const double bw = std::sqrt(3.0 / 256.0), bb = 1.0 / 16.0;
    CHECK(layer.weight.to_vec<float>() == uniform_real(-bw, bw, {256, 64}, gr).to_vec<float>());
    CHECK(layer.bias->to_vec<float>() == uniform_real(-bb, bb, {64}, gr).to_vec<float>());
    const Tensor X = uniform_real(-1.0, 1.0, {8, 256}, gr);
    const Tensor Y = layer.forward(X);
    CHECK(Y.shape() == Shape({8, 64}));
    CHECK(allclose(Y.to_vec<float>(), (matmul(X, layer.weight) + *layer.bias).to_vec<float>(), 1e-5, 1e-6));
}

TEST_CASE("Conv2d default init through the permuted view") {
    // nn::Conv2d (nn/conv2d.cpp:20-66): kaiming_uniform_ on weight.permute({1,0,2,3}) -- the draws run over [in,out,k,k]
    // with fan = in*k*k -- then the bias with fan = out*k*k.  Stated independently: a dense draw of [in,out,k,k],
    // permuted back and made contiguous.
    const int in = 5, out = 12, k = 3;
    Generator gl(11), gr(11);
    const nn::Conv2d layer(in, out, k, 1, 1, true, gl);
    CHECK(layer.weight.shape() == Shape({out, in, k, k}));
    CHECK(layer.weight.is_contiguous());
    const double bw = std::sqrt(3.0) * (1.0 / std::sqrt(static_cast<double>(in * k * k))), bb = 1.0 / std::sqrt(static_cast<double>(out * k * k));
    const Tensor dense = uniform_real(-bw, bw, {in, out, k, k}, gr);
    CHECK(layer.weight.to_vec<float>() == dense.permute({1, 0, 2, 3}).to_vec<float>());
    CHECK(layer.weight.to_vec<float>() != dense.to_vec<float>());
    CHECK(layer.bias->to_vec<float>() == uniform_real(-bb, bb, {out}, gr).to_vec<float>());
    CHECK(gl.state == gr.state);
    // in-place draws through a view leave the rest of the storage alone
    Tensor base = full(-7.0f, Shape({4, 6}), kAMD).contiguous();
    Generator g1(5), g2(5);
    Tensor cols = base.permute({1, 0});  // [6,4] view with strides (1,6)
    cols.uniform_real_(0.0, 1.0, g1);
    CHECK(base.to_vec<float>() == uniform_real(0.0, 1.0, {6, 4}, g2).permute({1, 0}).to_vec<float>());
    // forward = conv2d with the layer's stride and padding
    const Tensor x = uniform_real(-1.0, 1.0, {2, in, 9, 9}, gr);
    const Tensor y = layer.forward(x);
    CHECK(y.shape() == Shape({2, out, 9, 9}));
    CHECK(y.to_vec<float>() == conv2d(x, layer.weight, layer.bias, 1, 1).to_vec<float>());
    CHECK_THROWS_AS(std::ignore = layer.forward(uniform_real(-1.0, 1.0, {2, in + 1, 9, 9}, gr)), TTException);
    CHECK_THROWS_AS(nn::Conv2d(0, 4, 3, 1, 0, true, gl), TTException);
    CHECK_THROWS_AS(nn::Conv2d(4, 4, 3, 0, 0, true, gl), TTException);
    CHECK_THROWS_AS(nn::Conv2d(4, 4, 3, 1, -1, true, gl), TTException);
}

TEST_CASE("Integer sums are 64-bit") {
    // common/reduce.h:56-61: sums of bool and integer tensors accumulate in int64 and return an i64 tensor
    auto test = []<typename T>(Device device) {
        if constexpr (std::is_integral_v<T>) {
            const int N = 60000;
            std::vector<T> a;
            int64_t total = 0;
            for (int i = 0; i < N; ++i) {
                a.push_back(static_cast<T>(100 + i % 27));
                total += 100 + i % 27;
            }
            const Tensor A(a, {600, 100}, device);
            CHECK(A.sum().dtype() == kI64);
            CHECK(A.sum().template to_vec<int64_t>() == std::vector<int64_t>{total});  // 6.7e6: beyond u8 and i16
            std::vector<int64_t> cols(100, 0);
            for (int i = 0; i < N; ++i) cols[static_cast<std::size_t>(i % 100)] += static_cast<int64_t>(a[static_cast<std::size_t>(i)]);
            CHECK(A.sum(0).template to_vec<int64_t>() == cols);
        }
    };
    runner_all_except_bool(test);
    std::vector<bool> m;
    for (int i = 0; i < 1000; ++i) m.push_back(i % 3 == 0);
    const Tensor M(m, {10, 100}, kAMD);
    CHECK(M.sum().dtype() == kI64);
    CHECK(M.sum().to_vec<int64_t>() == std::vector<int64_t>{334});
}

namespace {
struct MlpGrads {
    Tensor loss, dW1, db1, dW2, db2, dW3, db3, dX;
};
// One training step of Linear-ReLU-Linear-ReLU-Linear + mse_loss, op for op as the reference's autograd emits it
// (nn/linear.cpp:42-50, autograd/unary_ops.cpp:568-573, nn/loss.cpp:69-72, autograd/binary_ops.cpp:173-179).
MlpGrads mlp_step(const Tensor &x, const Tensor &t, const nn::Linear &l1, const nn::Linear &l2, const nn::Linear &l3) {
    const Device dev = x.device();
    const Tensor z1 = l1.forward(x), a1 = relu(z1), z2 = l2.forward(a1), a2 = relu(z2), y = l3.forward(a2);
    const Tensor diff = y - t;
    const float n = static_cast<float>(y.numel());
    MlpGrads g;
    g.loss = (diff * diff).sum() / full(n, Shape({1}), dev);
    const Tensor gy = full(1.0f / n * 2.0f, y.shape(), dev) * diff;
    g.db3 = gy.sum(0);
    auto [da2, dW3] = matmul_backward(a2.unsqueeze(0), l3.weight.unsqueeze(0), gy.unsqueeze(0));
    const Tensor zero = full(0.0f, z2.shape(), dev), one = full(1.0f, z2.shape(), dev);
    const Tensor dz2 = da2.squeeze(0) * where(z2 < zero, zero, one);
    g.db2 = dz2.sum(0);
    auto [da1, dW2] = matmul_backward(a1.unsqueeze(0), l2.weight.unsqueeze(0), dz2.unsqueeze(0));
    const Tensor zero1 = full(0.0f, z1.shape(), dev), one1 = full(1.0f, z1.shape(), dev);
    const Tensor dz1 = da1.squeeze(0) * where(z1 < zero1, zero1, one1);
    g.db1 = dz1.sum(0);
    auto [dX, dW1] = matmul_backward(x.unsqueeze(0), l1.weight.unsqueeze(0), dz1.unsqueeze(0));
    g.dW3 = dW3.squeeze(0);
    g.dW2 = dW2.squeeze(0);
    g.dW1 = dW1.squeeze(0);
    g.dX = dX.squeeze(0);
    return g;
}
// The same step from the fused forms: Linear + ReLU in one launch, the loss with its gradient and the head's bias
// gradient in one, and per layer one GEMM for dx (ReLU mask and bias gradient in its store) and one for dW.
MlpGrads mlp_step_fused(const Tensor &x, const Tensor &t, const nn::Linear &l1, const nn::Linear &l2, const nn::Linear &l3, bool own_bias = false,
                        bool head = false) {
    const auto [z1, a1] = l1.forward_relu(x);
    const auto [z2, a2] = l2.forward_relu(a1);
    if (head) {  // the last layer, the loss and their backward in one call; the other two layers as with own_bias
        const nn::HeadResult h = nn::linear_mse_head(a2, l3.weight, &*l3.bias, t, &z2);
        const nn::LinearGrads g2 = nn::linear_backward(h.dx, a1, l2.weight, &z1, nn::BiasGrad::kOwn);
        const nn::LinearGrads g1 = nn::linear_backward(g2.dx, x, l1.weight, nullptr, nn::BiasGrad::kOwn);
        return MlpGrads{h.loss, g1.dW, *g1.db, g2.dW, *g2.db, h.dW, *h.db, g1.dx};
    }
    const Tensor y = l3.forward(a2);
    const nn::MseLoss loss = nn::mse_loss(y, t, true);
    MlpGrads g;
    g.loss = loss.loss;
    g.db3 = *loss.grad_colsum;
    if (own_bias) {  // layers 1 and 2 take their bias gradients from the weight-gradient products
        const nn::LinearGrads g3 = nn::linear_backward(loss.grad_input, a2, l3.weight, &z2);
        const nn::LinearGrads g2 = nn::linear_backward(g3.dx, a1, l2.weight, &z1, nn::BiasGrad::kOwn);
        const nn::LinearGrads g1 = nn::linear_backward(g2.dx, x, l1.weight, nullptr, nn::BiasGrad::kOwn);
        g.dW3 = g3.dW;
        g.db2 = *g2.db;
        g.dW2 = g2.dW;
        g.db1 = *g1.db;
        g.dW1 = g1.dW;
        g.dX = g1.dx;
        return g;
    }
    const nn::LinearGrads g3 = nn::linear_backward(loss.grad_input, a2, l3.weight, &z2, nn::BiasGrad::kPrev);
    const nn::LinearGrads g2 = nn::linear_backward(g3.dx, a1, l2.weight, &z1, nn::BiasGrad::kPrev);
    const nn::LinearGrads g1 = nn::linear_backward(g2.dx, x, l1.weight);
    g.dW3 = g3.dW;
    g.db2 = *g3.db;
    g.dW2 = g2.dW;
    g.db1 = *g2.db;
    g.dW1 = g1.dW;
    g.dX = g1.dx;
    return g;
}
}  // namespace

TEST_CASE("MLP training step") {
    // small layer sizes against a finite-difference check of the loss, then the benchmark-sized step for its time
    Generator gen(3);
    const int B = 16, D0 = 12, D1 = 9, D2 = 7, D3 = 4;
    const nn::Linear l1(D0, D1, true, gen), l2(D1, D2, true, gen), l3(D2, D3, true, gen);
    const Tensor x = uniform_real(0.0, 1.0, {B, D0}, gen), t = uniform_real(0.0, 1.0, {B, D3}, gen);
    const MlpGrads g = mlp_step(x, t, l1, l2, l3);
    const float loss0 = g.loss.to_vec<float>()[0];
    CHECK(loss0 > 0.0f);
    // d loss / d W3[i][j] by central differences on a copy of the weights
    const auto w3 = l3.weight.to_vec<float>(), dW3 = g.dW3.to_vec<float>();
    for (int idx : {0, 5, 13, 27}) {
        auto wp = w3, wm = w3;
        wp[static_cast<std::size_t>(idx)] += 1e-2f;
        wm[static_cast<std::size_t>(idx)] -= 1e-2f;
        const nn::Linear lp(Tensor(wp, {D2, D3}, kAMD), l3.bias), lm(Tensor(wm, {D2, D3}, kAMD), l3.bias);
        const float fp = mlp_step(x, t, l1, l2, lp).loss.to_vec<float>()[0], fm = mlp_step(x, t, l1, l2, lm).loss.to_vec<float>()[0];
        CHECK(std::abs((fp - fm) / 2e-2f - dW3[static_cast<std::size_t>(idx)]) < 2e-3f);
    }
    // bias gradients are the column sums of the layer's output gradient: db3 = sum over the batch of gy
    CHECK(g.db3.shape() == Shape({D3}));
    CHECK(g.dW1.shape() == Shape({D0, D1}));
    CHECK(g.dX.shape() == Shape({B, D0}));
    // benchmark size: batch 1024, 784 -> 1024 -> 1024 -> 10
    Generator gb(0);
    const nn::Linear b1(784, 1024, true, gb), b2(1024, 1024, true, gb), b3(1024, 10, true, gb);
    const Tensor X = uniform_real(0.0, 1.0, {1024, 784}, gb), T = uniform_real(0.0, 1.0, {1024, 10}, gb);
    for (int i = 0; i < 5; ++i) (void)mlp_step(X, T, b1, b2, b3);
    check(ttamd_device_synchronize(0));
    const auto t0 = std::chrono::steady_clock::now();
    const int iters = 30;
    for (int i = 0; i < iters; ++i) (void)mlp_step(X, T, b1, b2, b3);
    check(ttamd_device_synchronize(0));
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / iters;
    std::printf("  MLP training step 1024 x (784-1024-1024-10), C++ host layer, op by op: %.3f ms per step\n", ms);
    CHECK(ms < 50.0);
    // the same step from the fused forms (at most 15 launches); every result against the op-by-op step
    const MlpGrads ref = mlp_step(X, T, b1, b2, b3), fused = mlp_step_fused(X, T, b1, b2, b3);
    auto close = [](const Tensor &a, const Tensor &b) {
        const auto va = a.to_vec<float>(), vb = b.to_vec<float>();
        float big = 0.0f, err = 0.0f;
        for (std::size_t i = 0; i < va.size(); ++i) {
            big = std::max(big, std::abs(vb[i]));
            err = std::max(err, std::abs(va[i] - vb[i]));
        }
        return va.size() == vb.size() && err <= 1e-5f * big;
    };
    CHECK(close(fused.loss, ref.loss));
    CHECK(close(fused.dW1, ref.dW1));
    CHECK(close(fused.db1, ref.db1));
    CHECK(close(fused.dW2, ref.dW2));
    CHECK(close(fused.db2, ref.db2));
    CHECK(close(fused.dW3, ref.dW3));
    CHECK(close(fused.db3, ref.db3));
    CHECK(close(fused.dX, ref.dX));
    for (int i = 0; i < 5; ++i) (void)mlp_step_fused(X, T, b1, b2, b3);
    check(ttamd_device_synchronize(0));
    const auto t1 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i) (void)mlp_step_fused(X, T, b1, b2, b3);
    check(ttamd_device_synchronize(0));
    const double ms_fused = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t1).count() / iters;
    std::printf("  the same step from the fused forms (11 launches): %.3f ms per step\n", ms_fused);
    CHECK(ms_fused < 50.0);
    // ... with the bias gradients of layers 1 and 2 from the weight-gradient products (10 launches)
    const MlpGrads own = mlp_step_fused(X, T, b1, b2, b3, true);
    CHECK(close(own.db1, ref.db1));
    CHECK(close(own.db2, ref.db2));
    CHECK(close(own.dW1, ref.dW1));
    CHECK(close(own.dW2, ref.dW2));
    CHECK(close(own.dW3, ref.dW3));
    CHECK(close(own.dX, ref.dX));
    for (int i = 0; i < 5; ++i) (void)mlp_step_fused(X, T, b1, b2, b3, true);
    check(ttamd_device_synchronize(0));
    const auto t2 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i) (void)mlp_step_fused(X, T, b1, b2, b3, true);
    check(ttamd_device_synchronize(0));
    const double ms_own = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t2).count() / iters;
    std::printf("  the same with the bias gradients from the weight-gradient products (10 launches): %.3f ms per step\n", ms_own);
    CHECK(ms_own < 50.0);
    // ... and with the last layer, the loss and their backward in one call (8 launches)
    const MlpGrads hd = mlp_step_fused(X, T, b1, b2, b3, true, true);
    CHECK(close(hd.loss, ref.loss));
    CHECK(close(hd.db1, ref.db1));
    CHECK(close(hd.db2, ref.db2));
    CHECK(close(hd.db3, ref.db3));
    CHECK(close(hd.dW1, ref.dW1));
    CHECK(close(hd.dW2, ref.dW2));
    CHECK(close(hd.dW3, ref.dW3));
    CHECK(close(hd.dX, ref.dX));
    for (int i = 0; i < 5; ++i) (void)mlp_step_fused(X, T, b1, b2, b3, true, true);
    check(ttamd_device_synchronize(0));
    const auto t3 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i) (void)mlp_step_fused(X, T, b1, b2, b3, true, true);
    check(ttamd_device_synchronize(0));
    const double ms_head = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t3).count() / iters;
    std::printf("  the same with the last layer and the loss in one call (8 launches): %.3f ms per step\n", ms_head);
    CHECK(ms_head < 50.0);
}

int main(int argc, char **argv) { return mini::run_all(argc, argv); }
