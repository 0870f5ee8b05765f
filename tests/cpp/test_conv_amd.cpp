// test_conv_amd.cpp — the reference's conv2d forward test (tests/test_conv.cpp:29-143: B4, C3 -> 128, 64x64, k3,
// (s1,p0) and (s2,p1), data i % 10, naive 7-deep loop as the oracle, all non-bool dtypes) against the AMD device,
// plus the backward pass checked through the adjoint identities <g, conv(x,w)> = <gX, x> = <gW, w>.
#include "mini_test.h"

using namespace tt_amd;

namespace {
template <typename T>
std::vector<T> conv_forward(const std::vector<T> &X, const std::vector<T> &W, int B, int C_in, int C_out, int H_in, int W_in, int K, int S, int P) {
    const int H_out = (H_in + 2 * P - K) / S + 1, W_out = (W_in + 2 * P - K) / S + 1;
    std::vector<T> Y(static_cast<std::size_t>(B) * C_out * H_out * W_out, 0);
    for (int b = 0; b < B; ++b)
        for (int m = 0; m < C_out; ++m)
            for (int h = 0; h < H_out; ++h)
                for (int w = 0; w < W_out; ++w)
                    for (int c = 0; c < C_in; ++c)
                        for (int p = 0; p < K; ++p)
                            for (int q = 0; q < K; ++q) {
                                const int h_in = S * h + p - P, w_in = S * w + q - P;
                                if (h_in < 0 || w_in < 0 || h_in >= H_in || w_in >= W_in) continue;
                                Y[((static_cast<std::size_t>(b) * C_out + m) * H_out + h) * W_out + w] += static_cast<T>(
                                    X[((static_cast<std::size_t>(b) * C_in + c) * H_in + h_in) * W_in + w_in] * W[((m * C_in + c) * K + p) * K + q]);
                            }
    return Y;
}
template <typename T>
std::vector<T> init_vec(int size) {
    std::vector<T> res;
    for (int i = 0; i < size; ++i) res.push_back(static_cast<T>(i % 10));
    return res;
}
template <typename T>
double dot(const std::vector<T> &a, const std::vector<T> &b) {
    double s = 0;
    for (std::size_t i = 0; i < a.size(); ++i) s += static_cast<double>(a[i]) * static_cast<double>(b[i]);
    return s;
}
}  // namespace

TEST_CASE("Conv2D Forward") {
    for (auto [S, P] : {std::pair{1, 0}, std::pair{2, 1}}) {
        auto test = [S = S, P = P]<typename T>(Device device) {
            const int B = 4, C_in = 3, C_out = 128, H_in = 64, W_in = 64, K = 3;
            const int H_out = (H_in + 2 * P - K) / S + 1, W_out = (W_in + 2 * P - K) / S + 1;
            const auto _X = init_vec<T>(B * C_in * H_in * W_in), _W = init_vec<T>(C_out * C_in * K * K);
            const Tensor X(_X, {B, C_in, H_in, W_in}, device), W(_W, {C_out, C_in, K, K}, device);
            const Tensor Y = conv2d(X, W, {}, S, P);
            CHECK(Y.shape() == Shape({B, C_out, H_out, W_out}));
            CHECK(Y.template to_vec<T>() == conv_forward(_X, _W, B, C_in, C_out, H_in, W_in, K, S, P));
        };
        runner_all_except_bool(test);
    }
}

TEST_CASE("Conv2D Backward adjoints") {
    auto test = []<typename T>(Device device) {
        const int B = 3, C = 4, O = 5, H = 9, W = 8, K = 3, S = 2, P = 1;
        std::vector<T> x, w, bias(O, T(0)), g;
        for (int i = 0; i < B * C * H * W; ++i) x.push_back(static_cast<T>(i % 7 - 3));
        for (int i = 0; i < O * C * K * K; ++i) w.push_back(static_cast<T>(i % 5 - 2));
        const Tensor X(x, {B, C, H, W}, device), Wt(w, {O, C, K, K}, device), Bi(bias, {O}, device);
        const Tensor Y = conv2d(X, Wt, Bi, S, P);
        const auto y = Y.template to_vec<T>();
        CHECK(y == conv_forward(x, w, B, C, O, H, W, K, S, P));
        for (std::size_t i = 0; i < y.size(); ++i) g.push_back(static_cast<T>(static_cast<int>(i % 3) - 1));
        const auto [gX, gW, gB] = conv2d_backward(Tensor(g, Y.shape(), device), X, Wt, Bi, S, P);
        CHECK(gB.has_value());
        const double lhs = dot(g, y);
        CHECK(lhs == dot(gX.template to_vec<T>(), x));  // integer-valued data: exact
        CHECK(lhs == dot(gW.template to_vec<T>(), w));
        // grad_bias = sum of g over batch and space
        const auto gb = gB->template to_vec<T>();
        const int HoWo = Y.size(2) * Y.size(3);
        for (int o = 0; o < O; ++o) {
            double s = 0;
            for (int b = 0; b < B; ++b)
                for (int i = 0; i < HoWo; ++i) s += static_cast<double>(g[(static_cast<std::size_t>(b) * O + o) * HoWo + i]);
            CHECK(static_cast<double>(gb[static_cast<std::size_t>(o)]) == s);
        }
        const auto [gX2, gW2, gB2] = conv2d_backward(Tensor(g, Y.shape(), device), X, Wt, {}, S, P);
        CHECK(!gB2.has_value());
    };
    runner_floating_point(test);
    CHECK_THROWS_AS((void)conv2d(Tensor(std::vector<float>(2 * 3 * 8 * 8, 1.f), {2, 3, 8, 8}, kAMD),
                                 Tensor(std::vector<float>(4 * 2 * 3 * 3, 1.f), {4, 2, 3, 3}, kAMD)), TTException);
}

int main(int argc, char **argv) { return mini::run_all(argc, argv); }
