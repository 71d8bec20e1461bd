// Runs the C++ host veneer (dlf-style DevTensor front-ends over gpgpu::dnn over
// the C ABI) against the literal vectors the reference's own tests hold, plus
// the veneer's error and temporary-buffer behaviour.  Needs a GPU.  Exit code 0
// when every check passes; failures are listed on stderr.
//
// Vectors: dlf/test/UniformTest.cpp:1857-1965 (reduce), :2106-2189 (scan),
// :2304-2377 (sort), dlf/test/DNNTest.cpp:861-1019 (argmax/argmin),
// dlf/test/model/PredictTest.cpp:609-637 (top_k), dlf/test/UniformTest.cpp:2065-2080
// (count), :2553-2561 (nonzero), :2250-2283 (merge), dlf/test/DNNTest.cpp:796-858
// (softmax, logsoftmax, hardmax).
#include <algorithm>
#include <cmath>
#include <complex>
#include <cstdio>
#include <random>

#include "dev_tensor.h"

using namespace dlf;

static int g_failed = 0, g_checked = 0;

#define CHECK(cond)                                                              \
    do {                                                                         \
        ++g_checked;                                                             \
        if (!(cond)) {                                                           \
            ++g_failed;                                                          \
            std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
        }                                                                        \
    } while (0)

template <typename T>
static bool near(const Tensor<T>& a, const Tensor<T>& b, double tol = 1e-4) {
    if (a.shape() != b.shape()) return false;
    for (size_t i = 0; i < a.size(); ++i) {
        const double x = a.values()[i], y = b.values()[i];
        if (std::fabs(x - y) > tol && std::fabs(x - y) > tol * std::fabs(y)) return false;
    }
    return true;
}

static void test_reduce() {
    auto X = Tensor<float>({3, 2, 2}, {5, 1, 20, 2, 30, 1, 40, 2, 55, 1, 60, 2});
    CHECK(reduce_max(dev(X), {}, true).read() == Tensor<float>({1, 1, 1}, {60}));
    CHECK(reduce_max(dev(X), {1}, false).read() == Tensor<float>({3, 2}, {20, 2, 40, 2, 60, 2}));
    CHECK(reduce_max(dev(X), {1}, true).read() == Tensor<float>({3, 1, 2}, {20, 2, 40, 2, 60, 2}));
    CHECK(reduce_min(dev(X), {}, true).read() == Tensor<float>({1, 1, 1}, {1}));
    CHECK(reduce_min(dev(X), {1}).read() == Tensor<float>({3, 2}, {5, 1, 30, 1, 55, 1}));

    auto R = Tensor<float>({3, 3, 3}).range();
    CHECK(reduce_sum(dev(R), {0}).read() == Tensor<float>({3, 3}, {27, 30, 33, 36, 39, 42, 45, 48, 51}));
    CHECK(reduce_sum(dev(R), {1}).read() == Tensor<float>({3, 3}, {9, 12, 15, 36, 39, 42, 63, 66, 69}));
    CHECK(reduce_sum(dev(R), {2}).read() == Tensor<float>({3, 3}, {3, 12, 21, 30, 39, 48, 57, 66, 75}));
    CHECK(reduce_sum(dev(R), {0, 2}).read() == Tensor<float>({3}, {90, 117, 144}));
    CHECK(reduce_mean(dev(R), {0}, true).read() == Tensor<float>({1, 3, 3}, {9, 10, 11, 12, 13, 14, 15, 16, 17}));
    CHECK(reduce_mean(dev(R), {0, 2}, true).read() == Tensor<float>({1, 3, 1}, {10, 13, 16}));
    CHECK(reduce_sum(dev(R), {-1}).read() == reduce_sum(dev(R), {2}).read());

    auto P = Tensor<float>({3, 2, 2}).range(1);
    CHECK(near(reduce_prod(dev(P), {}, true).read(), Tensor<float>({1, 1, 1}, {4.790016e+08f})));
    CHECK(near(reduce_prod(dev(P), {1}).read(), Tensor<float>({3, 2}, {3, 8, 35, 48, 99, 120})));
    // log_sum_exp(X) == log(sum_exp(X)) (UniformTest.cpp:1995-1998)
    auto lse = reduce_log_sum_exp(dev(P), {1}).read();
    auto se = reduce_sum_exp(dev(P), {1}).read();
    for (size_t i = 0; i < lse.size(); ++i) CHECK(std::fabs(lse.values()[i] - std::log(se.values()[i])) < 1e-4);

    // transposed view (a non-contiguous input)
    auto dX = dev(R);
    CHECK(reduce_sum(dX.transpose(), {0}).read() == Tensor<float>({3, 3}, {3, 30, 57, 12, 39, 66, 21, 48, 75}));
}

static void test_arg_reduce() {
    auto X = Tensor<float>({2, 3, 4}, {21, 22, 2, 15, 16, 7, 14, 0, 18, 20, 6, 9, 23, 4, 12, 11, 10, 5, 3, 8, 17, 19, 13, 1});
    CHECK(argmax(dev(X), 0).read() == Tensor<int>({1, 3, 4}, {1, 0, 1, 0, 0, 0, 0, 1, 0, 0, 1, 0}));
    CHECK(argmax(dev(X), 0, false).read() == Tensor<int>({3, 4}, {1, 0, 1, 0, 0, 0, 0, 1, 0, 0, 1, 0}));
    CHECK(argmax(dev(X), 1).read() == Tensor<int>({2, 1, 4}, {0, 0, 1, 0, 0, 2, 2, 0}));
    CHECK(argmax(dev(X), 2, false).read() == Tensor<int>({2, 3}, {1, 0, 1, 0, 0, 1}));
    auto N = Tensor<float>({2, 3, 4}, {0, 6, 9, 22, 18, 7, 21, 14, 17, 23, 12, 5, 8, 4, 20, 2, 15, 1, 10, 19, 1, 16, 11, 13});
    CHECK(argmin(dev(N), 0).read() == Tensor<int>({1, 3, 4}, {0, 1, 0, 1, 1, 1, 1, 0, 1, 1, 1, 0}));
    CHECK(argmin(dev(N), 1, false).read() == Tensor<int>({2, 4}, {0, 0, 0, 2, 2, 1, 1, 0}));
    CHECK(argmin(dev(N), 2).read() == Tensor<int>({2, 3, 1}, {0, 1, 3, 3, 1, 0}));
    CHECK(argmax(dev(X), -1).read() == argmax(dev(X), 2).read());
}

static void test_scan() {
    auto A = Tensor<int>({5, 5}).range(1);
    auto dA = dev(A);
    CHECK(cumsum(dA, 0).read() == Tensor<int>({5, 5}, {1, 2, 3, 4, 5, 7, 9, 11, 13, 15, 18, 21, 24, 27, 30, 34, 38, 42, 46, 50, 55, 60, 65, 70, 75}));
    CHECK(cumsum(dA, 1).read() == Tensor<int>({5, 5}, {1, 3, 6, 10, 15, 6, 13, 21, 30, 40, 11, 23, 36, 50, 65, 16, 33, 51, 70, 90, 21, 43, 66, 90, 115}));
    CHECK(cumsum(dA, 0, true).read() == Tensor<int>({5, 5}, {0, 0, 0, 0, 0, 1, 2, 3, 4, 5, 7, 9, 11, 13, 15, 18, 21, 24, 27, 30, 34, 38, 42, 46, 50}));
    CHECK(cumsum(dA, 1, false, true).read() == Tensor<int>({5, 5}, {15, 14, 12, 9, 5, 40, 34, 27, 19, 10, 65, 54, 42, 29, 15, 90, 74, 57, 39, 20, 115, 94, 72, 49, 25}));
    CHECK(cumsum(dA, 0, true, true).read() == Tensor<int>({5, 5}, {54, 58, 62, 66, 70, 48, 51, 54, 57, 60, 37, 39, 41, 43, 45, 21, 22, 23, 24, 25, 0, 0, 0, 0, 0}));
    auto B = Tensor<int>({10}).range(1);
    CHECK(cumprod(dev(B), 0).read() == Tensor<int>({10}, {1, 2, 6, 24, 120, 720, 5040, 40320, 362880, 3628800}));

    // [2, 100000] random ints against a serial host scan (UniformTest.cpp:2188-2189)
    std::mt19937 rg(7);
    std::vector<int> v(2 * 100000);
    for (auto& e : v) e = static_cast<int>(rg());
    auto X = Tensor<int>({2, 100000}, v);
    auto got = cumsum(dev(X)).read();
    bool same = true;
    for (int r = 0; r < 2; ++r) {
        unsigned acc = 0;
        for (int i = 0; i < 100000; ++i) {
            acc += static_cast<unsigned>(v[r * 100000 + i]);
            same = same && got.values()[r * 100000 + i] == static_cast<int>(acc);
        }
    }
    CHECK(same);
    // in place
    auto dX = dev(X);
    cumsum(dX, dX, 1);
    CHECK(dX.read() == got);
}

static void test_sort() {
    auto X = Tensor<int>({3, 4, 5}, {8, 19, 11, 41, 53, 79, 2, 10, 0, 94, 37, 30, 82, 81, 75, 60, 18, 66, 47, 51,
                                     91, 83, 67, 88, 76, 17, 17, 73, 16, 65, 66, 62, 56, 90, 18, 32, 65, 11, 46, 24,
                                     57, 38, 77, 56, 0, 82, 69, 78, 3, 83, 57, 37, 97, 93, 32, 78, 96, 15, 80, 95});
    auto dX = dev(X);
    CHECK(sorted(dX, 0).read() == Tensor<int>({3, 4, 5}, {8, 19, 11, 41, 0, 17, 2, 10, 0, 65, 37, 30, 56, 81, 18, 32, 18, 11, 46, 24,
                                                           57, 38, 67, 56, 53, 79, 17, 73, 3, 83, 57, 37, 82, 90, 32, 60, 65, 15, 47, 51,
                                                           91, 83, 77, 88, 76, 82, 69, 78, 16, 94, 66, 62, 97, 93, 75, 78, 96, 66, 80, 95}));
    CHECK(sorted(dX, 2).read() == Tensor<int>({3, 4, 5}, {8, 11, 19, 41, 53, 0, 2, 10, 79, 94, 30, 37, 75, 81, 82, 18, 47, 51, 60, 66,
                                                           67, 76, 83, 88, 91, 16, 17, 17, 65, 73, 18, 56, 62, 66, 90, 11, 24, 32, 46, 65,
                                                           0, 38, 56, 57, 77, 3, 69, 78, 82, 83, 32, 37, 57, 93, 97, 15, 78, 80, 95, 96}));
    // argsort: gather(X, I) == sorted(X); values variant and in-place values (UniformTest.cpp:2403-2440)
    for (int axis = 0; axis < 3; ++axis) {
        auto S = sorted(dX, axis).read();
        DevTensor<int> Y;
        DevTensor<int32_t> I;
        argsort(dX, Y, I, axis);
        CHECK(Y.read() == S);
        auto idx = I.read();
        auto xv = moveaxis(dX, axis, -1).read(), sv = moveaxis(dev(S), axis, -1).read(), iv = moveaxis(I, axis, -1).read();
        const size_t n = xv.extent(-1);
        bool ok = true;
        for (size_t i = 0; i < xv.size(); ++i) ok = ok && xv.values()[(i / n) * n + iv.values()[i]] == sv.values()[i];
        CHECK(ok);
        CHECK(argsort(dX, axis).read() == idx);
        auto Z = dev(X);
        argsort(Z, Z, I, axis);
        CHECK(Z.read() == S);
    }
    auto D = sorted(dX, 1, true).read(), A = sorted(dX, 1, false).read();
    bool rev = true;
    for (size_t b = 0; b < 3; ++b)
        for (size_t j = 0; j < 4; ++j)
            for (size_t c = 0; c < 5; ++c) rev = rev && D.values()[b * 20 + j * 5 + c] == A.values()[b * 20 + (3 - j) * 5 + c];
    CHECK(rev);
    auto one = Tensor<float>({4, 1}, {3, 1, 2, 0});
    CHECK(sorted(dev(one), 1).read() == one);
}

static void test_top_k() {
    auto X = Tensor<float>({3, 4}, {0, 1, 2, 3, 7, 6, 5, 4, 10, 11, 9, 8});
    auto r = top_k(dev(X), 3);
    CHECK(r.first.read() == Tensor<float>({3, 3}, {3, 2, 1, 7, 6, 5, 11, 10, 9}));
    CHECK(r.second.read() == Tensor<int32_t>({3, 3}, {3, 2, 1, 0, 1, 2, 1, 0, 2}));
    auto c = top_k(dev(X), 100, 0, false);              // limit clamps to the extent
    CHECK(c.first.read() == Tensor<float>({3, 4}, {0, 1, 2, 3, 7, 6, 5, 4, 10, 11, 9, 8}));
    auto T = Tensor<int>({1, 6}, {5, 9, 5, 9, 1, 9});
    CHECK(top_k(dev(T), 4).second.read() == Tensor<int32_t>({1, 4}, {1, 3, 5, 0}));   // lowest index first among ties
}

static void test_count_nonzero() {
    auto A = Tensor<float>({3, 3}, {1, 0, 3, 0, 2, 4, 0, 0, 3});
    auto dA = dev(A);
    CHECK(count(dA, 0.0f, {0}).read() == Tensor<int>({3}, {2, 2, 0}));
    CHECK(count(dA, 0.0f, {1}).read() == Tensor<int>({3}, {1, 1, 2}));
    CHECK(count(dA, 0.0f).read() == Tensor<int>(Shape(std::vector<size_t>{}), {4}));
    CHECK(count(dA.transpose(), 0.0f, {1}).read() == Tensor<int>({3}, {2, 2, 0}));

    auto X = Tensor<float>({2, 2, 2}, {1, 0, 0, 2, 5, 6, 0, 0});
    auto Y = Tensor<int32_t>({3, 4}, {0, 0, 1, 1, 0, 1, 0, 0, 0, 1, 0, 1});
    CHECK(nonzero(dev(X), true).read() == Y);
    CHECK(nonzero(dev(X)).transpose().read() == Y);
    CHECK(nonzero(dev(Tensor<float>({2, 2}, {0, 0, 0, 0}))).empty());
    // a transposed input is walked in the row-major order of the view
    auto Xt = dev(Tensor<int64_t>({2, 3}, {0, 7, 0, 8, 0, 9})).transpose();
    CHECK(nonzero(Xt).read() == Tensor<int32_t>({3, 2}, {0, 1, 1, 0, 2, 1}));
}

static void test_softmax_family() {
    // DNNTest.cpp:796-858
    auto X = Tensor<float>({2, 4}, {0, 1, 2, 3, 10000, 10001, 10002, 10003});
    CHECK(near(dnn::softmax(dev(X)).read(), Tensor<float>({2, 4}, {0.0320586f, 0.08714432f, 0.23688284f, 0.64391428f,
                                                                   0.0320586f, 0.08714432f, 0.23688284f, 0.64391428f})));
    CHECK(near(dnn::logsoftmax(dev(X)).read(), Tensor<float>({2, 4}, {-3.4401896f, -2.4401896f, -1.44018972f, -0.44018969f,
                                                                      -3.4401896f, -2.4401896f, -1.44018972f, -0.44018969f})));
    auto H = Tensor<float>({4, 4}, {3, 0, 1, 2, 2, 5, 1, 0, 0, 1, 3, 2, 0, 1, 2, 3});
    CHECK(dnn::hardmax(dev(H)).read() == Tensor<float>({4, 4}, {1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1}));
    CHECK(dnn::hardmax(dev(Tensor<float>({1, 4}, {3, 3, 3, 1}))).read() == Tensor<float>({1, 4}, {1, 0, 0, 0}));
    // in place, and a transposed input (copied to row-major order first)
    auto D = dev(H);
    dnn::hardmax(D, D);
    CHECK(D.read() == Tensor<float>({4, 4}, {1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1}));
    CHECK(dnn::hardmax(dev(H).transpose()).read() == Tensor<float>({4, 4}, {1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1}));
}

static void test_merge() {
    // UniformTest.cpp:2250-2283: merge of two sorted vectors == std::merge
    std::mt19937 rng(7);
    std::vector<int> a(2000), b(3000), want(5000);
    for (auto& v : a) v = static_cast<int>(rng() % 100000);
    for (auto& v : b) v = static_cast<int>(rng() % 100000);
    std::sort(a.begin(), a.end());
    std::sort(b.begin(), b.end());
    std::merge(a.begin(), a.end(), b.begin(), b.end(), want.begin());
    auto C = merge(dev(Tensor<int>({2000}, a)), dev(Tensor<int>({3000}, b)));
    CHECK(C.read() == Tensor<int>({5000}, want));
    // along the first axis of matrices (a strided axis)
    auto A2 = dev(Tensor<float>({3, 2}, {1, 10, 3, 20, 5, 30}));
    auto B2 = dev(Tensor<float>({2, 2}, {2, 15, 4, 25}));
    CHECK(merge(A2, B2, 0).read() == Tensor<float>({5, 2}, {1, 10, 2, 15, 3, 20, 4, 25, 5, 30}));
    bool threw = false;
    try { merge(A2, dev(Tensor<float>({2, 3}).range()), 0); } catch (const shape_error&) { threw = true; }
    CHECK(threw);
}

// 16-bit element types through the same front-ends: order-based results are exact, half sums
// are formed in float and rounded once.
static void test_16bit_types() {
    using gpgpu::blas::half;
    auto S = Tensor<int16_t>({2, 6}, {5, -3, 300, -30000, 7, 5, 1, 1, 0, -1, 32767, -32768});
    DevTensor<int16_t> SS;
    sort(dev(S), SS, -1);
    CHECK(SS.read() == Tensor<int16_t>({2, 6}, {-30000, -3, 5, 5, 7, 300, -32768, -1, 0, 1, 1, 32767}));
    DevTensor<int16_t> SV;
    DevTensor<int32_t> SI;
    argsort(dev(S), SV, SI, -1, true);
    CHECK(SI.read() == Tensor<int32_t>({2, 6}, {2, 4, 0, 5, 1, 3, 4, 0, 1, 2, 3, 5}));
    CHECK(argmax(dev(S), 1, false).read() == Tensor<int>({2}, {2, 4}));
    DevTensor<int16_t> TV;
    DevTensor<int32_t> TI;
    top_k(dev(S), TV, TI, 2, -1, true);
    CHECK(TV.read() == Tensor<int16_t>({2, 2}, {300, 7, 32767, 1}));
    CHECK(TI.read() == Tensor<int32_t>({2, 2}, {2, 4, 4, 0}));

    std::vector<half> hv;
    for (float f : {1.5f, -2.25f, 0.0f, 1024.0f, 0.5f, -0.125f, 3.0f, 3.0f}) hv.push_back(half(f));
    auto H = Tensor<half>({2, 4}, hv);
    auto sum = reduce_sum(dev(H), {1}).read();
    CHECK(static_cast<float>(sum.values()[0]) == 1023.0f);                // 1023.25 rounds to the even neighbour 1023
    CHECK(static_cast<float>(sum.values()[1]) == 6.375f);
    auto mx = reduce_max(dev(H), {1}).read();
    CHECK(static_cast<float>(mx.values()[0]) == 1024.0f && static_cast<float>(mx.values()[1]) == 3.0f);
    DevTensor<half> HS;
    sort(dev(H), HS, -1);
    auto hs = HS.read();
    CHECK(static_cast<float>(hs.values()[0]) == -2.25f && static_cast<float>(hs.values()[3]) == 1024.0f);
    CHECK(argmax(dev(H), 1, false).read() == Tensor<int>({2}, {3, 2}));
    auto sm = dnn::hardmax(dev(H), 1).read();
    CHECK(static_cast<float>(sm.values()[3]) == 1.0f && static_cast<float>(sm.values()[6]) == 1.0f &&
          static_cast<float>(sm.values()[7]) == 0.0f);
}

// dlf/test/UniformTest.cpp:2060-2063 through the device front-end, plus a complex running sum
static void test_complex() {
    using C = std::complex<float>;
    auto X = Tensor<C>({2}, {C(3, 4), C(5, 12)});
    auto nrm = reduce_nrm2(dev(X), {0}).read();
    CHECK(std::abs(nrm.values()[0] - C(std::sqrt(194.f))) < 1e-5f);
    auto Y = Tensor<C>({2, 3}, {C(1, 1), C(2, -1), C(0, 3), C(-1, 0), C(0, 0), C(4, 4)});
    CHECK(reduce_sum(dev(Y), {1}).read() == Tensor<C>({2}, {C(3, 3), C(3, 4)}));
    CHECK(cumsum(dev(Y), 1).read() == Tensor<C>({2, 3}, {C(1, 1), C(3, 0), C(3, 3), C(-1, 0), C(-1, 0), C(3, 4)}));
    CHECK(count(dev(Y), C(0, 0), {}).read() == Tensor<int>({}, {1}));
}

static void test_errors_and_temporaries() {
    auto X = dev(Tensor<float>({2, 3}).range());
    bool threw = false;
    try { DevTensor<float> Y; reduce("reduce_bogus", X, Y, {1}); } catch (const gpgpu::RuntimeErrorCode& e) { threw = e.status() == DLFX_ERR_UNKNOWN_OP; }
    CHECK(threw);
    threw = false;
    try { argmax(X, 5); } catch (const shape_error&) { threw = true; }
    CHECK(threw);
    threw = false;
    try { reduce_sum(X, {0, 0, 7}); } catch (const shape_error&) { threw = true; }
    CHECK(threw);
    // temporary buffers are a stack: out-of-order release is an error (gpgpu.cpp:208-214)
    auto& ctx = gpgpu::current::context();
    threw = false;
    {
        auto* a = new gpgpu::TemporaryBuffer<float>(ctx.getTemporaryBuffer<float>(100));
        auto* b = new gpgpu::TemporaryBuffer<float>(ctx.getTemporaryBuffer<float>(100));
        try { delete a; } catch (const gpgpu::LogicError&) { threw = true; }
        delete b;
    }
    CHECK(threw);
    // nested temporaries of odd sizes release cleanly in stack order
    threw = false;
    try {
        auto outer = ctx.getTemporaryBuffer<int32_t>(7);
        { auto inner = ctx.getTemporaryBuffer<char>(0); }
        { auto inner = ctx.getTemporaryBuffer<double>(3); auto innermost = ctx.getTemporaryBuffer<char>(5); }
    } catch (const gpgpu::LogicError&) { threw = true; }
    CHECK(!threw);
    // event timing brackets a call
    gpgpu::Event ev;
    auto big = DevTensor<float>(Shape({64, 1 << 16}));
    DevTensor<float> out;
    out.resize(Shape({64}));
    gpgpu::dnn::reduce<float>("reduce_sum", 64, 1 << 16, {64, 1 << 16}, {1 << 16, 1}, big.data(), 0, {64}, {1}, out.data(), 0,
                              gpgpu::current::queue(), &ev);
    CHECK(ev.getElapsedTime() > 0.0f);
}

int main() {
    test_reduce();
    test_arg_reduce();
    test_scan();
    test_sort();
    test_top_k();
    test_count_nonzero();
    test_merge();
    test_softmax_family();
    test_16bit_types();
    test_complex();
    test_errors_and_temporaries();
    std::printf("veneer_test: %d checks, %d failed\n", g_checked, g_failed);
    return g_failed ? 1 : 0;
}
