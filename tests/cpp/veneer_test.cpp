// Runs the C++ host veneer (dlf-style DevTensor front-ends over gpgpu::dnn over
// the C ABI) against the literal vectors the reference's own tests hold, plus
// the veneer's error and temporary-buffer behaviour.  Needs a GPU.  Exit code 0
// when every check passes; failures are listed on stderr.
//
// Vectors: dlf/test/UniformTest.cpp:1857-1965 (reduce), :2106-2189 (scan),
// :2304-2377 (sort), dlf/test/DNNTest.cpp:861-1019 (argmax/argmin),
// dlf/test/model/PredictTest.cpp:609-637 (top_k), dlf/test/UniformTest.cpp:2065-2080
// (count), :2553-2561 (nonzero), :2250-2283 (merge), dlf/test/DNNTest.cpp:796-858
// (softmax, logsoftmax, hardmax), dlf/test/model/PredictTest.cpp:290-319 (Reduce nodes),
// :609-637 (TopK node).
#include <algorithm>
#include <cmath>
#include <complex>
#include <cstdio>
#include <future>
#include <random>

#include "dev_tensor.h"
#include "onnx_nodes.h"

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

// Scratch comes from the context of the queue a routine is given (xreduce.cpp:78, xscan.cpp:82),
// not from the calling thread's: a call on another queue leaves this thread's arena alone.
static void test_queue_contexts() {
    const gpgpu::Queue& mine = gpgpu::current::queue();
    CHECK(mine.context() == gpgpu::current::context());
    gpgpu::Queue other;                                   // a context and arena of its own
    CHECK(other.context() != mine.context());
    gpgpu::Queue sibling = mine.context().createQueue(); // shares this thread's context, as in the reference
    CHECK(sibling.context() == mine.context() && sibling != mine);

    // a live temporary of this thread's context with known contents
    const size_t words = 1 << 16;
    auto held = mine.context().getTemporaryBuffer<int32_t>(words);
    std::vector<int32_t> pattern(words);
    for (size_t i = 0; i < words; ++i) pattern[i] = static_cast<int32_t>(i * 2654435761u);
    held.write(mine, pattern.data(), words, held.offset());

    // long rows on the other queue: both routines need scratch (partials, tile states)
    const size_t m = 3, n = 1 << 20;
    std::vector<int32_t> xs(m * n);
    std::mt19937 rng(11);
    for (auto& v : xs) v = static_cast<int32_t>(rng() % 100);
    auto X = dev(Tensor<int32_t>({m, n}, xs));
    DevTensor<int32_t> S(Shape({m})), C(Shape({m, n}));
    const size_t in_use = mine.context().temporary_bytes_in_use();
    gpgpu::dnn::reduce<int32_t>("reduce_sum", m, n, {m, n}, {n, 1}, X.data(), 0, {m}, {1}, S.data(), 0, other);
    gpgpu::dnn::scan<int32_t>("cumsum", m, n, false, {m, n}, X.data(), 0, {n, 1}, C.data(), 0, {n, 1}, other);
    other.finish();
    CHECK(mine.context().temporary_bytes_in_use() == in_use);
    CHECK(other.context().temporary_bytes_in_use() == 0);
    auto sums = S.read(), scan = C.read();
    bool ok = true;
    for (size_t r = 0; r < m; ++r) {
        int32_t acc = 0;
        for (size_t j = 0; j < n; ++j) {
            acc += xs[r * n + j];
            ok = ok && scan.values()[r * n + j] == acc;
        }
        ok = ok && sums.values()[r] == acc;
    }
    CHECK(ok);
    std::vector<int32_t> back(words);
    held.read(mine, back.data(), words, held.offset());
    CHECK(back == pattern);
}

// A live temporary survives a softmax that needs scratch of its own from the same arena
// (few rows, too long for one workgroup's registers).
static void test_softmax_scratch_is_its_own_slice() {
    const gpgpu::Queue& q = gpgpu::current::queue();
    const size_t words = 1 << 14;
    auto held = q.context().getTemporaryBuffer<float>(words);
    std::vector<float> pattern(words);
    for (size_t i = 0; i < words; ++i) pattern[i] = static_cast<float>(i) * 0.5f - 7.0f;
    held.write(q, pattern.data(), words, held.offset());
    const size_t m = 4, n = 1 << 20;
    CHECK(dlfx_softmax_scratch_bytes(DLFX_F32, m, n) > 0);
    std::vector<float> xs(m * n);
    std::mt19937 rng(12);
    for (auto& v : xs) v = static_cast<float>(rng() % 2000) * 0.001f;
    auto X = dev(Tensor<float>({m, n}, xs));
    auto Y = dnn::softmax(X, 1).read();
    bool ok = true;
    for (size_t r = 0; r < m; ++r) {
        double sum = 0;
        for (size_t j = 0; j < n; ++j) sum += Y.values()[r * n + j];
        ok = ok && std::fabs(sum - 1.0) < 1e-4;
    }
    CHECK(ok);
    std::vector<float> back(words);
    held.read(q, back.data(), words, held.offset());
    CHECK(back == pattern);
}

// Out-of-place and strided row normalisation, extent-1 sort / argsort: no host round trip.
static void test_layout_steps_stay_on_the_device() {
    auto host = Tensor<float>({2, 3}, {-1, 0, 1, 2, 4, 8});
    auto X = dev(host);
    DevTensor<float> Y;
    size_t& reads = gpgpu::detail::device_to_host_reads();
    const size_t before = reads;
    dnn::softmax(X, Y, 1);                                   // dense input, out of place
    DevTensor<float> Z;
    dnn::logsoftmax(X.transpose(), Z, 1);                    // strided view: device copy, then in place
    DevTensor<float> S;
    auto col = dev(Tensor<float>({4, 1}, {3, 1, 2, 0}));
    sort(col, S, 1);                                         // extent 1: a copy
    DevTensor<float> AV;
    DevTensor<int32_t> AI;
    argsort(col.transpose(), AV, AI, 0);                     // [1, 4] along axis 0: copy + zero indices
    CHECK(reads == before);
    CHECK(near(Y.read(), Tensor<float>({2, 3}, {0.09003057f, 0.24472848f, 0.66524094f, 0.00242826f, 0.01794253f, 0.97962922f})));
    // rows of the transposed view are (-1, 2), (0, 4), (1, 8)
    auto z = Z.read();
    CHECK(z.shape() == Shape({3, 2}));
    CHECK(std::fabs(z.values()[0] - (-3.0485873f)) < 1e-4 && std::fabs(z.values()[1] - (-0.0485873f)) < 1e-4);
    CHECK(std::fabs(z.values()[5] - (-0.00091147f)) < 1e-5);
    CHECK(X.read() == host);                                 // the input is untouched
    CHECK(S.read() == Tensor<float>({4, 1}, {3, 1, 2, 0}));
    CHECK(AV.read() == Tensor<float>({1, 4}, {3, 1, 2, 0}));
    CHECK(AI.read() == Tensor<int32_t>({1, 4}, {0, 0, 0, 0}));
    // reorder of a flipped, sliced view
    auto R = dev(Tensor<int32_t>({3, 4}).range());
    DevTensor<int32_t> RR;
    reorder(flip(R, 1).slice(0, 1, 3), RR);
    CHECK(RR.read() == Tensor<int32_t>({2, 4}, {7, 6, 5, 4, 11, 10, 9, 8}));
    // the flat copy repeats a shorter source (xcopy.cl:8-26); fill writes a strided view
    auto src = dev(Tensor<int32_t>({3}, {1, 2, 3}));
    DevTensor<int32_t> dst(Shape({8}));
    gpgpu::dnn::copy<int32_t>(3, src.data(), 0, 8, dst.data(), 0);
    CHECK(dst.read() == Tensor<int32_t>({8}, {1, 2, 3, 1, 2, 3, 1, 2}));
    gpgpu::dnn::fill<int32_t>(4, {4}, {2}, dst.data(), 1, -5);
    CHECK(dst.read() == Tensor<int32_t>({8}, {1, -5, 3, -5, 2, -5, 1, -5}));
}

// ONNX nodes as the interpreter binds them (predict.h:1078-1201, 1486-1510, 2031-2044):
// attribute defaults, output shapes and order.
static void test_logits_head() {
    // one launch against the five front-end calls on the same logits
    std::mt19937 rng(11);
    std::vector<float> v(40 * 1000);
    for (auto& e : v) e = static_cast<float>(static_cast<int>(rng() % 2001) - 1000) / 64.0f;      // many equal values
    auto X = dev(Tensor<float>({40, 1000}, v));
    DevTensor<float> S({40}), M({40}), L({40}), BV({40, 5});
    DevTensor<int> A({40}), BI({40, 5});
    gpgpu::dnn::logits_head(40, 1000, X.data(), 0, 1000, &S.data(), &M.data(), &A.data(), &L.data(), 5, &BV.data(), &BI.data());
    CHECK(M.read() == reduce_max(X, {1}).read());
    CHECK(A.read() == argmax(X, 1, false).read());
    CHECK(near(S.read(), reduce_sum(X, {1}).read()));
    CHECK(near(L.read(), reduce_log_sum_exp(X, {1}).read()));
    auto r = top_k(X, 5);
    CHECK(BV.read() == r.first.read());
    CHECK(BI.read() == r.second.read());
}

static void test_onnx_nodes() {
    using namespace dlf::predict;
    // PredictTest.cpp:290-319
    auto X = dev(Tensor<float>({3, 2, 2}).range(1));
    DevTensor<float> A, B, C;
    Node<float> n;
    n.op_type = "ReduceSum";
    n.inputs = {&X};
    n.outputs = {&A};
    evaluate(n);                                                        // every axis, keepdims 1
    CHECK(A.read() == Tensor<float>({1, 1, 1}, {78}));
    n.attrs.set_is("axes", {1});
    n.outputs = {&B};
    evaluate(n);
    CHECK(B.read() == Tensor<float>({3, 1, 2}, {4, 6, 12, 14, 20, 22}));
    n.attrs.set_i("keepdims", 0);
    n.outputs = {&C};
    evaluate(n);
    CHECK(C.read() == Tensor<float>({3, 2}, {4, 6, 12, 14, 20, 22}));
    // every reduction node kind against a host loop over axis -1
    const char* kinds[] = {"ReduceMax", "ReduceMin", "ReduceSum", "ReduceSumSquare", "ReduceMean", "ReduceProd",
                           "ReduceLogSum", "ReduceLogSumExp", "ReduceL1", "ReduceL2"};
    auto P = Tensor<float>({2, 3}, {1.5f, 0.5f, 2.0f, 3.0f, 0.25f, 1.0f});
    auto dP = dev(P);
    for (const char* kind : kinds) {
        Node<float> r;
        DevTensor<float> out;
        r.op_type = kind;
        r.inputs = {&dP};
        r.outputs = {&out};
        r.attrs.set_is("axes", {-1}).set_i("keepdims", 0);
        evaluate(r);
        std::vector<float> want;
        for (int row = 0; row < 2; ++row) {
            const float* v = P.data() + row * 3;
            const std::string k = kind;
            double acc = (k == "ReduceProd") ? 1 : 0, mx = v[0], mn = v[0];
            for (int j = 0; j < 3; ++j) {
                mx = std::max<double>(mx, v[j]);
                mn = std::min<double>(mn, v[j]);
                if (k == "ReduceProd") acc *= v[j];
                else if (k == "ReduceSumSquare" || k == "ReduceL2") acc += double(v[j]) * v[j];
                else if (k == "ReduceLogSumExp") acc += std::exp(double(v[j]));
                else if (k == "ReduceL1") acc += std::fabs(v[j]);
                else acc += v[j];
            }
            if (k == "ReduceMax") acc = mx;
            if (k == "ReduceMin") acc = mn;
            if (k == "ReduceMean") acc /= 3;
            if (k == "ReduceLogSum" || k == "ReduceLogSumExp") acc = std::log(acc);
            if (k == "ReduceL2") acc = std::sqrt(acc);
            want.push_back(static_cast<float>(acc));
        }
        CHECK(near(out.read(), Tensor<float>({2}, want), 1e-5));
    }

    // ArgMax / ArgMin: axis 0 and keepdims 1 by default (DNNTest.cpp:861-1019 vectors)
    auto M = dev(Tensor<float>({2, 3, 4}, {21, 22, 2, 15, 16, 7, 14, 0, 18, 20, 6, 9, 23, 4, 12, 11, 10, 5, 3, 8, 17, 19, 13, 1}));
    DevTensor<int32_t> I;
    Node<float> am;
    am.op_type = "ArgMax";
    am.inputs = {&M};
    am.index_outputs = {&I};
    evaluate(am);
    CHECK(I.read() == Tensor<int32_t>({1, 3, 4}, {1, 0, 1, 0, 0, 0, 0, 1, 0, 0, 1, 0}));
    am.attrs.set_i("axis", 2).set_i("keepdims", 0);
    evaluate(am);
    CHECK(I.read() == Tensor<int32_t>({2, 3}, {1, 0, 1, 0, 0, 1}));
    am.op_type = "ArgMin";
    am.attrs.set_i("axis", 1).set_i("keepdims", 1);
    evaluate(am);
    CHECK(I.read() == Tensor<int32_t>({2, 1, 4}, {1, 1, 0, 1, 1, 0, 1, 2}));

    // CumSum: the axis is a tensor read on the host; exclusive / reverse default to 0; in place
    auto S = dev(Tensor<int32_t>({2, 3}, {1, 2, 3, 4, 5, 6}));
    Tensor<int64_t> axis({}, {1});
    DevTensor<int32_t> CS;
    Node<int32_t> cs;
    cs.op_type = "CumSum";
    cs.inputs = {&S};
    cs.host_inputs = {&axis};
    cs.outputs = {&CS};
    evaluate(cs);
    CHECK(CS.read() == Tensor<int32_t>({2, 3}, {1, 3, 6, 4, 9, 15}));
    cs.attrs.set_i("exclusive", 1).set_i("reverse", 1);
    evaluate(cs);
    CHECK(CS.read() == Tensor<int32_t>({2, 3}, {5, 3, 0, 11, 6, 0}));
    cs.attrs = Attributes();
    cs.outputs = {&S};                                                  // allocInplace: output is the input
    evaluate(cs);
    CHECK(S.read() == Tensor<int32_t>({2, 3}, {1, 3, 6, 4, 9, 15}));

    // TopK (PredictTest.cpp:609-637): K is an int64 tensor; axis -1, largest 1 by default
    auto T = dev(Tensor<float>({3, 4}, {0, 1, 2, 3, 7, 6, 5, 4, 10, 11, 9, 8}));
    Tensor<int64_t> K({1}, {3});
    DevTensor<float> TV;
    DevTensor<int32_t> TI;
    Node<float> tk;
    tk.op_type = "TopK";
    tk.inputs = {&T};
    tk.host_inputs = {&K};
    tk.outputs = {&TV};
    tk.index_outputs = {&TI};
    evaluate(tk);
    CHECK(TV.read() == Tensor<float>({3, 3}, {3, 2, 1, 7, 6, 5, 11, 10, 9}));
    CHECK(TI.read() == Tensor<int32_t>({3, 3}, {3, 2, 1, 0, 1, 2, 1, 0, 2}));
    tk.attrs.set_i("axis", 0).set_i("largest", 0);
    Tensor<int64_t> K1({1}, {1});
    tk.host_inputs = {&K1};
    evaluate(tk);
    CHECK(TV.read() == Tensor<float>({1, 4}, {0, 1, 2, 3}));
    CHECK(TI.read() == Tensor<int32_t>({1, 4}, {0, 0, 0, 0}));

    // NonZero: [rank, n] (UniformTest.cpp:2553-2561 layout)
    auto Z = dev(Tensor<float>({2, 3}, {1, 0, 0, 0, 2, 3}));
    DevTensor<int32_t> NZ;
    Node<float> nz;
    nz.op_type = "NonZero";
    nz.inputs = {&Z};
    nz.index_outputs = {&NZ};
    evaluate(nz);
    CHECK(NZ.read() == Tensor<int32_t>({2, 3}, {0, 1, 1, 0, 1, 2}));

    // Softmax family: axis 1 by default; rows are everything from the axis on
    auto L = dev(Tensor<float>({2, 3}, {-1, 0, 1, 2, 4, 8}));
    DevTensor<float> SO;
    Node<float> sm;
    sm.op_type = "Softmax";
    sm.inputs = {&L};
    sm.outputs = {&SO};
    evaluate(sm);
    CHECK(near(SO.read(), Tensor<float>({2, 3}, {0.09003057f, 0.24472848f, 0.66524094f, 0.00242826f, 0.01794253f, 0.97962922f})));
    sm.op_type = "Hardmax";
    sm.attrs.set_i("axis", 0);                                          // one row of six
    evaluate(sm);
    CHECK(SO.read() == Tensor<float>({2, 3}, {0, 0, 0, 0, 0, 1}));
    sm.op_type = "LogSoftmax";
    sm.attrs.set_i("axis", 1);
    auto op = make_operator(sm);                                        // bound once, run twice
    op->evaluate();
    op->evaluate();
    CHECK(std::fabs(SO.read().values()[2] - std::log(0.66524094f)) < 1e-5);

    bool threw = false;
    Node<float> conv;
    conv.op_type = "Conv";
    conv.inputs = {&L};
    conv.outputs = {&SO};
    try { evaluate(conv); } catch (const unsupported_operator&) { threw = true; }
    CHECK(threw);
    threw = false;
    Node<float> bad;
    bad.op_type = "TopK";
    bad.inputs = {&T};
    try { evaluate(bad); } catch (const std::invalid_argument&) { threw = true; }
    CHECK(threw);
}

// Two host threads, each on the queue and context its first use creates for it
// (dlf/test/GPGPUTest.cpp:716-733; gpgpu/src/gpgpu.cpp:139-185): a long-row reduction, a chained
// scan and an argsort of long rows per thread, all three with scratch from the thread's own
// arena, running at the same time; results equal the single-thread ones.
struct ThreadResult {
    Tensor<int32_t> sums, scan, order;
    bool own_queue = false;
    size_t left_in_use = 1;
};
static ThreadResult thread_work(const std::vector<int32_t>& xs, size_t m, size_t n, const gpgpu::Queue* main_queue) {
    ThreadResult r;
    const gpgpu::Queue& mine = gpgpu::current::queue();
    r.own_queue = main_queue == nullptr || (mine != *main_queue && mine.context() != main_queue->context());
    auto X = dev(Tensor<int32_t>({m, n}, xs));
    for (int round = 0; round < 3; ++round) {            // several rounds so that the threads' launches interleave
        r.sums = reduce_sum(X, {1}).read();
        r.scan = cumsum(X, 1).read();
        r.order = argsort(X, 1).read();
    }
    mine.finish();
    r.left_in_use = mine.context().temporary_bytes_in_use();
    return r;
}
static void test_two_threads() {
    const size_t m = 4, n = 300000;
    std::vector<int32_t> a(m * n), b(m * n);
    std::mt19937 rng(23);
    for (auto& v : a) v = static_cast<int32_t>(rng() % 1000);
    for (auto& v : b) v = static_cast<int32_t>(rng() % 50) - 25;
    const gpgpu::Queue& main_queue = gpgpu::current::queue();
    const ThreadResult alone_a = thread_work(a, m, n, nullptr), alone_b = thread_work(b, m, n, nullptr);
    auto fa = std::async(std::launch::async, thread_work, std::cref(a), m, n, &main_queue);
    auto fb = std::async(std::launch::async, thread_work, std::cref(b), m, n, &main_queue);
    const ThreadResult ta = fa.get(), tb = fb.get();
    CHECK(ta.own_queue && tb.own_queue);
    CHECK(ta.left_in_use == 0 && tb.left_in_use == 0);
    CHECK(ta.sums == alone_a.sums && ta.scan == alone_a.scan && ta.order == alone_a.order);
    CHECK(tb.sums == alone_b.sums && tb.scan == alone_b.scan && tb.order == alone_b.order);
    // ... and the single-thread results are right: serial host scan, stable order
    bool ok = true;
    for (size_t r = 0; r < m; ++r) {
        int32_t acc = 0;
        for (size_t j = 0; j < n; ++j) {
            acc += a[r * n + j];
            ok = ok && alone_a.scan.values()[r * n + j] == acc;
        }
        ok = ok && alone_a.sums.values()[r] == acc;
        for (size_t j = 1; j < n; ++j) {
            const int32_t p = alone_a.order.values()[r * n + j - 1], q = alone_a.order.values()[r * n + j];
            ok = ok && (a[r * n + p] < a[r * n + q] || (a[r * n + p] == a[r * n + q] && p < q));
        }
    }
    CHECK(ok);
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
    test_queue_contexts();
    test_softmax_scratch_is_its_own_slice();
    test_layout_steps_stay_on_the_device();
    test_onnx_nodes();
    test_logits_head();
    test_two_threads();
    std::printf("veneer_test: %d checks, %d failed\n", g_checked, g_failed);
    return g_failed ? 1 : 0;
}
