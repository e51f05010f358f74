// The reference's own benchmark loop (Tensor.Benchmark/Benchmark.fs:95-317: one operation + device synchronisation per
// measurement, result allocation included, host clock) through the compiled C++ host layer, for the operations of the hot path.
// Prints the reference's CSV columns: Method,Shape,Type,Dev,Mean [ms],StdDev [ms].
//
//   bench_suite [iters] [warmup]          defaults 30 and 5; shapes 1000x1000, 2000x2000, 4000x4000 (Benchmark.fs:216)
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <random>
#include <string>
#include <vector>

#include "hip_tensor.hpp"

namespace T = Tensor;

template <class X> const char* type_name();
template <> const char* type_name<float>() { return "single"; }
template <> const char* type_name<double>() { return "double"; }
template <> const char* type_name<int32_t>() { return "int32"; }

static void sync() { T::check(dnh_stream_sync(T::Cfg::Stream())); }

static void measure(const char* method, int64_t n, const char* type, int iters, int warmup, const std::function<void()>& op) {
    for (int i = 0; i < warmup; i++) { op(); sync(); }
    std::vector<double> ms(iters);
    for (int i = 0; i < iters; i++) {
        const auto t0 = std::chrono::steady_clock::now();
        op();
        sync();
        ms[i] = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    }
    double mean = 0, var = 0;
    for (double v : ms) mean += v;
    mean /= iters;
    for (double v : ms) var += (v - mean) * (v - mean);
    std::printf("%s,%lldx%lld,%s,Hip,%.4f,%.4f\n", method, (long long)n, (long long)n, type, mean, std::sqrt(var / (iters > 1 ? iters - 1 : 1)));
    std::fflush(stdout);
}

template <class X>
static void run_type(int64_t n, int iters, int warmup) {
    std::mt19937 rng(123);
    std::vector<X> ha((size_t)(n * n)), hb((size_t)(n * n));
    for (auto& v : ha) v = (X)((int)(rng() % 2001) - 1000) / (X)(std::is_floating_point<X>::value ? 500 : 1);
    for (auto& v : hb) v = (X)((int)(rng() % 2001) - 1000) / (X)(std::is_floating_point<X>::value ? 500 : 1) + (X)3;
    const auto a = T::Tensor<X>::ofHost(ha, {n, n});
    const auto b = T::Tensor<X>::ofHost(hb, {n, n});
    const auto mask = a > b;
    const char* ty = type_name<X>();
    measure("Zeros", n, ty, iters, warmup, [&] { auto c = T::Tensor<X>::zeros({n, n}); });
    measure("Add", n, ty, iters, warmup, [&] { auto c = a + b; });
    measure("Multiply", n, ty, iters, warmup, [&] { auto c = a * b; });
    measure("Negate", n, ty, iters, warmup, [&] { auto c = -a; });
    measure("Greater", n, ty, iters, warmup, [&] { auto c = a > b; });
    measure("IfThenElse", n, ty, iters, warmup, [&] { auto c = T::Tensor<X>::ifThenElse(mask, a, b); });
    measure("SumAxis", n, ty, iters, warmup, [&] { auto c = a.sumAxis(1); });
    measure("MaxAxis", n, ty, iters, warmup, [&] { auto c = a.maxAxis(1); });
    measure("ArgMaxAxis", n, ty, iters, warmup, [&] { auto c = a.argMaxAxis(1); });
    measure("SumAxis0", n, ty, iters, warmup, [&] { auto c = a.sumAxis(0); });
    measure("MaskedGet", n, ty, iters, warmup, [&] { auto c = a.M(mask); });
    if constexpr (std::is_floating_point<X>::value) {
        measure("Tanh", n, ty, iters, warmup, [&] { auto c = a.tanh(); });
        measure("Exp", n, ty, iters, warmup, [&] { auto c = a.exp(); });
        measure("Dot", n, ty, iters, warmup, [&] { auto c = a.dot(b); });
        if (n <= 2000) measure("Invert", n, ty, iters < 5 ? iters : 5, 1, [&] { auto c = T::Tensor<X>::invert(b); });
    }
}

int main(int argc, char** argv) {
    const int iters = argc > 1 ? std::atoi(argv[1]) : 30, warmup = argc > 2 ? std::atoi(argv[2]) : 5;
    try {
        T::check(dnh_init(0));
        std::printf("Method,Shape,Type,Dev,Mean [ms],StdDev [ms]\n");
        for (int64_t n : {1000, 2000, 4000}) {
            run_type<float>(n, iters, warmup);
            run_type<double>(n, iters, warmup);
            run_type<int32_t>(n, iters, warmup);
        }
    } catch (const std::exception& e) {
        std::fprintf(stderr, "bench_suite: %s\n", e.what());
        return 1;
    }
    return 0;
}
