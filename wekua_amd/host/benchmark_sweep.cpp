// The size sweeps of the reference's benchmark program in the C++ mirror of its API, measured the way it
// measures them (benchmark/gemm.zig:150-283: f32, n = 4 * 2^i for i = 0 .. 11, all four operation pairs, ten
// calls with a fresh alpha and beta each, wall clock from the first enqueue to the end of waitAndCleanup,
// divided by the calls; benchmark/axpy.zig:120-210: f32, n = 4096 * 2^i for i = 0 .. 11, a thousand calls that
// swap x and y, wall clock of the whole batch).  Beside the reference's figure every row gives the host's share:
// the wall clock until the last call has returned, before the wait -- what a call costs the calling thread
// (validation, the choice of a kernel, the launch), which is all that is left of a product of a few rows.
//
// Build (one line): g++ -O2 -std=c++20 -I include -I wekua_amd/host wekua_amd/host/benchmark_sweep.cpp
//                   -L wekua_amd -lwekua_hip -Wl,-rpath,$PWD/wekua_amd -o benchmark_sweep
// Run: ./benchmark_sweep [gemm|axpy|all] [largest exponent i, default 11]
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "wekua.hpp"

namespace {

using namespace wekua;
using Clock = std::chrono::steady_clock;

double us_since(Clock::time_point t0) { return std::chrono::duration<double, std::micro>(Clock::now() - t0).count(); }

struct Timing {
    double per_call_us; // first enqueue .. end of waitAndCleanup, over the calls (the reference's figure)
    double enqueue_us;  // first enqueue .. last call returned, over the calls
};

Timing gemm_case(Context *context, Pipeline *pipeline, uint64_t n, GemmOperation op_a, GemmOperation op_b, std::mt19937 &rng) {
    constexpr int calls = 10;
    std::uniform_real_distribution<float> unit(0.0f, 1.0f);
    std::vector<float> ha(n * n), hb(n * n), hc(n * n);
    for (auto *h : {&ha, &hb, &hc})
        for (float &v : *h) v = unit(rng);
    float alphas[calls], betas[calls];
    for (int i = 0; i < calls; ++i) {
        alphas[i] = unit(rng);
        betas[i] = unit(rng);
    }
    Tensor<float> *a = Tensor<float>::alloc(context, pipeline, {n, n});
    Tensor<float> *b = Tensor<float>::alloc(context, pipeline, {n, n});
    Tensor<float> *c = Tensor<float>::alloc(context, pipeline, {n, n});
    memory::readFromBuffer<float>(pipeline, a, ha.data(), ha.size());
    memory::readFromBuffer<float>(pipeline, b, hb.data(), hb.size());
    memory::readFromBuffer<float>(pipeline, c, hc.data(), hc.size());
    auto *packed = GemmPackedTensors<float>::init(pipeline, c, n, true);
    blas::gemm<float>(pipeline, 1.0f, a, op_a, b, op_b, 0.0f, c, packed); // the reference's warm-up call
    pipeline->waitAndCleanup();

    const auto t0 = Clock::now();
    for (int i = 0; i < calls; ++i) blas::gemm<float>(pipeline, alphas[i], a, op_a, b, op_b, betas[i], c, packed);
    const double enqueued = us_since(t0);
    pipeline->waitAndCleanup();
    const double done = us_since(t0);

    packed->deinit(pipeline);
    a->release(pipeline);
    b->release(pipeline);
    c->release(pipeline);
    return {done / calls, enqueued / calls};
}

Timing axpy_case(Context *context, Pipeline *pipeline, uint64_t n, std::mt19937 &rng) {
    constexpr int calls = 1000;
    std::uniform_real_distribution<float> unit(0.0f, 1.0f);
    std::vector<float> hx(n), hy(n), alphas(calls);
    for (float &v : hx) v = unit(rng);
    for (float &v : hy) v = unit(rng);
    for (float &v : alphas) v = -10.0f + 20.0f * unit(rng);
    Tensor<float> *x = Tensor<float>::alloc(context, pipeline, {n});
    Tensor<float> *y = Tensor<float>::alloc(context, pipeline, {n});
    blas::axpy<float>(pipeline, x, 0.0f, y); // the reference's warm-up call
    memory::readFromBuffer<float>(pipeline, x, hx.data(), hx.size());
    memory::readFromBuffer<float>(pipeline, y, hy.data(), hy.size());
    pipeline->waitAndCleanup();

    const auto t0 = Clock::now();
    for (int i = 0; i < calls; ++i) {
        if (i % 2 == 0) blas::axpy<float>(pipeline, x, alphas[i], y);
        else blas::axpy<float>(pipeline, y, alphas[i], x);
    }
    const double enqueued = us_since(t0);
    pipeline->waitAndCleanup();
    const double done = us_since(t0);

    x->release(pipeline);
    y->release(pipeline);
    return {done / calls, enqueued / calls};
}

} // namespace

int main(int argc, char **argv) {
    const char *what = argc > 1 ? argv[1] : "all";
    const int last = argc > 2 ? std::atoi(argv[2]) : 11;
    if (last < 0 || last > 11) {
        std::fprintf(stderr, "largest exponent: 0 .. 11\n");
        return 2;
    }
    try {
        Context *context = Context::initFromDeviceType(core::DeviceType::all);
        Pipeline *pipeline = Pipeline::init(&context->command_queues[0]);
        std::mt19937 rng(2024);
        if (!std::strcmp(what, "gemm") || !std::strcmp(what, "all")) {
            static const struct { const char *name; GemmOperation a, b; } ops[] = {
                {"NN", GemmOperation::no_transpose, GemmOperation::no_transpose},
                {"NT", GemmOperation::no_transpose, GemmOperation::transpose},
                {"TN", GemmOperation::transpose, GemmOperation::no_transpose},
                {"TT", GemmOperation::transpose, GemmOperation::transpose}};
            std::printf("GEMM f32, 10 calls per point: us per call (first enqueue .. end of wait) / us per call until enqueued; TFLOP/s of N,N\n");
            std::printf("%6s %21s %21s %21s %21s %9s\n", "n", "NN", "NT", "TN", "TT", "TFLOP/s");
            for (int i = 0; i <= last; ++i) {
                const uint64_t n = 4ull << i;
                std::printf("%6llu", (unsigned long long)n);
                double nn = 0.0;
                for (const auto &op : ops) {
                    const Timing t = gemm_case(context, pipeline, n, op.a, op.b, rng);
                    if (&op == &ops[0]) nn = t.per_call_us;
                    std::printf(" %11.2f / %7.2f", t.per_call_us, t.enqueue_us);
                }
                std::printf(" %9.3f\n", 2.0 * n * n * n / nn / 1e6);
                std::fflush(stdout);
            }
        }
        if (!std::strcmp(what, "axpy") || !std::strcmp(what, "all")) {
            std::printf("AXPY f32, 1000 calls per point: us per call (first enqueue .. end of wait) / us per call until enqueued; GB/s\n");
            for (int i = 0; i <= last; ++i) {
                const uint64_t n = 4096ull << i;
                const Timing t = axpy_case(context, pipeline, n, rng);
                std::printf("%9llu %11.2f / %7.2f %9.1f\n", (unsigned long long)n, t.per_call_us, t.enqueue_us,
                            3.0 * n * sizeof(float) / t.per_call_us / 1e3);
                std::fflush(stdout);
            }
        }
        pipeline->deinit();
        context->deinit();
    } catch (const Error &e) {
        std::fprintf(stderr, "wekua error %d: %s\n", e.code, e.what());
        return 1;
    }
    return 0;
}
