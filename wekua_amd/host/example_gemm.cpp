// The reference's benchmark/gemm.zig:170-200 in the C++ mirror of its API: allocate three tensors,
// upload, make a GemmPackedTensors, run blas::gemm, read C back, and time a few calls.
//
// Build (one line): g++ -O2 -std=c++20 -I include -I wekua_amd/host wekua_amd/host/example_gemm.cpp
//                   -L wekua_amd -lwekua_hip -Wl,-rpath,$PWD/wekua_amd -o example_gemm
// Run: ./example_gemm 2048
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "wekua.hpp"

int main(int argc, char **argv) {
    using namespace wekua;
    using T = float;
    const uint64_t size = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 1024;
    try {
        Context *context = Context::initFromDeviceType(core::DeviceType::all);
        Pipeline *pipeline = Pipeline::init(&context->command_queues[0]);

        std::mt19937 rng(42);
        std::uniform_real_distribution<T> dist(-1, 1);
        std::vector<T> buf1(size * size), buf2(size * size), buf3(size * size);
        for (auto *b : {&buf1, &buf2, &buf3})
            for (T &v : *b) v = dist(rng);

        Tensor<T> *a = Tensor<T>::alloc(context, pipeline, {size, size});
        Tensor<T> *b = Tensor<T>::alloc(context, pipeline, {size, size});
        Tensor<T> *c = Tensor<T>::alloc(context, pipeline, {size, size});
        memory::readFromBuffer<T>(pipeline, a, buf1.data(), buf1.size());
        memory::readFromBuffer<T>(pipeline, b, buf2.data(), buf2.size());
        memory::readFromBuffer<T>(pipeline, c, buf3.data(), buf3.size());

        auto *packed_tensors = GemmPackedTensors<T>::init(pipeline, c, size, true);

        blas::gemm<T>(pipeline, 1.0f, a, GemmOperation::no_transpose, b, GemmOperation::no_transpose, 0.0f, c, packed_tensors);
        pipeline->waitAndCleanup();

        const int calls = 10;
        const auto start = std::chrono::steady_clock::now();
        for (int i = 0; i < calls; ++i)
            blas::gemm<T>(pipeline, 1.5f, a, GemmOperation::no_transpose, b, GemmOperation::transpose, 0.5f, c, packed_tensors);
        pipeline->waitAndCleanup();
        const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - start).count() / calls;

        memory::writeToBuffer<T>(pipeline, c, buf3.data(), buf3.size());
        pipeline->waitAndCleanup();
        std::printf("gemm f32 %llu^3: %.3f ms per call, %.1f TFLOP/s, c[0][0] = %g\n", (unsigned long long)size, ms,
                    2.0 * size * size * size / ms / 1e9, (double)buf3[0]);

        packed_tensors->deinit(pipeline);
        a->release(pipeline);
        b->release(pipeline);
        c->release(pipeline);
        pipeline->deinit();
        context->deinit();
    } catch (const Error &e) {
        std::fprintf(stderr, "wekua error %d: %s\n", e.code, e.what());
        return 1;
    }
    return 0;
}
