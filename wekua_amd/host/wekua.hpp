// wekua.hpp -- host-side mirror of wekua's public API for the BLAS hot path, on top of the
// C ABI of libwekua_hip (include/wekua_hip.h).
//
// The reference's host layer is Zig generics over OpenCL.  No Zig toolchain is available to
// this build, so the same surface is written as C++ templates with the reference's names,
// parameter order and error behaviour, one for one:
//
//   wekua::core::Context        src/core/context.zig:13-196
//   wekua::core::CommandQueue   src/core/command_queue.zig:10-229
//   wekua::core::Pipeline       src/core/pipeline.zig:6-66
//   wekua::core::types          src/core/types.zig:1-115
//   wekua::Tensor<T>            src/tensor/main.zig:62-279
//   wekua::memory::*            src/tensor/memory/{read_from_buffer,write_to_buffer}.zig
//   wekua::fill::*, identity    src/tensor/fill.zig:16-95, identity.zig:16-70
//   wekua::blas::axpy           src/blas/axpy.zig:93-169
//   wekua::blas::gemm           src/blas/gemm.zig:834-874 (validateTensors :442-485)
//   wekua::blas::PackedTensors  src/blas/gemm.zig:60-359
//
// Zig error unions become exceptions of type wekua::Error carrying the WK_E_* code whose
// name is the Zig error name; Zig optionals (`?T`) become std::optional<T>.
//
// What differs on purpose (MI355X-first):
//   * a Context owns one HIP device; its single CommandQueue is an in-order HIP stream;
//   * a Pipeline orders work by the stream, so its "events" are tickets kept only for the
//     prevEvents()/append() bookkeeping callers rely on; waitAndCleanup() syncs the stream;
//   * Tensor rows are padded to 16 bytes (the per-lane load width of gfx950), not to an
//     even vector count, row counts are not padded at all, and row pitches that are a
//     multiple of 1 KiB and at least 16 KiB are skewed by 512 bytes to avoid channel aliasing;
//   * PackedTensors holds device memory only for the 8/16/32-bit integers (the signed-digit planes of
//     the int8 matrix-core product), for cf32 / cf64 and for the complex 8/16/32-bit integers
//     (operands rebuilt as real matrices), all filled by pack passes inside gemm; for every other type the
//     HIP kernels tile straight from the row-major operands through LDS and pack() only validates.
#pragma once

#include <algorithm>
#include <charconv>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <exception>
#include <limits>
#include <atomic>
#include <optional>
#include <string>
#include <type_traits>
#include <vector>

#include "wekua_hip.h"

namespace wekua {

struct Error : std::exception {
    int code;
    explicit Error(int c) : code(c) {}
    const char *what() const noexcept override { return wk_strerror(code); }
};

inline void check(int code) {
    if (code != WK_OK) throw Error(code);
}

namespace core {

// ---- types (src/core/types.zig) ----------------------------------------------------------
template <typename R> struct Complex {
    R real, imag;
};

template <typename T> struct is_complex : std::false_type {};
template <typename R> struct is_complex<Complex<R>> : std::true_type {};
template <typename T> struct scalar_of { using type = T; };
template <typename R> struct scalar_of<Complex<R>> { using type = R; };

template <typename T> constexpr bool isComplex() { return is_complex<T>::value; }
enum class Space : uint8_t { real = 0, imag = 1 }; // src/core/types.zig:1-4

// getTypeId: 0..9 over the scalar type (types.zig:88-104)
template <typename T> constexpr int getTypeId() {
    using R = typename scalar_of<T>::type;
    if constexpr (std::is_same_v<R, int8_t>) return 0;
    else if constexpr (std::is_same_v<R, uint8_t>) return 1;
    else if constexpr (std::is_same_v<R, int16_t>) return 2;
    else if constexpr (std::is_same_v<R, uint16_t>) return 3;
    else if constexpr (std::is_same_v<R, int32_t>) return 4;
    else if constexpr (std::is_same_v<R, uint32_t>) return 5;
    else if constexpr (std::is_same_v<R, int64_t>) return 6;
    else if constexpr (std::is_same_v<R, uint64_t>) return 7;
    else if constexpr (std::is_same_v<R, float>) return 8;
    else if constexpr (std::is_same_v<R, double>) return 9;
    else static_assert(sizeof(R) == 0, "Type not supported");
}
// getTypeIndex: 0..19 (types.zig:60-86); also the dtype id of the C ABI
template <typename T> constexpr int getTypeIndex() { return getTypeId<T>() + (isComplex<T>() ? 10 : 0); }

template <typename T> constexpr T getOne() {
    if constexpr (isComplex<T>()) return T{1, 0};
    else return T(1);
}

// ---- CommandQueue / Context ------------------------------------------------------------------
struct Context;

enum class DeviceType { cpu, gpu, all };
enum class LocalMemType { local, global };

struct CommandQueue {
    const Context *context = nullptr;
    wk_stream *stream = nullptr;
    uint32_t wekua_id = 0;
    std::string device_name;
    LocalMemType local_mem_type = LocalMemType::local;
    uint64_t local_mem_size = 0;
    uint32_t compute_units = 0;
    uint64_t max_work_group_size = 0;
    uint32_t cache_line_size = 0;
    // elements per 16-byte lane access for the 10 scalar types (command_queue.zig:81-98 keeps the
    // OpenCL native widths here)
    uint32_t vector_widths[10] = {16, 16, 8, 8, 4, 4, 2, 2, 4, 2};

    template <typename T> bool isTypeSupported() const { return true; }
};

struct Context {
    wk_device *device = nullptr;
    std::vector<CommandQueue> command_queues;

    // Context.init with an explicit device ordinal
    static Context *init(int ordinal) {
        Context *ctx = new Context;
        int rc = wk_device_open(ordinal, &ctx->device);
        if (rc) {
            delete ctx;
            throw Error(rc);
        }
        ctx->command_queues.resize(1);
        CommandQueue &q = ctx->command_queues[0];
        q.context = ctx;
        rc = wk_stream_create(ctx->device, &q.stream);
        if (rc) {
            wk_device_close(ctx->device);
            delete ctx;
            throw Error(rc);
        }
        wk_props props;
        wk_device_props(ctx->device, &props);
        q.device_name = std::string(props.name) + " " + props.arch;
        q.local_mem_size = props.local_mem_bytes;
        q.compute_units = (uint32_t)props.compute_units;
        q.max_work_group_size = (uint64_t)props.max_work_group_size;
        q.cache_line_size = (uint32_t)props.cache_line_size;
        return ctx;
    }

    // Context.initFromDeviceType (context.zig:36-65): this build only has GPU devices
    static Context *initFromDeviceType(DeviceType type) {
        if (type == DeviceType::cpu) throw Error(WK_E_NO_DEVICE);
        return init(0);
    }

    // Context.initFromBestDevice (context.zig:67-93): the reference scores devices by work-group
    // size x sub-device count; with identical GPUs that is ordinal 0
    static Context *initFromBestDevice(DeviceType type) { return initFromDeviceType(type); }

    void deinit() {
        for (CommandQueue &q : command_queues) wk_stream_destroy(q.stream);
        wk_device_close(device);
        delete this;
    }
};

// ---- Pipeline ------------------------------------------------------------------------------
// The reference chains cl_events: each enqueue waits on prevEvents() (the last appended batch)
// and appends its own event.  On an in-order HIP stream the chain is implicit; the ticket list
// only preserves the observable bookkeeping (pipeline.zig:35-61).
struct Pipeline {
    CommandQueue *command_queue = nullptr;
    std::vector<uint64_t> events;
    size_t prev_batch_start = 0;
    uint64_t next_ticket = 1;

    static Pipeline *init(CommandQueue *cq) {
        Pipeline *p = new Pipeline;
        p->command_queue = cq;
        return p;
    }
    void deinit() { delete this; }
    void prealloc(size_t capacity) { events.reserve(capacity); }

    // last appended batch, empty when nothing is pending
    std::pair<const uint64_t *, size_t> prevEvents() const {
        if (events.empty()) return {nullptr, 0};
        return {events.data() + prev_batch_start, events.size() - prev_batch_start};
    }
    void append(size_t count) {
        prev_batch_start = events.size();
        for (size_t i = 0; i < count; ++i) events.push_back(next_ticket++);
    }
    void waitAndCleanup() {
        if (events.empty()) return;
        check(wk_stream_sync(command_queue->stream));
        events.clear();
        prev_batch_start = 0;
    }
    void clear() {
        events.clear();
        events.shrink_to_fit();
        prev_batch_start = 0;
    }
};

} // namespace core

using core::Context;
using core::Pipeline;

// src/tensor/work_configuration.zig:9-16
enum class GemmAlgorithm : uint8_t { a2x2 = 0, a4x4 = 1, a8x8 = 2, a16x16 = 3, a32x32 = 4, a64x64 = 5 };

struct CreateConfig {
    bool vectors_enabled = true; // src/tensor/main.zig:35-39 (cl_mem_flags / host_ptr have no HIP meaning)
};

namespace detail {
inline uint64_t nextTensorSerial() {
    static std::atomic<uint64_t> counter{0};
    return counter.fetch_add(1, std::memory_order_relaxed) + 1;
}
} // namespace detail

template <typename T> struct Tensor {
    struct Dimensions {
        std::vector<uint64_t> shape, vl_shape, pitches;
        uint64_t number_of_elements = 0;
        uint64_t number_of_elements_without_padding = 0;
    };
    struct MemoryLayout {
        uint64_t row_pitch = 0, row_pitch_for_vectors = 0;
        uint64_t slice_pitch = 0, slice_pitch_for_vectors = 0;
        uint64_t number_of_vectors = 0;
        size_t size = 0;
    };
    struct Flags {
        bool vectors_enabled = false;
    };
    struct WorkConfiguration {
        std::vector<GemmAlgorithm> gemm_algorithm_per_device;
    };

    const Context *context = nullptr;
    void *buffer = nullptr; // device memory (hipMalloc)
    // Unique per tensor ever created in this process (never reused, unlike the address of the object
    // or of its buffer): what a cache keyed on "this tensor" compares.  No counterpart in the reference.
    uint64_t serial = 0;
    Dimensions dimensions;
    MemoryLayout memory_layout;
    Flags flags;
    WorkConfiguration work_configuration;

    // logical {depth, rows, cols} view used by every kernel launch
    uint64_t depth() const {
        uint64_t d = 1;
        const size_t n = dimensions.shape.size();
        for (size_t i = 0; i + 2 < n; ++i) d *= dimensions.shape[i];
        return d;
    }
    uint64_t rows() const {
        const size_t n = dimensions.shape.size();
        return n >= 2 ? dimensions.shape[n - 2] : 1;
    }
    uint64_t cols() const { return dimensions.shape.back(); }

    // Tensor.empty, src/tensor/main.zig:112-251.  Layout differences are listed at the top of
    // this file; the fields keep their meaning.
    static Tensor *empty(const Context *context, Pipeline *pipeline, const std::vector<uint64_t> &shape,
                         CreateConfig config = {}) {
        (void)pipeline;
        if (shape.empty()) throw Error(WK_E_INVALID_VALUE);
        for (uint64_t s : shape)
            if (s == 0) throw Error(WK_E_INVALID_VALUE);

        Tensor *t = new Tensor;
        t->context = context;
        t->serial = detail::nextTensorSerial();
        t->dimensions.shape = shape;
        t->dimensions.vl_shape = shape;

        constexpr bool cplx = core::isComplex<T>();
        const bool vectors_enabled = !cplx && config.vectors_enabled;
        const uint64_t vw = vectors_enabled ? context->command_queues[0].vector_widths[core::getTypeId<T>()] : 1;
        t->flags.vectors_enabled = vectors_enabled && vw > 1;

        const uint64_t cols = shape.back();
        const uint64_t rows = shape.size() >= 2 ? shape[shape.size() - 2] : 1;
        uint64_t depth = 1;
        for (size_t i = 0; i + 2 < shape.size(); ++i) depth *= shape[i];

        uint64_t row_pitch = cols;
        if (vw > 1 && row_pitch % vw) row_pitch += vw - row_pitch % vw;
        // Long rows whose byte pitch is a multiple of 1 KiB land on the same memory channels
        // (measured on MI355X, f32 gemm NN: 8192^3 runs at 135.8 TFLOP/s with a pitch of 32768
        // bytes and at 140 with 32768 + 512; 4096^3 and 2048^3 do not care; at 1024^3 any skew
        // costs a quarter of the rate).  The layout is ours to choose, so pitches from 16 KiB
        // up are skewed by 512 bytes, which keeps row starts on cache-line boundaries.
        if (rows * depth > 1 && row_pitch * sizeof(T) >= 16384 && (row_pitch * sizeof(T)) % 1024 == 0)
            row_pitch += 512 / sizeof(T);

        t->dimensions.number_of_elements_without_padding = depth * rows * cols;
        t->memory_layout.row_pitch = row_pitch;
        t->memory_layout.row_pitch_for_vectors = row_pitch / vw;
        t->dimensions.vl_shape.back() = row_pitch / vw;
        t->memory_layout.slice_pitch = row_pitch * rows;
        t->memory_layout.slice_pitch_for_vectors = t->memory_layout.slice_pitch / vw;
        t->dimensions.number_of_elements = t->memory_layout.slice_pitch * depth;
        t->memory_layout.number_of_vectors = t->dimensions.number_of_elements / vw;
        t->memory_layout.size = (size_t)t->dimensions.number_of_elements * sizeof(T);

        // pitches per dimension (main.zig:198-220): element strides of the padded layout
        const size_t nd = shape.size();
        t->dimensions.pitches.assign(nd, 1);
        if (nd >= 2) t->dimensions.pitches[nd - 2] = row_pitch;
        uint64_t p = t->memory_layout.slice_pitch;
        for (size_t i = nd; i-- > 0;) {
            if (i + 3 > nd) continue; // last two handled above
            t->dimensions.pitches[i] = p;
            p *= shape[i];
        }

        // GemmAlgorithm kept for API compatibility (work_configuration.zig:110-193, `.local`
        // branch): largest block <= 64 dividing the (evened) row count and the row pitch.  The
        // HIP kernels choose their own macro tile per call.
        GemmAlgorithm alg = GemmAlgorithm::a2x2;
        const uint64_t h = rows + rows % 2, w = row_pitch + row_pitch % 2;
        for (int b = 2, i = 0; b <= 64; b *= 2, ++i)
            if (h % b == 0 && w % b == 0) alg = static_cast<GemmAlgorithm>(i);
        t->work_configuration.gemm_algorithm_per_device.assign(context->command_queues.size(), alg);

        int rc = wk_malloc(context->device, t->memory_layout.size, &t->buffer);
        if (rc) {
            delete t;
            throw Error(rc);
        }
        return t;
    }

    // Tensor.alloc = empty + fill.zeroes (main.zig:265-277)
    static Tensor *alloc(const Context *context, Pipeline *pipeline, const std::vector<uint64_t> &shape,
                         CreateConfig config = {}) {
        Tensor *t = empty(context, pipeline, shape, config);
        int rc = wk_memset_async(pipeline->command_queue->stream, t->buffer, 0, t->memory_layout.size);
        if (rc) {
            wk_free(context->device, t->buffer);
            delete t;
            throw Error(rc);
        }
        pipeline->append(1);
        return t;
    }

    // Tensor.release drains the pipeline first (main.zig:253-263)
    void release(Pipeline *pipeline) {
        pipeline->waitAndCleanup();
        wk_free(context->device, buffer);
        delete this;
    }
};

namespace helpers {
// src/tensor/helpers.zig:53-57
template <typename T> void eqlTensorsShape(const Tensor<T> *a, const Tensor<T> *b) {
    if (a->dimensions.shape != b->dimensions.shape) throw Error(WK_E_UNQUAL_TENSORS_SHAPE);
}
} // namespace helpers

namespace memory {
// HOST -> DEVICE of the logical region (src/tensor/memory/read_from_buffer.zig:13-63)
template <typename T> void readFromBuffer(Pipeline *pipeline, Tensor<T> *tensor, const T *buffer, size_t len) {
    if (len != tensor->dimensions.number_of_elements_without_padding) throw Error(WK_E_INVALID_BUFFER);
    const size_t width = (size_t)tensor->cols() * sizeof(T), rows = (size_t)tensor->rows(), depth = (size_t)tensor->depth();
    check(wk_copy_h2d_rect_async(pipeline->command_queue->stream, tensor->buffer,
                                 (size_t)tensor->memory_layout.row_pitch * sizeof(T),
                                 (size_t)tensor->memory_layout.slice_pitch * sizeof(T), buffer, width, width * rows, width,
                                 rows, depth));
    pipeline->append(1);
}
// DEVICE -> HOST of the logical region (src/tensor/memory/write_to_buffer.zig:13-63)
template <typename T> void writeToBuffer(Pipeline *pipeline, Tensor<T> *tensor, T *buffer, size_t len) {
    if (len != tensor->dimensions.number_of_elements_without_padding) throw Error(WK_E_INVALID_BUFFER);
    const size_t width = (size_t)tensor->cols() * sizeof(T), rows = (size_t)tensor->rows(), depth = (size_t)tensor->depth();
    check(wk_copy_d2h_rect_async(pipeline->command_queue->stream, buffer, width, width * rows, tensor->buffer,
                                 (size_t)tensor->memory_layout.row_pitch * sizeof(T),
                                 (size_t)tensor->memory_layout.slice_pitch * sizeof(T), width, rows, depth));
    pipeline->append(1);
}
// DEVICE -> DEVICE of the logical region (src/tensor/memory/copy.zig:84-98)
template <typename T> void copy(Pipeline *pipeline, Tensor<T> *src, Tensor<T> *dst) {
    helpers::eqlTensorsShape<T>(src, dst);
    const size_t width = (size_t)src->cols() * sizeof(T);
    check(wk_copy_d2d_rect_async(pipeline->command_queue->stream, dst->buffer, (size_t)dst->memory_layout.row_pitch * sizeof(T),
                                 (size_t)dst->memory_layout.slice_pitch * sizeof(T), src->buffer,
                                 (size_t)src->memory_layout.row_pitch * sizeof(T),
                                 (size_t)src->memory_layout.slice_pitch * sizeof(T), width, (size_t)src->rows(),
                                 (size_t)src->depth()));
    pipeline->append(1);
}
// element offset of a coordinate (get_value.zig:18-27): InvalidCoordinates on rank or range mismatch
template <typename T> size_t elementOffset(const Tensor<T> *tensor, const std::vector<uint64_t> &coor) {
    const auto &shape = tensor->dimensions.shape;
    if (coor.size() != shape.size()) throw Error(WK_E_INVALID_COORDINATES);
    size_t offset = 0;
    for (size_t i = 0; i < coor.size(); ++i) {
        if (coor[i] >= shape[i]) throw Error(WK_E_INVALID_COORDINATES);
        offset += (size_t)(coor[i] * tensor->dimensions.pitches[i]);
    }
    return offset;
}
// src/tensor/memory/get_value.zig:11-47: non-blocking read of one element into *scalar
template <typename T> void getValue(Pipeline *pipeline, Tensor<T> *tensor, const std::vector<uint64_t> &coor, T *scalar) {
    const size_t offset = elementOffset<T>(tensor, coor);
    check(wk_copy_d2h_rect_async(pipeline->command_queue->stream, scalar, sizeof(T), sizeof(T),
                                 static_cast<const T *>(tensor->buffer) + offset, sizeof(T), sizeof(T), sizeof(T), 1, 1));
    pipeline->append(1);
}
// src/tensor/memory/put_value.zig:11-47
template <typename T> void putValue(Pipeline *pipeline, Tensor<T> *tensor, const std::vector<uint64_t> &coor, const T *scalar) {
    const size_t offset = elementOffset<T>(tensor, coor);
    check(wk_copy_h2d_rect_async(pipeline->command_queue->stream, static_cast<T *>(tensor->buffer) + offset, sizeof(T), sizeof(T),
                                 scalar, sizeof(T), sizeof(T), sizeof(T), 1, 1));
    pipeline->append(1);
}
} // namespace memory

namespace fill {
// src/tensor/fill.zig:70-95
template <typename T> void zeroes(Pipeline *pipeline, Tensor<T> *tensor) {
    check(wk_memset_async(pipeline->command_queue->stream, tensor->buffer, 0, tensor->memory_layout.size));
    pipeline->append(1);
}
// src/tensor/fill.zig:16-57
template <typename T> void constant(Pipeline *pipeline, Tensor<T> *tensor, T value) {
    const uint64_t shape3[3] = {tensor->depth(), tensor->rows(), tensor->cols()};
    check(wk_fill(pipeline->command_queue->stream, core::getTypeIndex<T>(), tensor->buffer, shape3,
                  tensor->memory_layout.row_pitch, tensor->memory_layout.slice_pitch, &value));
    pipeline->append(1);
}
template <typename T> void one(Pipeline *pipeline, Tensor<T> *tensor) { constant<T>(pipeline, tensor, core::getOne<T>()); }
} // namespace fill

// src/tensor/identity.zig:16-70
template <typename T> void identity(Pipeline *pipeline, Tensor<T> *tensor) {
    const uint64_t size = tensor->dimensions.shape[0];
    for (uint64_t s : tensor->dimensions.shape)
        if (s != size) throw Error(WK_E_INVALID_VALUE);
    fill::zeroes<T>(pipeline, tensor);
    uint64_t pitch_sum = 0;
    for (uint64_t p : tensor->dimensions.pitches) pitch_sum += p;
    check(wk_identity(pipeline->command_queue->stream, core::getTypeIndex<T>(), tensor->buffer, size, pitch_sum));
    pipeline->append(1);
}

// src/tensor/transpose.zig:14-105: result = tensor with dimensions dim0 and dim1 exchanged
template <typename T> void transpose(Pipeline *pipeline, Tensor<T> *result_tensor, Tensor<T> *tensor, uint64_t dim0, uint64_t dim1) {
    const auto &shape_a = result_tensor->dimensions.shape, &shape_b = tensor->dimensions.shape;
    if (shape_a.size() != shape_b.size()) throw Error(WK_E_UNQUAL_TENSORS_DIMENSION);
    if (dim0 >= shape_a.size() || dim1 >= shape_a.size()) throw Error(WK_E_INVALID_VALUE);
    if (tensor->dimensions.number_of_elements_without_padding != result_tensor->dimensions.number_of_elements_without_padding)
        throw Error(WK_E_UNQUAL_TENSORS_DIMENSION);
    if (shape_a[dim0] != shape_b[dim1] || shape_a[dim1] != shape_b[dim0]) throw Error(WK_E_INVALID_VALUE);
    if (dim0 == dim1) {
        memory::copy<T>(pipeline, tensor, result_tensor);
        return;
    }
    // the kernel walks the source, so every other dimension has to agree too (the reference's
    // kernel would write out of the result's bounds otherwise)
    for (size_t x = 0; x < shape_a.size(); ++x)
        if (x != dim0 && x != dim1 && shape_a[x] != shape_b[x]) throw Error(WK_E_INVALID_VALUE);
    check(wk_transpose(pipeline->command_queue->stream, core::getTypeIndex<T>(), (int)shape_b.size(), shape_b.data(),
                       tensor->dimensions.pitches.data(), result_tensor->dimensions.pitches.data(), (int)dim0, (int)dim1,
                       tensor->buffer, result_tensor->buffer));
    pipeline->append(1);
}

namespace random {
// src/tensor/random/uniform.zig:60-135.  seed == nullopt draws it from the clock, as there.
template <typename T>
void uniform(Pipeline *pipeline, Tensor<T> *tensor, std::optional<uint64_t> seed,
             std::optional<typename core::scalar_of<T>::type> min_value, std::optional<typename core::scalar_of<T>::type> max_value) {
    using Sub = typename core::scalar_of<T>::type;
    const uint64_t global_seed =
        seed ? *seed : (uint64_t)std::chrono::duration_cast<std::chrono::seconds>(std::chrono::system_clock::now().time_since_epoch()).count();
    const uint64_t shape3[3] = {tensor->depth(), tensor->rows(), tensor->cols()};
    Sub mn{}, range{};
    const bool range_defined = min_value.has_value() || max_value.has_value();
    if (range_defined) {
        mn = min_value.value_or(std::numeric_limits<Sub>::lowest());
        const Sub mx = max_value.value_or(std::numeric_limits<Sub>::max());
        if constexpr (std::is_integral_v<Sub>) {
            using U = std::make_unsigned_t<Sub>;
            range = (Sub)(U)((U)mx - (U)mn); // wraps like the reference's release build when the span exceeds the type
        } else {
            range = mx - mn;
        }
    }
    check(wk_random_uniform(pipeline->command_queue->stream, core::getTypeIndex<T>(), shape3, tensor->buffer,
                            tensor->memory_layout.row_pitch, tensor->memory_layout.slice_pitch, global_seed,
                            range_defined ? &mn : nullptr, range_defined ? &range : nullptr));
    pipeline->append(1);
}
} // namespace random

namespace convertions {
// src/tensor/convertions/to_complex.zig:52-98
template <typename R> void toComplex(Pipeline *pipeline, Tensor<R> *src, Tensor<core::Complex<R>> *dst, core::Space space) {
    if (src->dimensions.shape != dst->dimensions.shape) throw Error(WK_E_UNQUAL_TENSORS_SHAPE);
    const uint64_t shape3[3] = {src->depth(), src->rows(), src->cols()};
    check(wk_to_complex(pipeline->command_queue->stream, core::getTypeIndex<R>(), shape3, src->buffer, src->memory_layout.row_pitch,
                        src->memory_layout.slice_pitch, dst->buffer, dst->memory_layout.row_pitch, dst->memory_layout.slice_pitch,
                        (int)space));
    pipeline->append(1);
}
// src/tensor/convertions/to_real.zig:51-97
template <typename R> void toReal(Pipeline *pipeline, Tensor<core::Complex<R>> *src, Tensor<R> *dst, core::Space space) {
    if (src->dimensions.shape != dst->dimensions.shape) throw Error(WK_E_UNQUAL_TENSORS_SHAPE);
    const uint64_t shape3[3] = {src->depth(), src->rows(), src->cols()};
    check(wk_to_real(pipeline->command_queue->stream, core::getTypeIndex<R>(), shape3, src->buffer, src->memory_layout.row_pitch,
                     src->memory_layout.slice_pitch, dst->buffer, dst->memory_layout.row_pitch, dst->memory_layout.slice_pitch,
                     (int)space));
    pipeline->append(1);
}
} // namespace convertions

// ---- print (src/tensor/print.zig) -----------------------------------------------------------------
// Host-side text rendering of a tensor: the first and last entries of every dimension, numpy style.
// The layout rules (how many items per row, "..." elision, widths, brackets, the trailing
// shape / dtype line) follow print.zig:103-361; number formatting follows Zig's `{d}` / `{e}`
// (exponent without sign padding: 1.50000e0, 1.00000e-3).
namespace print_detail {
inline void pad(std::string &o, size_t n) { o.append(n, ' '); }
inline void right(std::string &o, const std::string &v, size_t width) {
    if (v.size() < width) o.append(width - v.size(), ' ');
    o += v;
    o += ',';
}
// Zig renders a float by taking the shortest decimal that round-trips in ITS type (so 0.3f is "3",
// exponent -1, not 0.30000001192...) and then rounding that decimal, half up, to the requested
// number of fraction digits.
struct Decimal {
    bool negative;
    std::string digits; // d1 d2 d3 ...: value = d1.d2d3... * 10^exponent
    int exponent;
};
template <typename F> Decimal shortest(F v) {
    char buf[64];
    auto r = std::to_chars(buf, buf + sizeof buf, v, std::chars_format::scientific);
    std::string t(buf, r.ptr);
    Decimal d{false, "", 0};
    size_t i = 0;
    if (t[0] == '-') d.negative = true, i = 1;
    for (; i < t.size() && t[i] != 'e'; ++i)
        if (t[i] != '.') d.digits += t[i];
    d.exponent = std::atoi(t.c_str() + i + 1);
    return d;
}
// keeps `keep` leading digits of d.digits (may be <= 0), rounding half up; returns true on a carry out
inline bool round_digits(std::string &digits, long keep) {
    if (keep < 0) {
        digits.clear();
        return false;
    }
    if ((long)digits.size() <= keep) {
        digits.append(keep - digits.size(), '0');
        return false;
    }
    const bool up = digits[keep] >= '5';
    digits.resize(keep);
    if (!up) return false;
    for (long i = keep; i-- > 0;) {
        if (digits[i] != '9') {
            ++digits[i];
            return false;
        }
        digits[i] = '0';
    }
    return true;
}
template <typename F> std::string special(F v) { return std::isnan(v) ? "nan" : v < 0 ? "-inf" : "inf"; }
template <typename F> std::string zig_e(F v, int prec) {
    if (!std::isfinite(v)) return special(v);
    Decimal d = shortest(v);
    if (round_digits(d.digits, prec + 1)) {
        d.digits.insert(d.digits.begin(), '1');
        d.digits.pop_back();
        ++d.exponent;
    }
    std::string o = d.negative ? "-" : "";
    o += d.digits[0];
    if (prec > 0) o += "." + d.digits.substr(1);
    return o + "e" + std::to_string(d.exponent);
}
template <typename F> std::string zig_d(F v, int prec) {
    if (!std::isfinite(v)) return special(v);
    Decimal d = shortest(v);
    long int_digits = (long)d.exponent + 1; // digits in front of the point (<= 0: leading zeros behind it)
    std::string digits = d.digits;
    if (int_digits <= 0) {
        digits.insert(0, (size_t)(1 - int_digits), '0');
        int_digits = 1;
    }
    if (round_digits(digits, int_digits + prec)) {
        digits.insert(digits.begin(), '1');
        ++int_digits;
    }
    std::string o = d.negative ? "-" : "";
    o += digits.substr(0, int_digits);
    if (prec > 0) o += "." + digits.substr(int_digits);
    return o;
}
template <typename I> std::string int_str(I v) { return std::to_string((long long)v); }
template <> inline std::string int_str<uint64_t>(uint64_t v) { return std::to_string(v); }

template <typename T> void vector(std::string &o, size_t padding, const T *buf, uint64_t cols) {
    using Sub = typename core::scalar_of<T>::type;
    constexpr bool cplx = core::isComplex<T>();
    pad(o, padding);
    auto loop = [&](uint64_t head, uint64_t max_items, size_t ell_width, auto &&item) {
        for (uint64_t i = 0; i < head && i < cols; ++i) item(i);
        if (cols > head) {
            uint64_t dec = head + 1;
            if (cols > max_items) {
                dec = head;
                right(o, "...", ell_width);
            }
            for (uint64_t i = std::max<uint64_t>(head, cols - dec); i < cols; ++i) item(i);
        }
    };
    if constexpr (std::is_integral_v<Sub>) {
        const std::string ext = std::is_signed_v<Sub> ? int_str(std::numeric_limits<Sub>::min()) : int_str(std::numeric_limits<Sub>::max());
        const std::string widest = cplx ? (std::is_signed_v<Sub> ? ext + ext + "j" : ext + "+" + ext + "j") : ext;
        const size_t width = widest.size() + 1;
        uint64_t max_items = std::max<uint64_t>(cplx ? 3 : 5, 65 / widest.size());
        if (max_items % 2 == 0) ++max_items;
        const uint64_t head = std::min<uint64_t>(cols, (max_items - 1) / 2);
        loop(head, max_items, width, [&](uint64_t i) {
            if constexpr (cplx) {
                const Sub re = buf[i].real, im = buf[i].imag;
                std::string v;
                if (re != 0 && im != 0) v = int_str(re) + (im < 0 ? "" : "+") + int_str(im) + "j";
                else if (im != 0) v = int_str(im) + "j";
                else v = int_str(re);
                right(o, v, width);
            } else {
                right(o, int_str(buf[i]), width);
            }
        });
    } else if constexpr (cplx) {
        loop(2, 5, 24, [&](uint64_t i) {
            const Sub re = buf[i].real, im = buf[i].imag;
            const bool rz = std::fabs(re) < 1e-8, iz = std::fabs(im) < 1e-8;
            std::string v;
            if (!rz && !iz) v = zig_e(re, 2) + (im < 0 ? "" : "+") + zig_e(im, 2) + "j";
            else if (rz && !iz) v = zig_e(im, 5) + "j";
            else v = zig_e(re, 5);
            right(o, v, 24);
        });
    } else {
        loop(4, 9, 14, [&](uint64_t i) {
            const T v = buf[i];
            right(o, (10000.0 - std::fabs((double)v)) > 1e-8 ? zig_d(v, 8) : zig_e(v, 5), 14);
        });
    }
}

template <typename T>
void dim(std::string &o, size_t padding, const T *buf, const uint64_t *shape, const uint64_t *pitches, size_t nd) {
    pad(o, padding);
    o += '[';
    if (nd > 2) {
        o += '\n';
        const uint64_t n = shape[0], pitch = pitches[0];
        for (uint64_t i = 0; i < std::min<uint64_t>(2, n); ++i) dim<T>(o, padding + 2, buf + i * pitch, shape + 1, pitches + 1, nd - 1);
        if (n > 2) {
            if (n > 4) {
                o += '\n';
                pad(o, padding + 2);
                o += "... \n";
            }
            for (uint64_t i = std::max<uint64_t>(2, n - 2); i < n; ++i) dim<T>(o, padding + 2, buf + i * pitch, shape + 1, pitches + 1, nd - 1);
        }
        o += '\n';
    } else if (nd == 1) {
        vector<T>(o, padding, buf, shape[0]);
    } else {
        const uint64_t rows = shape[0], cols = shape[1], pitch = pitches[0];
        for (uint64_t i = 0; i < std::min<uint64_t>(2, rows); ++i) {
            o += '\n';
            vector<T>(o, padding + 2, buf + i * pitch, cols);
        }
        if (rows > 2) {
            if (rows > 4) {
                o += '\n';
                pad(o, padding + 2);
                o += " ... ";
            }
            for (uint64_t i = std::max<uint64_t>(2, rows - 2); i < rows; ++i) {
                o += '\n';
                vector<T>(o, padding + 2, buf + i * pitch, cols);
            }
        }
        o += '\n';
    }
    pad(o, padding);
    o += "],";
    if (padding > 0) o += '\n';
}
template <typename T> const char *type_name() {
    using Sub = typename core::scalar_of<T>::type;
    if constexpr (std::is_same_v<Sub, float>) return "f32";
    else if constexpr (std::is_same_v<Sub, double>) return "f64";
    else if constexpr (std::is_signed_v<Sub>) return sizeof(Sub) == 1 ? "i8" : sizeof(Sub) == 2 ? "i16" : sizeof(Sub) == 4 ? "i32" : "i64";
    else return sizeof(Sub) == 1 ? "u8" : sizeof(Sub) == 2 ? "u16" : sizeof(Sub) == 4 ? "u32" : "u64";
}
} // namespace print_detail

// printZ (print.zig:316-361): drains the pipeline, copies the buffer to the host, renders it
template <typename T> std::string printZ(Pipeline *pipeline, Tensor<T> *tensor) {
    std::vector<T> host(tensor->dimensions.number_of_elements);
    check(wk_copy_d2h_rect_async(pipeline->command_queue->stream, host.data(), tensor->memory_layout.size, tensor->memory_layout.size,
                                 tensor->buffer, tensor->memory_layout.size, tensor->memory_layout.size, tensor->memory_layout.size,
                                 1, 1));
    pipeline->append(1);
    pipeline->waitAndCleanup();
    std::string o = "Tensor(";
    const auto &shape = tensor->dimensions.shape;
    print_detail::dim<T>(o, 0, host.data(), shape.data(), tensor->dimensions.pitches.data(), shape.size());
    o += " shape=(" + std::to_string(shape[0]);
    for (size_t i = 1; i < shape.size(); ++i) o += ", " + std::to_string(shape[i]);
    o += ')';
    o += core::isComplex<T>() ? std::string(", dtype=complex_") + print_detail::type_name<T>() + ")\n"
                              : std::string(", dtype=") + print_detail::type_name<T>() + ")\n";
    return o;
}
// print (print.zig:363-382): to standard output
template <typename T> void print(Pipeline *pipeline, Tensor<T> *tensor) {
    const std::string o = printZ<T>(pipeline, tensor);
    std::fwrite(o.data(), 1, o.size(), stdout);
    std::fflush(stdout);
}

namespace blas {

enum class Operation : uint8_t { no_transpose = 0, transpose = 1 }; // src/blas/gemm.zig:25-29

// src/blas/axpy.zig:93-169.  alpha == nullopt: y += x; alpha == -1: y -= x; else y += alpha*x.
template <typename T> void axpy(Pipeline *pipeline, Tensor<T> *x, std::optional<T> alpha, Tensor<T> *y) {
    helpers::eqlTensorsShape<T>(x, y);
    const uint64_t shape3[3] = {x->depth(), x->rows(), x->cols()};
    const T a = alpha.value_or(T{});
    check(wk_axpy(pipeline->command_queue->stream, core::getTypeIndex<T>(), shape3, x->buffer, x->memory_layout.row_pitch,
                  x->memory_layout.slice_pitch, y->buffer, y->memory_layout.row_pitch, y->memory_layout.slice_pitch,
                  alpha ? &a : nullptr));
    pipeline->append(1);
}

// src/blas/gemm.zig:60-359.  n_size = rows of C, m_size = columns of C (the reference's naming).
template <typename T> struct PackedTensors {
    uint64_t m_size = 0, n_size = 0, k_size = 0;
    Tensor<T> *packed_a = nullptr, *packed_b = nullptr; // never allocated: the packed form is not a tensor here
    bool vectors_enabled = false;
    GemmAlgorithm algorithm = GemmAlgorithm::a2x2;
    // device memory the library's gemm packs into (wk_gemm_workspace_bytes; zero bytes for most types)
    wk_device *device = nullptr;
    void *workspace = nullptr;
    size_t workspace_bytes = 0;
    // No counterpart in the reference, which packs both operands before every product
    // (gemm.zig:713-719).  keepB(true) declares B a constant operand (weights): gemm calls after the
    // first with the same B tensor, op_b, queue and alpha (alpha is folded into the packed B of the
    // complex types) leave B's packed form in the workspace as it is and pack only A.  After B's
    // contents change, invalidateB() makes the next call pack it again.
    // B is recognised by the tensor's serial (a released B whose address a new tensor reuses is a
    // different tensor), its buffer and its row pitch, and is recorded only once a product with it
    // has been enqueued without error.
    bool keep_b = false;
    uint64_t kept_b_serial = 0; // 0: the workspace holds no B
    const void *kept_b_buffer = nullptr;
    uint64_t kept_b_pitch = 0;
    Operation kept_op_b = Operation::no_transpose;
    const void *kept_stream = nullptr;
    std::optional<T> kept_alpha;
    void keepB(bool on) {
        keep_b = on;
        kept_b_serial = 0;
    }
    void invalidateB() { kept_b_serial = 0; }
    // true when the workspace holds this B already
    bool holdsB(const Tensor<T> *b, Operation op_b, const void *stream, const std::optional<T> &alpha) const {
        if (!keep_b || kept_b_serial == 0) return false;
        const bool same_alpha = alpha.has_value() == kept_alpha.has_value() &&
                                (!alpha || std::memcmp(&*alpha, &*kept_alpha, sizeof(T)) == 0);
        return kept_b_serial == b->serial && kept_b_buffer == b->buffer && kept_b_pitch == b->memory_layout.row_pitch &&
               kept_op_b == op_b && kept_stream == stream && same_alpha;
    }
    // after a product with this B went through
    void recordB(const Tensor<T> *b, Operation op_b, const void *stream, const std::optional<T> &alpha) {
        if (!keep_b) return;
        kept_b_serial = b->serial;
        kept_b_buffer = b->buffer;
        kept_b_pitch = b->memory_layout.row_pitch;
        kept_op_b = op_b;
        kept_stream = stream;
        kept_alpha = alpha;
    }

    static PackedTensors *init(Pipeline *pipeline, Tensor<T> *result_tensor, uint64_t k_size, bool vectors_enabled) {
        const auto &shape = result_tensor->dimensions.shape;
        if (shape.size() != 2) throw Error(WK_E_INVALID_VALUE);
        const uint32_t id = pipeline->command_queue->wekua_id;
        return initWithDimensions(pipeline, shape[0], shape[1], k_size,
                                  result_tensor->work_configuration.gemm_algorithm_per_device[id], vectors_enabled);
    }
    static PackedTensors *initWithDimensions(Pipeline *pipeline, uint64_t n_size, uint64_t m_size, uint64_t k_size,
                                             GemmAlgorithm recommended_algorithm, bool vectors_enabled) {
        if (!n_size || !m_size || !k_size) throw Error(WK_E_INVALID_VALUE);
        PackedTensors *p = new PackedTensors;
        p->n_size = n_size;
        p->m_size = m_size;
        p->k_size = k_size;
        p->vectors_enabled = !core::isComplex<T>() && vectors_enabled;
        p->algorithm = recommended_algorithm;
        p->device = pipeline->command_queue->context->device;
        p->workspace_bytes = wk_gemm_workspace_bytes(core::getTypeIndex<T>(), 0, 0, n_size, m_size, k_size);
        if (p->workspace_bytes) {
            const int rc = wk_malloc(p->device, p->workspace_bytes, &p->workspace);
            if (rc) {
                delete p;
                throw Error(rc);
            }
        }
        return p;
    }
    void deinit(Pipeline *pipeline) {
        pipeline->waitAndCleanup(); // the reference's deinit releases two tensors, each draining the pipeline
        if (workspace) wk_free(device, workspace);
        delete this;
    }
    // gemm.zig:250-270
    void validateTensors(const Tensor<T> *a, Operation op_a, const Tensor<T> *b, Operation op_b) const {
        const auto &as = a->dimensions.shape, &bs = b->dimensions.shape;
        if (as.size() != 2 || bs.size() != 2) throw Error(WK_E_INVALID_VALUE);
        bool valid = op_a == Operation::no_transpose ? (as[0] == n_size && as[1] == k_size)
                                                     : (as[1] == n_size && as[0] == k_size);
        valid &= op_b == Operation::no_transpose ? (bs[0] == k_size && bs[1] == m_size)
                                                 : (bs[1] == k_size && bs[0] == m_size);
        if (!valid) throw Error(WK_E_INVALID_VALUE);
    }
    // gemm.zig:272-357: validation; the pack pass itself runs inside wk_gemm, on the workspace
    void pack(Pipeline *pipeline, Tensor<T> *a, Operation op_a, Tensor<T> *b, Operation op_b) {
        (void)pipeline;
        validateTensors(a, op_a, b, op_b);
    }
};

// src/blas/gemm.zig:442-485
template <typename T>
void validateTensors(const Tensor<T> *a, const Tensor<T> *b, const Tensor<T> *c, Operation op_a, Operation op_b) {
    if (a->context != b->context || a->context != c->context) throw Error(WK_E_UNQUAL_TENSORS_CONTEXT);
    const auto &as = a->dimensions.shape, &bs = b->dimensions.shape, &cs = c->dimensions.shape;
    if (cs.size() != 2 || as.size() != 2 || bs.size() != 2) throw Error(WK_E_INVALID_VALUE);
    const uint64_t a_m = as[0], a_k = as[1], b_k = bs[0], b_n = bs[1], c_m = cs[0], c_n = cs[1];
    bool match;
    if (op_a == Operation::transpose)
        match = op_b == Operation::no_transpose ? (a_m == b_k && b_n == c_n && a_k == c_m)
                                                : (a_m == b_n && b_k == c_n && a_k == c_m);
    else
        match = op_b == Operation::no_transpose ? (a_k == b_k && b_n == c_n && a_m == c_m)
                                                : (a_k == b_n && b_k == c_n && a_m == c_m);
    if (!match) throw Error(WK_E_INVALID_VALUE);
}

// src/blas/gemm.zig:834-874
template <typename T>
void gemm(Pipeline *pipeline, std::optional<T> alpha, Tensor<T> *a, Operation op_a, Tensor<T> *b, Operation op_b,
          std::optional<T> beta, Tensor<T> *c, PackedTensors<T> *packed_tensors = nullptr) {
    validateTensors<T>(a, b, c, op_a, op_b);
    if (packed_tensors) packed_tensors->pack(pipeline, a, op_a, b, op_b);
    const uint64_t M = c->dimensions.shape[0], N = c->dimensions.shape[1];
    const uint64_t K = a->dimensions.shape[op_a == Operation::transpose ? 0 : 1];
    const T av = alpha.value_or(T{}), bv = beta.value_or(T{});
    wk_stream *stream = pipeline->command_queue->stream;
    const bool b_kept = packed_tensors && packed_tensors->holdsB(b, op_b, stream, alpha);
    const int rc = (b_kept ? wk_gemm_packed_b_kept : wk_gemm)(
        stream, core::getTypeIndex<T>(), (int)op_a, (int)op_b, M, N, K, alpha ? &av : nullptr, a->buffer,
        a->memory_layout.row_pitch, b->buffer, b->memory_layout.row_pitch, beta ? &bv : nullptr, c->buffer,
        c->memory_layout.row_pitch, packed_tensors ? packed_tensors->workspace : nullptr,
        packed_tensors ? packed_tensors->workspace_bytes : 0);
    if (packed_tensors) {
        if (rc) packed_tensors->invalidateB(); // whatever the workspace holds now, it is not trusted
        else packed_tensors->recordB(b, op_b, stream, alpha);
    }
    check(rc);
    pipeline->append(1);
}

} // namespace blas

using GemmOperation = blas::Operation;
template <typename T> using GemmPackedTensors = blas::PackedTensors<T>;

} // namespace wekua
