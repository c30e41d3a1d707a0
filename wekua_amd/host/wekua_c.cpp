// wekua_c.cpp -- flat C entry points over the C++ host mirror (wekua.hpp), one per public
// function of the reference's Zig API on the gemm/axpy path, with the element type passed as
// the dtype id of src/core/types.zig getTypeIndex.  This is what the Python package binds, so
// the parity tests exercise the same host logic (validation, layout, option handling) a C++
// caller gets.  Every function returns a WK_E_* code (the Zig error name) and never throws.
#include "wekua.hpp"
#include "wekua_nn.hpp"

#include <new>

using namespace wekua;
using wekua::blas::Operation;

namespace {

struct TensorHandle {
    int dtype;
    void *tensor; // Tensor<T>*
};

struct PackedHandle {
    int dtype;
    void *packed; // blas::PackedTensors<T>*
};

// nn objects exist for f32 and f64 only, like the reference's (src/nn/optimizers/gd.zig:17-20)
struct LayerHandle {
    int dtype;
    void *layer; // nn::Layer<T>*
};
struct CacheHandle {
    int dtype;
    void *cache; // nn::Cache<T>*
};
struct OptimizerHandle {
    int dtype;
    void *optimizer; // nn::optimizers::Optimizer<T>*
};

template <typename F> void dispatch_real_component(int dtype, F &&f) {
    switch (dtype) {
    case 0: f.template operator()<int8_t>(); break;
    case 1: f.template operator()<uint8_t>(); break;
    case 2: f.template operator()<int16_t>(); break;
    case 3: f.template operator()<uint16_t>(); break;
    case 4: f.template operator()<int32_t>(); break;
    case 5: f.template operator()<uint32_t>(); break;
    case 6: f.template operator()<int64_t>(); break;
    case 7: f.template operator()<uint64_t>(); break;
    case 8: f.template operator()<float>(); break;
    case 9: f.template operator()<double>(); break;
    default: throw Error(WK_E_TYPE_NOT_SUPPORTED);
    }
}
template <typename F> void dispatch_real(int dtype, F &&f) {
    switch (dtype) {
    case 8: f.template operator()<float>(); break;
    case 9: f.template operator()<double>(); break;
    default: throw Error(WK_E_TYPE_NOT_SUPPORTED);
    }
}

template <typename F> int guard(F &&f) {
    try {
        f();
        return WK_OK;
    } catch (const Error &e) {
        return e.code;
    } catch (const std::bad_alloc &) {
        return WK_E_OUT_OF_MEMORY;
    } catch (...) {
        return WK_E_INVALID_VALUE;
    }
}

template <typename F> void dispatch(int dtype, F &&f) {
    using namespace wekua::core;
    switch (dtype) {
    case 0: f.template operator()<int8_t>(); break;
    case 1: f.template operator()<uint8_t>(); break;
    case 2: f.template operator()<int16_t>(); break;
    case 3: f.template operator()<uint16_t>(); break;
    case 4: f.template operator()<int32_t>(); break;
    case 5: f.template operator()<uint32_t>(); break;
    case 6: f.template operator()<int64_t>(); break;
    case 7: f.template operator()<uint64_t>(); break;
    case 8: f.template operator()<float>(); break;
    case 9: f.template operator()<double>(); break;
    case 10: f.template operator()<Complex<int8_t>>(); break;
    case 11: f.template operator()<Complex<uint8_t>>(); break;
    case 12: f.template operator()<Complex<int16_t>>(); break;
    case 13: f.template operator()<Complex<uint16_t>>(); break;
    case 14: f.template operator()<Complex<int32_t>>(); break;
    case 15: f.template operator()<Complex<uint32_t>>(); break;
    case 16: f.template operator()<Complex<int64_t>>(); break;
    case 17: f.template operator()<Complex<uint64_t>>(); break;
    case 18: f.template operator()<Complex<float>>(); break;
    case 19: f.template operator()<Complex<double>>(); break;
    default: throw Error(WK_E_TYPE_NOT_SUPPORTED);
    }
}

template <typename T> std::optional<T> opt_scalar(const void *p) {
    if (!p) return std::nullopt;
    T v;
    std::memcpy(&v, p, sizeof(T));
    return v;
}

} // namespace

extern "C" {

struct wkz_tensor_info {
    int dtype;
    int ndim;
    uint64_t shape[8];
    uint64_t pitches[8];
    uint64_t number_of_elements;
    uint64_t number_of_elements_without_padding;
    uint64_t row_pitch, row_pitch_for_vectors, slice_pitch, slice_pitch_for_vectors, number_of_vectors;
    uint64_t size;
    int vectors_enabled;
    int gemm_algorithm;
    void *buffer;
};

// ---- Context / Pipeline --------------------------------------------------------------------
int wkz_context_init_from_device_type(int device_type, void **out) {
    return guard([&] { *out = Context::initFromDeviceType(static_cast<core::DeviceType>(device_type)); });
}
int wkz_context_init_from_best_device(int device_type, void **out) {
    return guard([&] { *out = Context::initFromBestDevice(static_cast<core::DeviceType>(device_type)); });
}
int wkz_context_init(int ordinal, void **out) {
    return guard([&] { *out = Context::init(ordinal); });
}
void wkz_context_deinit(void *ctx) {
    if (ctx) static_cast<Context *>(ctx)->deinit();
}
int wkz_context_num_queues(void *ctx) { return (int)static_cast<Context *>(ctx)->command_queues.size(); }
void *wkz_context_stream(void *ctx, int queue) { return static_cast<Context *>(ctx)->command_queues[queue].stream; }
void *wkz_context_device(void *ctx) { return static_cast<Context *>(ctx)->device; }

int wkz_pipeline_init(void *ctx, int queue, void **out) {
    return guard([&] {
        Context *c = static_cast<Context *>(ctx);
        if (queue < 0 || (size_t)queue >= c->command_queues.size()) throw Error(WK_E_INVALID_VALUE);
        *out = Pipeline::init(&c->command_queues[queue]);
    });
}
void wkz_pipeline_deinit(void *p) {
    if (p) static_cast<Pipeline *>(p)->deinit();
}
int wkz_pipeline_prealloc(void *p, uint64_t n) {
    return guard([&] { static_cast<Pipeline *>(p)->prealloc(n); });
}
int wkz_pipeline_wait_and_cleanup(void *p) {
    return guard([&] { static_cast<Pipeline *>(p)->waitAndCleanup(); });
}
uint64_t wkz_pipeline_pending(void *p) { return static_cast<Pipeline *>(p)->events.size(); }
uint64_t wkz_pipeline_prev_events(void *p) { return static_cast<Pipeline *>(p)->prevEvents().second; }
void wkz_pipeline_clear(void *p) { static_cast<Pipeline *>(p)->clear(); }

// ---- Tensor ----------------------------------------------------------------------------------
static int tensor_create(void *ctx, void *pipeline, int dtype, const uint64_t *shape, int ndim, int vectors_enabled,
                         bool zero, void **out) {
    return guard([&] {
        if (!out || ndim < 0 || ndim > 8 || (ndim > 0 && !shape)) throw Error(WK_E_INVALID_VALUE);
        std::vector<uint64_t> shp(shape, shape + ndim);
        CreateConfig cfg;
        cfg.vectors_enabled = vectors_enabled != 0;
        dispatch(dtype, [&]<typename T>() {
            Tensor<T> *t = zero ? Tensor<T>::alloc(static_cast<Context *>(ctx), static_cast<Pipeline *>(pipeline), shp, cfg)
                                : Tensor<T>::empty(static_cast<Context *>(ctx), static_cast<Pipeline *>(pipeline), shp, cfg);
            *out = new TensorHandle{dtype, t};
        });
    });
}
int wkz_tensor_alloc(void *ctx, void *pipeline, int dtype, const uint64_t *shape, int ndim, int vectors_enabled, void **out) {
    return tensor_create(ctx, pipeline, dtype, shape, ndim, vectors_enabled, true, out);
}
int wkz_tensor_empty(void *ctx, void *pipeline, int dtype, const uint64_t *shape, int ndim, int vectors_enabled, void **out) {
    return tensor_create(ctx, pipeline, dtype, shape, ndim, vectors_enabled, false, out);
}
int wkz_tensor_release(void *tensor, void *pipeline) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() { static_cast<Tensor<T> *>(h->tensor)->release(static_cast<Pipeline *>(pipeline)); });
        delete h;
    });
}
int wkz_tensor_get_info(void *tensor, wkz_tensor_info *info) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() {
            const Tensor<T> *t = static_cast<Tensor<T> *>(h->tensor);
            std::memset(info, 0, sizeof *info);
            info->dtype = h->dtype;
            info->ndim = (int)t->dimensions.shape.size();
            for (int i = 0; i < info->ndim; ++i) {
                info->shape[i] = t->dimensions.shape[i];
                info->pitches[i] = t->dimensions.pitches[i];
            }
            info->number_of_elements = t->dimensions.number_of_elements;
            info->number_of_elements_without_padding = t->dimensions.number_of_elements_without_padding;
            info->row_pitch = t->memory_layout.row_pitch;
            info->row_pitch_for_vectors = t->memory_layout.row_pitch_for_vectors;
            info->slice_pitch = t->memory_layout.slice_pitch;
            info->slice_pitch_for_vectors = t->memory_layout.slice_pitch_for_vectors;
            info->number_of_vectors = t->memory_layout.number_of_vectors;
            info->size = t->memory_layout.size;
            info->vectors_enabled = t->flags.vectors_enabled;
            info->gemm_algorithm = (int)t->work_configuration.gemm_algorithm_per_device[0];
            info->buffer = t->buffer;
        });
    });
}

// ---- memory / fill / identity ------------------------------------------------------------------
int wkz_read_from_buffer(void *pipeline, void *tensor, const void *host, uint64_t len) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() {
            memory::readFromBuffer<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor),
                                      static_cast<const T *>(host), (size_t)len);
        });
    });
}
int wkz_write_to_buffer(void *pipeline, void *tensor, void *host, uint64_t len) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() {
            memory::writeToBuffer<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor),
                                     static_cast<T *>(host), (size_t)len);
        });
    });
}
int wkz_fill_zeroes(void *pipeline, void *tensor) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() { fill::zeroes<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor)); });
    });
}
int wkz_fill_one(void *pipeline, void *tensor) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() { fill::one<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor)); });
    });
}
int wkz_fill_constant(void *pipeline, void *tensor, const void *host_scalar) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        if (!host_scalar) throw Error(WK_E_INVALID_VALUE);
        dispatch(h->dtype, [&]<typename T>() {
            fill::constant<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor), *opt_scalar<T>(host_scalar));
        });
    });
}
int wkz_identity(void *pipeline, void *tensor) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() { identity<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor)); });
    });
}

// ---- tensor support operations --------------------------------------------------------------------
int wkz_memory_copy(void *pipeline, void *src, void *dst) {
    return guard([&] {
        TensorHandle *hs = static_cast<TensorHandle *>(src), *hd = static_cast<TensorHandle *>(dst);
        if (hs->dtype != hd->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch(hs->dtype, [&]<typename T>() {
            memory::copy<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(hs->tensor), static_cast<Tensor<T> *>(hd->tensor));
        });
    });
}
int wkz_get_value(void *pipeline, void *tensor, const uint64_t *coor, uint64_t ncoor, void *host_scalar) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        if (!host_scalar || (ncoor && !coor)) throw Error(WK_E_INVALID_VALUE);
        dispatch(h->dtype, [&]<typename T>() {
            memory::getValue<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor),
                                std::vector<uint64_t>(coor, coor + ncoor), static_cast<T *>(host_scalar));
        });
    });
}
int wkz_put_value(void *pipeline, void *tensor, const uint64_t *coor, uint64_t ncoor, const void *host_scalar) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        if (!host_scalar || (ncoor && !coor)) throw Error(WK_E_INVALID_VALUE);
        dispatch(h->dtype, [&]<typename T>() {
            memory::putValue<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor),
                                std::vector<uint64_t>(coor, coor + ncoor), static_cast<const T *>(host_scalar));
        });
    });
}
int wkz_transpose(void *pipeline, void *result, void *tensor, uint64_t dim0, uint64_t dim1) {
    return guard([&] {
        TensorHandle *hr = static_cast<TensorHandle *>(result), *ht = static_cast<TensorHandle *>(tensor);
        if (hr->dtype != ht->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch(ht->dtype, [&]<typename T>() {
            transpose<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(hr->tensor), static_cast<Tensor<T> *>(ht->tensor), dim0,
                         dim1);
        });
    });
}
// seed, host_min, host_max: NULL for an absent (null) argument; min / max are of the real component type
int wkz_random_uniform(void *pipeline, void *tensor, const uint64_t *seed, const void *host_min, const void *host_max) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() {
            using Sub = typename core::scalar_of<T>::type;
            random::uniform<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor),
                               seed ? std::optional<uint64_t>(*seed) : std::nullopt, opt_scalar<Sub>(host_min), opt_scalar<Sub>(host_max));
        });
    });
}
int wkz_to_complex(void *pipeline, void *src, void *dst, int space) {
    return guard([&] {
        TensorHandle *hs = static_cast<TensorHandle *>(src), *hd = static_cast<TensorHandle *>(dst);
        if (hd->dtype != hs->dtype + 10 || (space != 0 && space != 1)) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch_real_component(hs->dtype, [&]<typename R>() {
            convertions::toComplex<R>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<R> *>(hs->tensor),
                                      static_cast<Tensor<core::Complex<R>> *>(hd->tensor), static_cast<core::Space>(space));
        });
    });
}
int wkz_to_real(void *pipeline, void *src, void *dst, int space) {
    return guard([&] {
        TensorHandle *hs = static_cast<TensorHandle *>(src), *hd = static_cast<TensorHandle *>(dst);
        if (hs->dtype != hd->dtype + 10 || (space != 0 && space != 1)) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch_real_component(hd->dtype, [&]<typename R>() {
            convertions::toReal<R>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<core::Complex<R>> *>(hs->tensor),
                                   static_cast<Tensor<R> *>(hd->tensor), static_cast<core::Space>(space));
        });
    });
}

// printZ into a caller buffer: returns the text length (without terminator) through *needed; copies at
// most capacity - 1 bytes plus a terminator.  Call with capacity 0 to size the buffer.
int wkz_print(void *pipeline, void *tensor, char *out, uint64_t capacity, uint64_t *needed) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch(h->dtype, [&]<typename T>() {
            const std::string text = printZ<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor));
            if (needed) *needed = text.size();
            if (out && capacity) {
                const size_t n = std::min<size_t>(text.size(), capacity - 1);
                std::memcpy(out, text.data(), n);
                out[n] = 0;
            }
        });
    });
}

// ---- blas -----------------------------------------------------------------------------------------
int wkz_axpy(void *pipeline, void *x, const void *host_alpha, void *y) {
    return guard([&] {
        TensorHandle *hx = static_cast<TensorHandle *>(x), *hy = static_cast<TensorHandle *>(y);
        if (hx->dtype != hy->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE); // Zig rejects this at compile time
        dispatch(hx->dtype, [&]<typename T>() {
            blas::axpy<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(hx->tensor), opt_scalar<T>(host_alpha),
                          static_cast<Tensor<T> *>(hy->tensor));
        });
    });
}

int wkz_packed_init(void *pipeline, void *result_tensor, uint64_t k_size, int vectors_enabled, void **out) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(result_tensor);
        dispatch(h->dtype, [&]<typename T>() {
            auto *p = blas::PackedTensors<T>::init(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor), k_size,
                                                   vectors_enabled != 0);
            *out = new PackedHandle{h->dtype, p};
        });
    });
}
int wkz_packed_init_with_dimensions(void *pipeline, int dtype, uint64_t n_size, uint64_t m_size, uint64_t k_size,
                                    int recommended_algorithm, int vectors_enabled, void **out) {
    return guard([&] {
        dispatch(dtype, [&]<typename T>() {
            auto *p = blas::PackedTensors<T>::initWithDimensions(static_cast<Pipeline *>(pipeline), n_size, m_size, k_size,
                                                                 static_cast<GemmAlgorithm>(recommended_algorithm),
                                                                 vectors_enabled != 0);
            *out = new PackedHandle{dtype, p};
        });
    });
}
int wkz_packed_deinit(void *packed, void *pipeline) {
    return guard([&] {
        PackedHandle *h = static_cast<PackedHandle *>(packed);
        dispatch(h->dtype, [&]<typename T>() { static_cast<blas::PackedTensors<T> *>(h->packed)->deinit(static_cast<Pipeline *>(pipeline)); });
        delete h;
    });
}
// bytes of device memory the handle holds for the library's pack pass (0 for most types)
int wkz_packed_workspace_bytes(void *packed, uint64_t *out) {
    return guard([&] {
        PackedHandle *h = static_cast<PackedHandle *>(packed);
        dispatch(h->dtype, [&]<typename T>() { *out = static_cast<blas::PackedTensors<T> *>(h->packed)->workspace_bytes; });
    });
}
int wkz_packed_keep_b(void *packed, int on) {
    return guard([&] {
        PackedHandle *h = static_cast<PackedHandle *>(packed);
        dispatch(h->dtype, [&]<typename T>() { static_cast<blas::PackedTensors<T> *>(h->packed)->keepB(on != 0); });
    });
}
int wkz_packed_invalidate_b(void *packed) {
    return guard([&] {
        PackedHandle *h = static_cast<PackedHandle *>(packed);
        dispatch(h->dtype, [&]<typename T>() { static_cast<blas::PackedTensors<T> *>(h->packed)->invalidateB(); });
    });
}
int wkz_packed_pack(void *packed, void *pipeline, void *a, int op_a, void *b, int op_b) {
    return guard([&] {
        PackedHandle *h = static_cast<PackedHandle *>(packed);
        TensorHandle *ha = static_cast<TensorHandle *>(a), *hb = static_cast<TensorHandle *>(b);
        if (ha->dtype != h->dtype || hb->dtype != h->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch(h->dtype, [&]<typename T>() {
            static_cast<blas::PackedTensors<T> *>(h->packed)->pack(static_cast<Pipeline *>(pipeline),
                                                                   static_cast<Tensor<T> *>(ha->tensor), static_cast<Operation>(op_a),
                                                                   static_cast<Tensor<T> *>(hb->tensor), static_cast<Operation>(op_b));
        });
    });
}

int wkz_gemm(void *pipeline, const void *host_alpha, void *a, int op_a, void *b, int op_b, const void *host_beta, void *c,
             void *packed) {
    return guard([&] {
        TensorHandle *ha = static_cast<TensorHandle *>(a), *hb = static_cast<TensorHandle *>(b), *hc = static_cast<TensorHandle *>(c);
        PackedHandle *hp = static_cast<PackedHandle *>(packed);
        if (ha->dtype != hb->dtype || ha->dtype != hc->dtype || (hp && hp->dtype != ha->dtype))
            throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        if ((op_a != 0 && op_a != 1) || (op_b != 0 && op_b != 1)) throw Error(WK_E_INVALID_VALUE);
        dispatch(ha->dtype, [&]<typename T>() {
            blas::gemm<T>(static_cast<Pipeline *>(pipeline), opt_scalar<T>(host_alpha), static_cast<Tensor<T> *>(ha->tensor),
                          static_cast<Operation>(op_a), static_cast<Tensor<T> *>(hb->tensor), static_cast<Operation>(op_b),
                          opt_scalar<T>(host_beta), static_cast<Tensor<T> *>(hc->tensor),
                          hp ? static_cast<blas::PackedTensors<T> *>(hp->packed) : nullptr);
        });
    });
}

// The same two calls `count` times in a row from one loop in this library: what a C++ or Zig caller's loop does,
// for the benchmarks (from Python a call costs 4-5 us of interpreter and ctypes time, more than a short launch).
int wkz_axpy_repeat(void *pipeline, void *x, const void *host_alpha, void *y, uint32_t count) {
    int rc = 0;
    for (uint32_t i = 0; i < count && !rc; ++i) rc = wkz_axpy(pipeline, x, host_alpha, y);
    return rc;
}
int wkz_gemm_repeat(void *pipeline, const void *host_alpha, void *a, int op_a, void *b, int op_b, const void *host_beta, void *c,
                    void *packed, uint32_t count) {
    int rc = 0;
    for (uint32_t i = 0; i < count && !rc; ++i) rc = wkz_gemm(pipeline, host_alpha, a, op_a, b, op_b, host_beta, c, packed);
    return rc;
}

// ---- math ------------------------------------------------------------------------------------------
int wkz_math_dot(void *pipeline, void *x, void *y) {
    return guard([&] {
        TensorHandle *hx = static_cast<TensorHandle *>(x), *hy = static_cast<TensorHandle *>(y);
        if (hx->dtype != hy->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch_real(hx->dtype, [&]<typename T>() {
            math::dot<T>(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(hx->tensor), static_cast<Tensor<T> *>(hy->tensor));
        });
    });
}
static int reduce(void *pipeline, void *x, void *host_result, bool mean) {
    return guard([&] {
        TensorHandle *hx = static_cast<TensorHandle *>(x);
        if (!host_result) throw Error(WK_E_INVALID_VALUE);
        dispatch_real(hx->dtype, [&]<typename T>() {
            Tensor<T> *t = static_cast<Tensor<T> *>(hx->tensor);
            const T r = mean ? math::mean<T>(static_cast<Pipeline *>(pipeline), t) : math::sum<T>(static_cast<Pipeline *>(pipeline), t);
            std::memcpy(host_result, &r, sizeof(T));
        });
    });
}
int wkz_math_sum(void *pipeline, void *x, void *host_result) { return reduce(pipeline, x, host_result, false); }
int wkz_math_mean(void *pipeline, void *x, void *host_result) { return reduce(pipeline, x, host_result, true); }

// ---- nn: activations ---------------------------------------------------------------------------------
int wkz_nn_activation_run(int kind, void *pipeline, void *tensor) {
    return guard([&] {
        TensorHandle *h = static_cast<TensorHandle *>(tensor);
        dispatch_real(h->dtype, [&]<typename T>() {
            nn::Activation<T>{kind}.run(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(h->tensor));
        });
    });
}
int wkz_nn_activation_get_derivative(int kind, void *pipeline, void *output, void *derivative) {
    return guard([&] {
        TensorHandle *ho = static_cast<TensorHandle *>(output), *hd = static_cast<TensorHandle *>(derivative);
        if (ho->dtype != hd->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch_real(ho->dtype, [&]<typename T>() {
            nn::Activation<T>{kind}.getDerivative(static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(ho->tensor),
                                                  static_cast<Tensor<T> *>(hd->tensor));
        });
    });
}

// ---- nn: layers ------------------------------------------------------------------------------------------
// activation_kind: WK_ACT_NONE for a layer without activation; seed: NULL draws it from the clock
int wkz_nn_linear_init(void *ctx, void *pipeline, int dtype, uint64_t input, uint64_t output, int activation_kind, uint64_t deep,
                       int enable_bias, const uint64_t *seed, void **out) {
    return guard([&] {
        if (!out) throw Error(WK_E_INVALID_VALUE);
        if (activation_kind != WK_ACT_NONE && activation_kind != WK_ACT_SIGMOID && activation_kind != WK_ACT_TANH)
            throw Error(WK_E_INVALID_VALUE);
        dispatch_real(dtype, [&]<typename T>() {
            nn::ExtraParams extra;
            extra.deep = (size_t)deep;
            extra.enable_bias = enable_bias != 0;
            if (seed) extra.seed = *seed;
            std::optional<nn::Activation<T>> acti;
            if (activation_kind != WK_ACT_NONE) acti = nn::Activation<T>{activation_kind};
            nn::Layer<T> *l =
                nn::Linear<T>::init(static_cast<Context *>(ctx), static_cast<Pipeline *>(pipeline), input, output, acti, extra);
            *out = new LayerHandle{dtype, l};
        });
    });
}
int wkz_nn_sequential_init(int dtype, void **out) {
    return guard([&] {
        if (!out) throw Error(WK_E_INVALID_VALUE);
        dispatch_real(dtype, [&]<typename T>() {
            nn::Layer<T> *l = nn::Sequential<T>::init();
            *out = new LayerHandle{dtype, l};
        });
    });
}
// the sequence takes ownership of `layer`; its handle is consumed
int wkz_nn_sequential_append(void *sequential, void *layer) {
    return guard([&] {
        LayerHandle *hs = static_cast<LayerHandle *>(sequential), *hl = static_cast<LayerHandle *>(layer);
        if (hs->dtype != hl->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch_real(hs->dtype, [&]<typename T>() {
            auto *seq = dynamic_cast<nn::Sequential<T> *>(static_cast<nn::Layer<T> *>(hs->layer));
            if (!seq) throw Error(WK_E_INVALID_VALUE);
            seq->append(static_cast<nn::Layer<T> *>(hl->layer));
        });
        delete hl;
    });
}
int wkz_nn_layer_deinit(void *layer, void *pipeline) {
    return guard([&] {
        LayerHandle *h = static_cast<LayerHandle *>(layer);
        dispatch_real(h->dtype, [&]<typename T>() { static_cast<nn::Layer<T> *>(h->layer)->deinit(static_cast<Pipeline *>(pipeline)); });
        delete h;
    });
}
// Borrowed views of a layer's tensors.  which: 0 weights, 1 bias, 2 gradients, 3 bias gradients
// (2 and 3 need the layer's cache), 4 cached output, 5 sensitivity (index ignored).  *count
// receives the list length; *out a tensor handle to pass to wkz_tensor_handle_drop (never to
// wkz_tensor_release), or NULL for an absent bias.
int wkz_nn_layer_tensor(void *layer, void *layer_cache, int which, uint64_t index, uint64_t *count, void **out) {
    return guard([&] {
        LayerHandle *h = static_cast<LayerHandle *>(layer);
        if ((which >= 2 && !layer_cache) || which < 0 || which > 5) throw Error(WK_E_INVALID_VALUE);
        dispatch_real(h->dtype, [&]<typename T>() {
            nn::Layer<T> *l = static_cast<nn::Layer<T> *>(h->layer);
            std::vector<Tensor<T> *> list;
            switch (which) {
            case 0: list = l->getWeights(); break;
            case 1: list = l->getBias(); break;
            case 2: list = l->getGradients(layer_cache); break;
            case 3: list = l->getBiasGradients(layer_cache); break;
            case 4: list = {l->getCachedOutput(layer_cache)}; break;
            default: list = {l->getSensitivity(layer_cache)}; break;
            }
            if (count) *count = list.size();
            if (out) {
                if (index >= list.size()) throw Error(WK_E_INVALID_COORDINATES);
                *out = list[index] ? new TensorHandle{h->dtype, list[index]} : nullptr;
            }
        });
    });
}
void wkz_tensor_handle_drop(void *tensor) { delete static_cast<TensorHandle *>(tensor); }

int wkz_nn_layer_forward(void *layer, void *pipeline, void *input, void *layer_cache, void **out) {
    return guard([&] {
        LayerHandle *h = static_cast<LayerHandle *>(layer);
        TensorHandle *hi = static_cast<TensorHandle *>(input);
        if (hi->dtype != h->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        if (!layer_cache) throw Error(WK_E_INVALID_VALUE);
        dispatch_real(h->dtype, [&]<typename T>() {
            Tensor<T> *o = static_cast<nn::Layer<T> *>(h->layer)->forward(static_cast<Pipeline *>(pipeline),
                                                                          static_cast<Tensor<T> *>(hi->tensor), layer_cache);
            if (out) *out = new TensorHandle{h->dtype, o};
        });
    });
}
int wkz_nn_layer_backward(void *layer, void *pipeline, void *layer_cache, void *input, void *input_gradient) {
    return guard([&] {
        LayerHandle *h = static_cast<LayerHandle *>(layer);
        TensorHandle *hi = static_cast<TensorHandle *>(input), *hg = static_cast<TensorHandle *>(input_gradient);
        if (hi->dtype != h->dtype || (hg && hg->dtype != h->dtype)) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        if (!layer_cache) throw Error(WK_E_INVALID_VALUE);
        dispatch_real(h->dtype, [&]<typename T>() {
            static_cast<nn::Layer<T> *>(h->layer)->backward(static_cast<Pipeline *>(pipeline), layer_cache,
                                                            static_cast<Tensor<T> *>(hi->tensor),
                                                            hg ? static_cast<Tensor<T> *>(hg->tensor) : nullptr);
        });
    });
}

// ---- nn: cache, loss, optimizers ----------------------------------------------------------------------
int wkz_nn_cache_init(void *ctx, void *pipeline, uint64_t number_of_elements, void *const *layers, uint64_t num_layers, void **out) {
    return guard([&] {
        if (!out || !layers || num_layers == 0) throw Error(WK_E_INVALID_VALUE);
        const int dtype = static_cast<LayerHandle *>(layers[0])->dtype;
        for (uint64_t i = 1; i < num_layers; ++i)
            if (static_cast<LayerHandle *>(layers[i])->dtype != dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch_real(dtype, [&]<typename T>() {
            std::vector<const nn::Layer<T> *> list;
            for (uint64_t i = 0; i < num_layers; ++i) list.push_back(static_cast<nn::Layer<T> *>(static_cast<LayerHandle *>(layers[i])->layer));
            *out = new CacheHandle{
                dtype, nn::Cache<T>::init(static_cast<Context *>(ctx), static_cast<Pipeline *>(pipeline), number_of_elements, list)};
        });
    });
}
int wkz_nn_cache_deinit(void *cache, void *pipeline) {
    return guard([&] {
        CacheHandle *h = static_cast<CacheHandle *>(cache);
        dispatch_real(h->dtype, [&]<typename T>() { static_cast<nn::Cache<T> *>(h->cache)->deinit(static_cast<Pipeline *>(pipeline)); });
        delete h;
    });
}
void *wkz_nn_cache_get_layer_cache(void *cache, uint64_t index) {
    CacheHandle *h = static_cast<CacheHandle *>(cache);
    void *r = nullptr;
    guard([&] {
        dispatch_real(h->dtype, [&]<typename T>() {
            auto *c = static_cast<nn::Cache<T> *>(h->cache);
            if (index < c->slots.size()) r = c->getLayerCache((size_t)index);
        });
    });
    return r;
}
int wkz_nn_cache_error_tensor(void *cache, void **out) {
    return guard([&] {
        CacheHandle *h = static_cast<CacheHandle *>(cache);
        dispatch_real(h->dtype, [&]<typename T>() { *out = new TensorHandle{h->dtype, static_cast<nn::Cache<T> *>(h->cache)->error_tensor}; });
    });
}
// host_error_result may be NULL (no mean is computed, nothing synchronises)
int wkz_nn_loss_mse(int calculate_derivative, void *pipeline, void *output, void *expected, void *cache, void *host_error_result) {
    return guard([&] {
        CacheHandle *hc = static_cast<CacheHandle *>(cache);
        TensorHandle *ho = static_cast<TensorHandle *>(output), *he = static_cast<TensorHandle *>(expected);
        if (ho->dtype != hc->dtype || he->dtype != hc->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch_real(hc->dtype, [&]<typename T>() {
            T result{};
            nn::loss::mse<T>(calculate_derivative != 0, static_cast<Pipeline *>(pipeline), static_cast<Tensor<T> *>(ho->tensor),
                             static_cast<Tensor<T> *>(he->tensor), static_cast<nn::Cache<T> *>(hc->cache),
                             host_error_result ? &result : nullptr);
            if (host_error_result) std::memcpy(host_error_result, &result, sizeof(T));
        });
    });
}
int wkz_nn_gd_init(int dtype, double lr, void **out) {
    return guard([&] {
        if (!out) throw Error(WK_E_INVALID_VALUE);
        dispatch_real(dtype, [&]<typename T>() {
            nn::optimizers::Optimizer<T> *o = nn::optimizers::GD<T>::init((T)lr);
            *out = new OptimizerHandle{dtype, o};
        });
    });
}
// eps < 0 selects the default (the machine epsilon of the element type)
int wkz_nn_adam_init(int dtype, double lr, double beta1, double beta2, double eps, void **out) {
    return guard([&] {
        if (!out) throw Error(WK_E_INVALID_VALUE);
        dispatch_real(dtype, [&]<typename T>() {
            nn::optimizers::Optimizer<T> *o = nn::optimizers::Adam<T>::init(lr, beta1, beta2, eps);
            *out = new OptimizerHandle{dtype, o};
        });
    });
}
int wkz_nn_optimizer_step(void *optimizer, void *pipeline, void *cache) {
    return guard([&] {
        OptimizerHandle *h = static_cast<OptimizerHandle *>(optimizer);
        CacheHandle *hc = static_cast<CacheHandle *>(cache);
        if (hc->dtype != h->dtype) throw Error(WK_E_UNQUAL_TENSORS_ATTRIBUTE);
        dispatch_real(h->dtype, [&]<typename T>() {
            static_cast<nn::optimizers::Optimizer<T> *>(h->optimizer)->step(static_cast<Pipeline *>(pipeline), static_cast<nn::Cache<T> *>(hc->cache));
        });
    });
}
int wkz_nn_optimizer_zero(void *optimizer, void *pipeline) {
    return guard([&] {
        OptimizerHandle *h = static_cast<OptimizerHandle *>(optimizer);
        dispatch_real(h->dtype, [&]<typename T>() { static_cast<nn::optimizers::Optimizer<T> *>(h->optimizer)->zero(static_cast<Pipeline *>(pipeline)); });
    });
}
int wkz_nn_optimizer_deinit(void *optimizer, void *pipeline) {
    return guard([&] {
        OptimizerHandle *h = static_cast<OptimizerHandle *>(optimizer);
        dispatch_real(h->dtype, [&]<typename T>() { static_cast<nn::optimizers::Optimizer<T> *>(h->optimizer)->deinit(static_cast<Pipeline *>(pipeline)); });
        delete h;
    });
}

} // extern "C"
