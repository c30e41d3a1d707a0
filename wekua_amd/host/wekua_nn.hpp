// wekua_nn.hpp -- host-side mirror of the part of wekua's `nn` / `math` modules that one MLP
// training step uses, on top of wekua.hpp and the C ABI (include/wekua_hip.h):
//
//   wekua::math::dot / sum / mean       src/math/basic.zig:18-77,128-244
//   wekua::nn::Activation, Sigmoid, Tanh  src/nn/activation/{main,sigmoid,tanh}.zig
//   wekua::nn::Layer (interface)        src/nn/layer/main.zig:14-135
//   wekua::nn::Linear                   src/nn/layer/linear.zig
//   wekua::nn::Sequential               src/nn/layer/sequential.zig
//   wekua::nn::Cache                    src/nn/layer/cache.zig
//   wekua::nn::loss::mse                src/nn/loss/mse.zig:63-132
//   wekua::nn::optimizers::GD           src/nn/optimizers/gd.zig (w += -lr * g through blas.axpy)
//   wekua::nn::optimizers::Adam         no Zig counterpart (src/nn/optimizers/adam.zig is empty):
//                                       textbook Adam, see wk_adam_step
//
// Differences chosen for this device: bias add and activation run as one fused kernel after the
// forward GEMM (same arithmetic, one pass over the output instead of two); the Xavier-uniform
// weight initialisation is drawn on the host and uploaded (the reference seeds its device generator
// from the wall clock, linear.zig:125-132, so there is no reproducible stream to match) and takes
// an optional seed.
#pragma once

#include <chrono>
#include <cmath>
#include <limits>
#include <memory>

#include "wekua.hpp"

namespace wekua {

namespace math {
// x = x * y element-wise, in place (math.dot)
template <typename T> void dot(Pipeline *pipeline, Tensor<T> *x, Tensor<T> *y) {
    helpers::eqlTensorsShape<T>(x, y);
    const uint64_t shape3[3] = {x->depth(), x->rows(), x->cols()};
    check(wk_hadamard(pipeline->command_queue->stream, core::getTypeIndex<T>(), shape3, x->buffer, x->memory_layout.row_pitch,
                      x->memory_layout.slice_pitch, y->buffer, y->memory_layout.row_pitch, y->memory_layout.slice_pitch));
    pipeline->append(1);
}

// scale * sum of all logical elements, returned on the host (synchronises the pipeline, as
// math.sum / math.mean do: src/math/basic.zig:128-244)
template <typename T> T scaledSum(Pipeline *pipeline, Tensor<T> *x, double scale) {
    const Context *ctx = x->context;
    void *ws = nullptr, *res = nullptr;
    check(wk_malloc(ctx->device, wk_sum_workspace_bytes(core::getTypeIndex<T>()), &ws));
    int rc = wk_malloc(ctx->device, sizeof(T), &res);
    if (rc) {
        wk_free(ctx->device, ws);
        throw Error(rc);
    }
    const uint64_t shape3[3] = {x->depth(), x->rows(), x->cols()};
    T host = T(0);
    rc = wk_sum(pipeline->command_queue->stream, core::getTypeIndex<T>(), shape3, x->buffer, x->memory_layout.row_pitch,
                x->memory_layout.slice_pitch, ws, res, scale);
    if (!rc)
        rc = wk_copy_d2h_rect_async(pipeline->command_queue->stream, &host, sizeof(T), 0, res, sizeof(T), 0, sizeof(T), 1, 1);
    if (!rc) {
        pipeline->append(1);
        pipeline->waitAndCleanup();
    }
    wk_free(ctx->device, ws);
    wk_free(ctx->device, res);
    check(rc);
    return host;
}
template <typename T> T sum(Pipeline *pipeline, Tensor<T> *x) { return scaledSum<T>(pipeline, x, 1.0); }
template <typename T> T mean(Pipeline *pipeline, Tensor<T> *x) {
    return scaledSum<T>(pipeline, x, 1.0 / (double)x->dimensions.number_of_elements_without_padding);
}
} // namespace math

namespace nn {

// ---- activations ----------------------------------------------------------------------------
template <typename T> struct Activation {
    int kind = WK_ACT_NONE;
    // in place on the layer output (Activation.run)
    void run(Pipeline *pipeline, Tensor<T> *net_output) const {
        const uint64_t shape3[3] = {net_output->depth(), net_output->rows(), net_output->cols()};
        check(wk_activation(pipeline->command_queue->stream, core::getTypeIndex<T>(), kind, shape3, net_output->buffer,
                            net_output->memory_layout.row_pitch, net_output->memory_layout.slice_pitch));
        pipeline->append(1);
    }
    // derivative expressed through the activation output (Activation.getDerivative)
    void getDerivative(Pipeline *pipeline, Tensor<T> *output, Tensor<T> *derivative) const {
        helpers::eqlTensorsShape<T>(output, derivative);
        const uint64_t shape3[3] = {output->depth(), output->rows(), output->cols()};
        check(wk_activation_dev(pipeline->command_queue->stream, core::getTypeIndex<T>(), kind, shape3, output->buffer,
                                output->memory_layout.row_pitch, output->memory_layout.slice_pitch, derivative->buffer,
                                derivative->memory_layout.row_pitch, derivative->memory_layout.slice_pitch));
        pipeline->append(1);
    }
};
template <typename T> struct Sigmoid {
    static Activation<T> init() { return Activation<T>{WK_ACT_SIGMOID}; }
};
template <typename T> struct Tanh {
    static Activation<T> init() { return Activation<T>{WK_ACT_TANH}; }
};

// ---- Layer interface (src/nn/layer/main.zig: the vtable) ---------------------------------------
template <typename T> struct Layer {
    using TensorT = Tensor<T>;
    virtual ~Layer() = default;
    virtual void deinit(Pipeline *pipeline) = 0;
    virtual TensorT *getCachedOutput(const void *cache) const = 0;
    virtual std::vector<TensorT *> getWeights() const = 0;
    virtual std::vector<TensorT *> getBias() const = 0; // entries may be null
    virtual void *prepareCache(Pipeline *pipeline, uint64_t number_of_elements) const = 0;
    virtual void releaseCache(Pipeline *pipeline, void *cache) const = 0;
    virtual TensorT *forward(Pipeline *pipeline, TensorT *input, void *cache) const = 0;
    virtual TensorT *getSensitivity(const void *cache) const = 0;
    virtual void backward(Pipeline *pipeline, void *cache, TensorT *input, TensorT *input_gradient) const = 0;
    virtual std::vector<TensorT *> getGradients(const void *cache) const = 0;
    virtual std::vector<TensorT *> getBiasGradients(const void *cache) const = 0; // entries may be null
};

// ---- Linear ------------------------------------------------------------------------------------
struct ExtraParams {
    size_t deep = 1;         // src/nn/layer/linear.zig:23-26: extra {output, output} layers behind the first
    bool enable_bias = true;
    // Seed of the Xavier-uniform initialisation.  The reference seeds tensor.random.uniform from the
    // clock (linear.zig:125-132: seed == null); nullopt does the same here, a value makes it repeatable.
    std::optional<uint64_t> seed = std::nullopt;
};

namespace detail {
inline uint64_t splitmix64(uint64_t &state) {
    uint64_t z = (state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
// uniform in [-limit, limit), limit = sqrt(6 / (input + output))  (getRandomLimits, linear.zig:28-45)
template <typename T> void xavierUniform(Pipeline *pipeline, Tensor<T> *w, uint64_t input, uint64_t output, uint64_t &state) {
    const double limit = std::sqrt(6.0 / (double)(input + output));
    std::vector<T> host(w->dimensions.number_of_elements_without_padding);
    for (T &v : host) v = (T)((2.0 * ((double)(splitmix64(state) >> 11) * 0x1.0p-53) - 1.0) * limit);
    memory::readFromBuffer<T>(pipeline, w, host.data(), host.size());
    pipeline->waitAndCleanup(); // `host` dies with this scope
}
} // namespace detail

template <typename T> struct Linear : Layer<T> {
    using TensorT = Tensor<T>;
    struct LinearCache {
        std::vector<TensorT *> outputs, sensitivities, acti_derivatives, gradients, bias_gradients;
    };

    const Context *context = nullptr;
    std::vector<TensorT *> weights; // [0] is {output, input}, the rest {output, output}
    std::vector<TensorT *> bias;    // {output} each, or nulls when disabled
    bool bias_enabled = true;
    std::optional<Activation<T>> activation;

    // Linear.init (linear.zig:86-180)
    static Linear *init(const Context *context, Pipeline *pipeline, uint64_t input, uint64_t output,
                        std::optional<Activation<T>> acti, ExtraParams extra = {}) {
        if (input == 0 || output == 0 || extra.deep == 0) throw Error(WK_E_INVALID_VALUE);
        auto self = std::make_unique<Linear>();
        self->context = context;
        self->activation = acti;
        self->bias_enabled = extra.enable_bias;
        uint64_t state = extra.seed ? *extra.seed : (uint64_t)std::chrono::steady_clock::now().time_since_epoch().count();
        try {
            for (size_t i = 0; i < extra.deep; ++i) {
                const uint64_t in = i == 0 ? input : output;
                self->weights.push_back(TensorT::alloc(context, pipeline, {output, in}));
                detail::xavierUniform<T>(pipeline, self->weights.back(), in, output, state);
            }
            self->bias.assign(extra.deep, nullptr);
            if (extra.enable_bias)
                for (size_t i = 0; i < extra.deep; ++i) self->bias[i] = TensorT::alloc(context, pipeline, {output});
        } catch (...) {
            for (TensorT *t : self->weights) t->release(pipeline);
            for (TensorT *t : self->bias)
                if (t) t->release(pipeline);
            throw;
        }
        return self.release();
    }
    void deinit(Pipeline *pipeline) override {
        for (TensorT *t : weights) t->release(pipeline);
        for (TensorT *t : bias)
            if (t) t->release(pipeline);
        delete this;
    }
    TensorT *getCachedOutput(const void *cache) const override { return static_cast<const LinearCache *>(cache)->outputs.back(); }
    std::vector<TensorT *> getWeights() const override { return weights; }
    std::vector<TensorT *> getBias() const override { return bias; }

    // prepareCache (linear.zig:202-398): per-batch-size outputs, sensitivities (filled with one),
    // activation derivatives (zero), gradients and bias gradients
    void *prepareCache(Pipeline *pipeline, uint64_t number_of_elements) const override {
        if (number_of_elements == 0) throw Error(WK_E_INVALID_VALUE);
        auto c = std::make_unique<LinearCache>();
        try {
            for (size_t i = 0; i < weights.size(); ++i) {
                const auto &wshape = weights[i]->dimensions.shape;
                c->outputs.push_back(TensorT::alloc(context, pipeline, {number_of_elements, wshape[0]}));
                c->sensitivities.push_back(TensorT::alloc(context, pipeline, {number_of_elements, wshape[0]}));
                c->acti_derivatives.push_back(TensorT::alloc(context, pipeline, {number_of_elements, wshape[0]}));
                fill::one<T>(pipeline, c->sensitivities.back());
                c->gradients.push_back(TensorT::alloc(context, pipeline, wshape));
                c->bias_gradients.push_back(TensorT::alloc(context, pipeline, {wshape[0]}));
            }
        } catch (...) {
            releaseCache(pipeline, c.release());
            throw;
        }
        return c.release();
    }
    void releaseCache(Pipeline *pipeline, void *cache) const override {
        LinearCache *c = static_cast<LinearCache *>(cache);
        for (auto *list : {&c->outputs, &c->sensitivities, &c->acti_derivatives, &c->gradients, &c->bias_gradients})
            for (TensorT *t : *list) t->release(pipeline);
        delete c;
    }

    // forward (linear.zig:480-525): out = in * W^T, then addBias and the activation -- here one
    // call: bias and activation run in the epilogue of the matrix-core kernel
    TensorT *forward(Pipeline *pipeline, TensorT *input, void *cache) const override {
        LinearCache *c = static_cast<LinearCache *>(cache);
        for (size_t i = 0; i < weights.size(); ++i) {
            TensorT *out = c->outputs[i];
            blas::validateTensors<T>(input, weights[i], out, blas::Operation::no_transpose, blas::Operation::transpose);
            check(wk_gemm_bias_activation(pipeline->command_queue->stream, core::getTypeIndex<T>(), 0, 1, out->rows(), out->cols(),
                                          input->cols(), input->buffer, input->memory_layout.row_pitch, weights[i]->buffer,
                                          weights[i]->memory_layout.row_pitch, out->buffer, out->memory_layout.row_pitch,
                                          bias_enabled ? bias[i]->buffer : nullptr,
                                          activation ? activation->kind : WK_ACT_NONE));
            pipeline->append(1);
            input = out;
        }
        return input;
    }
    TensorT *getSensitivity(const void *cache) const override {
        return static_cast<const LinearCache *>(cache)->sensitivities.back();
    }

    // backward (linear.zig:579-678).  As there, the sensitivity is multiplied by the cached
    // derivative tensor even when the layer has no activation; that tensor then still holds the
    // zeros it was created with, so such a layer yields zero gradients.
    void backward(Pipeline *pipeline, void *cache, TensorT *input, TensorT *input_sensitivity) const override {
        LinearCache *c = static_cast<LinearCache *>(cache);
        TensorT *sens = c->sensitivities.back();
        for (size_t i = weights.size(); i-- > 0;) {
            TensorT *prev_output = i >= 1 ? c->outputs[i - 1] : input;
            // activation derivative from the cached output, Hadamard product into the sensitivity and the
            // bias gradient (column sums of the new sensitivity) in one pass over the layer's output
            TensorT *dev = c->acti_derivatives[i];
            helpers::eqlTensorsShape<T>(sens, dev);
            helpers::eqlTensorsShape<T>(sens, c->outputs[i]);
            check(wk_sensitivity_step(pipeline->command_queue->stream, core::getTypeIndex<T>(),
                                      activation ? activation->kind : WK_ACT_NONE, sens->rows(), sens->cols(), c->outputs[i]->buffer,
                                      c->outputs[i]->memory_layout.row_pitch, sens->buffer, sens->memory_layout.row_pitch, dev->buffer,
                                      dev->memory_layout.row_pitch, bias_enabled ? c->bias_gradients[i]->buffer : nullptr));
            pipeline->append(1);
            // weight gradient: sens^T [O,B] * prev_output [B,I]
            blas::gemm<T>(pipeline, std::nullopt, sens, blas::Operation::transpose, prev_output, blas::Operation::no_transpose,
                          std::nullopt, c->gradients[i], nullptr);
            TensorT *next = i >= 1 ? c->sensitivities[i - 1] : input_sensitivity;
            if (!next) return;
            // sensitivity of what feeds this matrix: sens [B,O] * W [O,I]
            blas::gemm<T>(pipeline, std::nullopt, sens, blas::Operation::no_transpose, weights[i], blas::Operation::no_transpose,
                          std::nullopt, next, nullptr);
            sens = next;
        }
    }
    std::vector<TensorT *> getGradients(const void *cache) const override {
        return static_cast<const LinearCache *>(cache)->gradients;
    }
    std::vector<TensorT *> getBiasGradients(const void *cache) const override {
        if (!bias_enabled) return std::vector<TensorT *>(weights.size(), nullptr);
        return static_cast<const LinearCache *>(cache)->bias_gradients;
    }
};

// ---- Sequential --------------------------------------------------------------------------------
template <typename T> struct Sequential : Layer<T> {
    using TensorT = Tensor<T>;
    struct SequentialCache {
        std::vector<void *> caches;
    };
    std::vector<Layer<T> *> layers; // owned

    // Sequential.init / append (sequential.zig:40-90): starts empty, owns what is appended
    static Sequential *init() { return new Sequential; }
    void append(Layer<T> *layer) { layers.push_back(layer); }
    void deinit(Pipeline *pipeline) override {
        for (Layer<T> *l : layers) l->deinit(pipeline);
        delete this;
    }
    TensorT *getCachedOutput(const void *cache) const override {
        const auto *c = static_cast<const SequentialCache *>(cache);
        return layers.back()->getCachedOutput(c->caches.back());
    }
    std::vector<TensorT *> getWeights() const override {
        std::vector<TensorT *> out;
        for (Layer<T> *l : layers)
            for (TensorT *w : l->getWeights()) out.push_back(w);
        return out;
    }
    std::vector<TensorT *> getBias() const override {
        std::vector<TensorT *> out;
        for (Layer<T> *l : layers)
            for (TensorT *b : l->getBias()) out.push_back(b);
        return out;
    }
    void *prepareCache(Pipeline *pipeline, uint64_t number_of_elements) const override {
        if (layers.empty()) throw Error(WK_E_INVALID_VALUE);
        auto c = std::make_unique<SequentialCache>();
        try {
            for (Layer<T> *l : layers) c->caches.push_back(l->prepareCache(pipeline, number_of_elements));
        } catch (...) {
            for (size_t i = 0; i < c->caches.size(); ++i) layers[i]->releaseCache(pipeline, c->caches[i]);
            throw;
        }
        return c.release();
    }
    void releaseCache(Pipeline *pipeline, void *cache) const override {
        auto *c = static_cast<SequentialCache *>(cache);
        for (size_t i = 0; i < layers.size(); ++i) layers[i]->releaseCache(pipeline, c->caches[i]);
        delete c;
    }
    // sequential.zig:214-230
    TensorT *forward(Pipeline *pipeline, TensorT *input, void *cache) const override {
        auto *c = static_cast<SequentialCache *>(cache);
        TensorT *out = input;
        for (size_t i = 0; i < layers.size(); ++i) out = layers[i]->forward(pipeline, out, c->caches[i]);
        return out;
    }
    TensorT *getSensitivity(const void *cache) const override {
        const auto *c = static_cast<const SequentialCache *>(cache);
        return layers.back()->getSensitivity(c->caches.back());
    }
    // sequential.zig:242-274: last layer to first; layer i's input is layer i-1's cached output and
    // its input gradient is layer i-1's sensitivity
    void backward(Pipeline *pipeline, void *cache, TensorT *input, TensorT *input_gradient) const override {
        auto *c = static_cast<SequentialCache *>(cache);
        for (size_t i = layers.size(); i-- > 0;) {
            TensorT *in = i == 0 ? input : layers[i - 1]->getCachedOutput(c->caches[i - 1]);
            TensorT *in_grad = i == 0 ? input_gradient : layers[i - 1]->getSensitivity(c->caches[i - 1]);
            layers[i]->backward(pipeline, c->caches[i], in, in_grad);
        }
    }
    std::vector<TensorT *> getGradients(const void *cache) const override {
        const auto *c = static_cast<const SequentialCache *>(cache);
        std::vector<TensorT *> out;
        for (size_t i = 0; i < layers.size(); ++i)
            for (TensorT *g : layers[i]->getGradients(c->caches[i])) out.push_back(g);
        return out;
    }
    std::vector<TensorT *> getBiasGradients(const void *cache) const override {
        const auto *c = static_cast<const SequentialCache *>(cache);
        std::vector<TensorT *> out;
        for (size_t i = 0; i < layers.size(); ++i)
            for (TensorT *g : layers[i]->getBiasGradients(c->caches[i])) out.push_back(g);
        return out;
    }
};

// ---- Cache (src/nn/layer/cache.zig) --------------------------------------------------------------
template <typename T> struct Cache {
    struct Slot {
        void *cache;
        const Layer<T> *layer;
    };
    std::vector<Slot> slots;
    Tensor<T> *error_tensor = nullptr;

    static Cache *init(const Context *context, Pipeline *pipeline, uint64_t number_of_elements,
                       const std::vector<const Layer<T> *> &layers) {
        if (layers.empty()) throw Error(WK_E_INVALID_VALUE);
        auto self = std::make_unique<Cache>();
        try {
            for (const Layer<T> *l : layers) self->slots.push_back({l->prepareCache(pipeline, number_of_elements), l});
            const Slot &last = self->slots.back();
            self->error_tensor = Tensor<T>::alloc(context, pipeline, last.layer->getSensitivity(last.cache)->dimensions.shape);
        } catch (...) {
            for (const Slot &s : self->slots) s.layer->releaseCache(pipeline, s.cache);
            throw;
        }
        return self.release();
    }
    void *getLayerCache(size_t index) const { return slots[index].cache; }
    void deinit(Pipeline *pipeline) {
        for (const Slot &s : slots) s.layer->releaseCache(pipeline, s.cache);
        error_tensor->release(pipeline);
        delete this;
    }
};

// ---- loss ------------------------------------------------------------------------------------------
namespace loss {
// mse (src/nn/loss/mse.zig:63-132): error_tensor = (expected - output)^2; with calculate_derivative
// the last layer's sensitivity receives -2 (expected - output); error_result, when wanted, is the
// mean of error_tensor (this synchronises the pipeline, as math.mean does).
template <typename T>
void mse(bool calculate_derivative, Pipeline *pipeline, Tensor<T> *output, Tensor<T> *expected, const Cache<T> *cache,
         T *error_result) {
    Tensor<T> *err = cache->error_tensor;
    helpers::eqlTensorsShape<T>(output, expected);
    helpers::eqlTensorsShape<T>(err, output);
    Tensor<T> *sens = nullptr;
    if (calculate_derivative) {
        const auto &last = cache->slots.back();
        sens = last.layer->getSensitivity(last.cache);
    }
    const uint64_t shape3[3] = {output->depth(), output->rows(), output->cols()};
    check(wk_mse(pipeline->command_queue->stream, core::getTypeIndex<T>(), shape3, output->buffer, output->memory_layout.row_pitch,
                 output->memory_layout.slice_pitch, expected->buffer, expected->memory_layout.row_pitch,
                 expected->memory_layout.slice_pitch, err->buffer, err->memory_layout.row_pitch, err->memory_layout.slice_pitch,
                 sens ? sens->buffer : nullptr, sens ? sens->memory_layout.row_pitch : 0, sens ? sens->memory_layout.slice_pitch : 0));
    pipeline->append(1);
    if (error_result) *error_result = math::mean<T>(pipeline, err);
}
} // namespace loss

// ---- optimizers ----------------------------------------------------------------------------------
namespace optimizers {
template <typename T> struct Optimizer {
    virtual ~Optimizer() = default;
    virtual void step(Pipeline *pipeline, const Cache<T> *cache) = 0;
    virtual void zero(Pipeline *pipeline) = 0;
    virtual void deinit(Pipeline *pipeline) = 0;
};

// GD (src/nn/optimizers/gd.zig): w += (-lr) * g with blas.axpy, weights then biases, slot by slot
template <typename T> struct GD : Optimizer<T> {
    T lr; // stored negated, as gd.zig:39 does
    static GD *init(T lr) {
        GD *o = new GD;
        o->lr = -lr;
        return o;
    }
    void step(Pipeline *pipeline, const Cache<T> *cache) override {
        for (const auto &slot : cache->slots) {
            auto w = slot.layer->getWeights();
            auto g = slot.layer->getGradients(slot.cache);
            for (size_t i = 0; i < w.size(); ++i) blas::axpy<T>(pipeline, g[i], lr, w[i]);
            auto b = slot.layer->getBias();
            auto bg = slot.layer->getBiasGradients(slot.cache);
            for (size_t i = 0; i < b.size(); ++i)
                if (b[i] && bg[i]) blas::axpy<T>(pipeline, bg[i], lr, b[i]);
        }
    }
    void zero(Pipeline *) override {}
    void deinit(Pipeline *) override { delete this; }
};

// Adam: first/second moment tensors are created lazily with the shape of each parameter.
template <typename T> struct Adam : Optimizer<T> {
    double lr = 1e-3, beta1 = 0.9, beta2 = 0.999, eps = 0.0;
    uint64_t t = 0;
    std::vector<std::pair<Tensor<T> *, Tensor<T> *>> state; // (m, v) per parameter, in visiting order

    static Adam *init(double lr, double beta1 = 0.9, double beta2 = 0.999, double eps = -1.0) {
        Adam *o = new Adam;
        o->lr = lr;
        o->beta1 = beta1;
        o->beta2 = beta2;
        o->eps = eps >= 0.0 ? eps : (double)std::numeric_limits<T>::epsilon(); // the siblings' +FLT_EPSILON (rmsprop.cl:54)
        return o;
    }
    // one parameter tensor's entry of the step's update list (its moments are created on first sight)
    void collect(Pipeline *pipeline, size_t &index, Tensor<T> *w, Tensor<T> *g, std::vector<wk_adam_tensor> &list) {
        if (index == state.size()) {
            Tensor<T> *m = Tensor<T>::alloc(w->context, pipeline, w->dimensions.shape);
            Tensor<T> *v = nullptr;
            try {
                v = Tensor<T>::alloc(w->context, pipeline, w->dimensions.shape);
            } catch (...) {
                m->release(pipeline);
                throw;
            }
            state.push_back({m, v});
        }
        Tensor<T> *m = state[index].first, *v = state[index].second;
        helpers::eqlTensorsShape<T>(w, g);
        helpers::eqlTensorsShape<T>(w, m);
        wk_adam_tensor t{};
        t.w = w->buffer; t.g = g->buffer; t.m = m->buffer; t.v = v->buffer;
        t.shape3[0] = w->depth(); t.shape3[1] = w->rows(); t.shape3[2] = w->cols();
        t.w_row_pitch = w->memory_layout.row_pitch; t.w_slice_pitch = w->memory_layout.slice_pitch;
        t.g_row_pitch = g->memory_layout.row_pitch; t.g_slice_pitch = g->memory_layout.slice_pitch;
        t.mv_row_pitch = m->memory_layout.row_pitch; t.mv_slice_pitch = m->memory_layout.slice_pitch;
        list.push_back(t);
        ++index;
    }
    void step(Pipeline *pipeline, const Cache<T> *cache) override {
        ++t;
        size_t index = 0;
        std::vector<wk_adam_tensor> list;
        for (const auto &slot : cache->slots) {
            auto w = slot.layer->getWeights();
            auto g = slot.layer->getGradients(slot.cache);
            for (size_t i = 0; i < w.size(); ++i) collect(pipeline, index, w[i], g[i], list);
            auto b = slot.layer->getBias();
            auto bg = slot.layer->getBiasGradients(slot.cache);
            for (size_t i = 0; i < b.size(); ++i)
                if (b[i] && bg[i]) collect(pipeline, index, b[i], bg[i], list);
        }
        check(wk_adam_step_multi(pipeline->command_queue->stream, core::getTypeIndex<T>(), (uint32_t)list.size(), list.data(), lr, beta1,
                                 beta2, eps, t));
        pipeline->append(1);
    }
    void zero(Pipeline *pipeline) override {
        for (auto &mv : state) {
            fill::zeroes<T>(pipeline, mv.first);
            fill::zeroes<T>(pipeline, mv.second);
        }
        t = 0;
    }
    void deinit(Pipeline *pipeline) override {
        for (auto &mv : state) {
            mv.first->release(pipeline);
            mv.second->release(pipeline);
        }
        delete this;
    }
};
} // namespace optimizers

} // namespace nn
} // namespace wekua
