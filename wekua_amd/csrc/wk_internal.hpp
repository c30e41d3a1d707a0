// Internal declarations shared by the HIP translation units of libwekua_hip.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "wekua_hip.h"
#include "wekua_hip_test.h"

struct wk_device {
    int ordinal;
    hipDeviceProp_t props;
};

struct wk_stream {
    wk_device *dev;
    hipStream_t stream;
    // Device memory for partial results of two-pass reductions launched on this stream (the
    // stream is in order, so consecutive users never overlap).  Allocated with the stream.
    void *scratch;
    size_t scratch_bytes;
    // Arrival counters of the GEMM that splits k over work-groups: one per tile of C, zero between
    // launches (the work-group that arrives last at its tile's counter puts it back to zero).
    uint32_t *gemm_counters;
};

constexpr size_t WK_STREAM_SCRATCH_BYTES = 128u << 20;
constexpr size_t WK_GEMM_COUNTERS = 4096;
// what wk_bias_step uses of the scratch: the number of row bands, and with it the order of the
// additions, follows from this size, so it stays what it was when the scratch was this small
constexpr size_t WK_BIAS_STEP_SCRATCH_BYTES = 1u << 20;

struct wk_event {
    wk_device *dev;
    hipEvent_t event;
};

namespace wk {

// Switches of wk_test_option (wekua_hip_test.h): process-wide, set by tests and benchmarks only.
struct TestOptions {
    int gemm_walk_rows = 0; // 1: the direct-to-LDS kernels walk the tiles in groups of rows, not XCD-local patches
    int tail_strict = 0;    // 1: forced k-split tail variants plan like the automatic choice
    int alloc_colours = 1;  // 0: wk_malloc hands out blocks as hipMalloc returns them
    int stream_k = 1;       // 0: the automatic choice never deals work by k-slabs; 2: every tile dealt, none run whole; 3: whole rounds always run whole
    int persistent = 1;     // 0: a launch of more tiles than are resident is one work-group per tile, placed by the dispatcher; 2: never
    int skinny = 1;         // 0: products of at most 32 rows or columns go to the tile kernels; n >= 2: n work-groups per unit
    int strips = 1;         // 0: products are never multiplied in parts; 2: thin strips split off whatever the model says
};
extern TestOptions g_test_options;

inline int hip_code(hipError_t e) {
    if (e == hipSuccess) return WK_OK;
    if (e == hipErrorOutOfMemory) return WK_E_OUT_OF_MEMORY;
    return WK_E_HIP_BASE + static_cast<int>(e);
}

#define WK_HIP_TRY(expr)                                  \
    do {                                                  \
        hipError_t wk_e_ = (expr);                        \
        if (wk_e_ != hipSuccess) {                        \
            (void)hipGetLastError();                      \
            return ::wk::hip_code(wk_e_);                 \
        }                                                 \
    } while (0)

// Every launch is followed by this: a bad launch configuration surfaces here, not later.
inline int launch_status() { return hip_code(hipGetLastError()); }

// Looks up this device's address of the static scratch array of wk_bias_step_static (wk_nn.hip);
// wk_device_open calls it with the device current.
int static_scratch_setup(int ordinal);

// The arrival counters are only zero between launches when every counting kernel ran to its end; after
// a launch or a wait on the stream has failed they are put back to zero.
inline void reset_gemm_counters(wk_stream *s) {
    if (!s || !s->gemm_counters) return;
    (void)hipMemsetAsync(s->gemm_counters, 0, WK_GEMM_COUNTERS * sizeof(uint32_t), s->stream);
    (void)hipGetLastError();
}

inline int bind(wk_stream *s) {
    if (!s || !s->dev) return WK_E_INVALID_VALUE;
    WK_HIP_TRY(hipSetDevice(s->dev->ordinal));
    return WK_OK;
}

// ---- element types -------------------------------------------------------------------
// Integer dtypes are computed in the unsigned type of the same width: +, -, * modulo 2^w
// do not depend on signedness, and unsigned overflow is defined.  This is the wraparound
// of the reference's OpenCL kernels (i8/i16 promote to int there and truncate on store:
// the same low bits).
template <typename R>
struct cplx {
    R re, im;
};

template <typename T> struct elem_traits;
#define WK_REAL_TRAITS(T_, ACC_, ISF_)                                               \
    template <> struct elem_traits<T_> {                                             \
        using real = T_;                                                             \
        using acc = ACC_; /* accumulator: 32-bit for narrow ints, else same type */  \
        static constexpr bool is_complex = false;                                    \
        static constexpr bool is_float = ISF_;                                       \
    };
WK_REAL_TRAITS(uint8_t, uint32_t, false)
WK_REAL_TRAITS(uint16_t, uint32_t, false)
WK_REAL_TRAITS(uint32_t, uint32_t, false)
WK_REAL_TRAITS(uint64_t, uint64_t, false)
WK_REAL_TRAITS(float, float, true)
WK_REAL_TRAITS(double, double, true)
#undef WK_REAL_TRAITS
template <typename R> struct elem_traits<cplx<R>> {
    using real = R;
    using acc = cplx<typename elem_traits<R>::acc>;
    static constexpr bool is_complex = true;
    static constexpr bool is_float = elem_traits<R>::is_float;
};

template <typename A> __host__ __device__ inline A zero_of() { return A(0); }
template <> __host__ __device__ inline cplx<uint32_t> zero_of<cplx<uint32_t>>() { return {0u, 0u}; }
template <> __host__ __device__ inline cplx<uint64_t> zero_of<cplx<uint64_t>>() { return {0ull, 0ull}; }
template <> __host__ __device__ inline cplx<float> zero_of<cplx<float>>() { return {0.f, 0.f}; }
template <> __host__ __device__ inline cplx<double> zero_of<cplx<double>>() { return {0., 0.}; }

// widen / narrow between storage and accumulator types
template <typename A, typename T> __host__ __device__ inline A widen(T v) { return static_cast<A>(v); }
template <typename A, typename R> __host__ __device__ inline A widen(cplx<R> v) {
    return A{static_cast<decltype(A::re)>(v.re), static_cast<decltype(A::im)>(v.im)};
}
template <typename T, typename A> __host__ __device__ inline T narrow(A v) { return static_cast<T>(v); }
template <typename T, typename R> __host__ __device__ inline T narrow(cplx<R> v) {
    return T{static_cast<decltype(T::re)>(v.re), static_cast<decltype(T::im)>(v.im)};
}

template <typename A> __host__ __device__ inline A add(A a, A b) { return a + b; }
template <typename R> __host__ __device__ inline cplx<R> add(cplx<R> a, cplx<R> b) { return {a.re + b.re, a.im + b.im}; }
template <typename A> __host__ __device__ inline A sub(A a, A b) { return a - b; }
template <typename R> __host__ __device__ inline cplx<R> sub(cplx<R> a, cplx<R> b) { return {a.re - b.re, a.im - b.im}; }
template <typename A> __host__ __device__ inline A mul(A a, A b) { return a * b; }
// The reference's complex product (src/core/wekua_cl_lib.cl:648-653): three multiplies.
// Kept in this form so float rounding stays close to the reference's; for integers it is
// the ordinary product modulo 2^w.
template <typename R> __host__ __device__ inline cplx<R> mul(cplx<R> a, cplx<R> b) {
    const R k1 = b.re * (a.re + a.im);
    const R k2 = a.re * (b.im - b.re);
    const R k3 = a.im * (b.re + b.im);
    return {k1 - k3, k1 + k2};
}
// acc += a*b
template <typename A> __host__ __device__ inline A mad(A a, A b, A c) { return a * b + c; }
template <> __host__ __device__ inline float mad<float>(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
template <> __host__ __device__ inline double mad<double>(double a, double b, double c) { return __builtin_fma(a, b, c); }
template <typename R> __host__ __device__ inline cplx<R> mad(cplx<R> a, cplx<R> b, cplx<R> c) { return add(c, mul(a, b)); }

// dtype id -> run F.template operator()<T>() with the computational element type.
template <typename F> inline int dispatch_dtype(int dtype, F &&f) {
    switch (dtype) {
    case WK_I8: case WK_U8:   return f.template operator()<uint8_t>();
    case WK_I16: case WK_U16: return f.template operator()<uint16_t>();
    case WK_I32: case WK_U32: return f.template operator()<uint32_t>();
    case WK_I64: case WK_U64: return f.template operator()<uint64_t>();
    case WK_F32:              return f.template operator()<float>();
    case WK_F64:              return f.template operator()<double>();
    case WK_COMPLEX + WK_I8: case WK_COMPLEX + WK_U8:   return f.template operator()<cplx<uint8_t>>();
    case WK_COMPLEX + WK_I16: case WK_COMPLEX + WK_U16: return f.template operator()<cplx<uint16_t>>();
    case WK_COMPLEX + WK_I32: case WK_COMPLEX + WK_U32: return f.template operator()<cplx<uint32_t>>();
    case WK_COMPLEX + WK_I64: case WK_COMPLEX + WK_U64: return f.template operator()<cplx<uint64_t>>();
    case WK_COMPLEX + WK_F32: return f.template operator()<cplx<float>>();
    case WK_COMPLEX + WK_F64: return f.template operator()<cplx<double>>();
    default: return WK_E_TYPE_NOT_SUPPORTED;
    }
}

inline bool dtype_is_signed(int dtype) {
    const int r = dtype % 10;
    return r == WK_I8 || r == WK_I16 || r == WK_I32 || r == WK_I64 || r == WK_F32 || r == WK_F64;
}

// ---- gemm plumbing shared between wk_gemm.hip and the kernel files ------------------------
enum : int { EPI_STORE = 0, EPI_ALPHA = 1, EPI_ALPHA_BETA = 2 };

struct GemmProblem {
    int dtype, op_a, op_b;
    uint64_t M, N, K, lda, ldb, ldc;
    const void *A, *B;
    void *C;
    int epi;                          // EPI_*
    uint32_t num_cus;                 // compute units of the device the stream belongs to
    alignas(16) unsigned char alpha[16];  // one element of dtype (valid when epi != EPI_STORE)
    alignas(16) unsigned char beta[16];   // one element of dtype (valid when epi == EPI_ALPHA_BETA)
    // fused epilogue of Linear.forward: C = act(op(A)op(B) + bias[col]); only the f32 / f64 matrix-core
    // kernels for op N, T carry it (gemm_mfma_fuses)
    bool ext = false;
    const void *ext_bias = nullptr;   // N elements of dtype, or null
    int ext_act = -1;                 // WK_ACT_*
    // the workspace still holds op(B)'s packed form from the previous call (wk_gemm_packed_b_kept)
    bool reuse_b = false;
    // for kernels that split k over work-groups: device memory for the partial tiles and the tiles'
    // arrival counters (the stream's; null: such kernels are not chosen, and refuse when forced)
    void *scratch = nullptr;
    size_t scratch_bytes = 0;
    uint32_t *counters = nullptr;
    size_t num_counters = 0;
};

// How a launch that splits k over work-groups is laid out; host arithmetic only.
struct GemmSplitPlan {
    uint32_t shares = 1;   // work-groups per tile of C (grid y); 1: no split
    uint32_t klen = 0;     // k values per share, a multiple of the kernel's k-slab; the last share takes what is left
    uint64_t tiles = 0;    // tiles of C whose k is split (grid x) = arrival counters used
    uint64_t first_tile = 0; // their first tile number: the tiles before it are launched unsplit (0: every tile is split)
    size_t bytes = 0;      // partial tiles: shares * tiles * tile area * element size
};
// Plan for `variant` (a split-k variant) on p.  forced: split whenever k holds two slabs, whatever the
// number of tiles (tests); otherwise only when the tiles leave half the compute units idle and every
// share keeps a few slabs.  Returns false when the variant does not split or the plan does not fit
// p.scratch_bytes / p.num_counters (a null p.scratch or p.counters also fails).
bool gemm_mfma_split_plan(const GemmProblem &p, int variant, bool forced, GemmSplitPlan &plan);

// generic LDS-tiled VALU kernel, every dtype and shape (wk_gemm_generic.hip)
int gemm_generic_launch(hipStream_t st, const GemmProblem &p);
// MFMA kernels for f32 / f64 / i32 / u32 (wk_gemm_mfma.hip); `variant` indexes mfma_variant_name()
int gemm_mfma_launch(hipStream_t st, const GemmProblem &p, int variant);
// i32 / u32 on the int8 matrix cores (wk_gemm_imfma.hip); reached through the variant table
int gemm_i32_mfma_launch_64(hipStream_t st, const GemmProblem &p, bool edge);  // macro tile 64 x 128
int gemm_i32_mfma_launch_128(hipStream_t st, const GemmProblem &p, bool edge); // macro tile 128 x 128
// 8/16/32-bit integers with a pack pass into caller-provided workspace (wk_gemm_ipack.hip)
size_t gemm_int_packed_workspace_bytes(int dtype, uint64_t M, uint64_t N, uint64_t K); // 0: not applicable
int gemm_int_packed_launch(hipStream_t st, const GemmProblem &p, void *workspace, size_t workspace_bytes);
// 64-bit integers the same way: eight digit planes, 36 digit products (wk_gemm_i64pack.hip)
size_t gemm_i64_packed_workspace_bytes(uint64_t M, uint64_t N, uint64_t K); // 0: not applicable
int gemm_i64_packed_launch(hipStream_t st, const GemmProblem &p, void *workspace, size_t workspace_bytes);
constexpr int WK_CF32 = WK_COMPLEX + WK_F32, WK_CF64 = WK_COMPLEX + WK_F64;
// cf32 / cf64 and the complex 8/16/32-bit integers through the real matrix-core kernels, operands
// rebuilt in caller-provided workspace (wk_gemm_cpack.hip)
size_t gemm_complex_packed_workspace_bytes(int dtype, uint64_t M, uint64_t N, uint64_t K); // 0: not applicable
int gemm_complex_packed_prepare(hipStream_t st, const GemmProblem &p, void *workspace, size_t workspace_bytes,
                                int (*transpose)(void *ctx, int dtype, uint64_t rows, uint64_t cols, const void *src, uint64_t ld,
                                                 void *dst),
                                void *ctx, GemmProblem &real, void **rest, size_t *rest_bytes);
// f32, interior shapes only: k-slabs brought straight from global memory into LDS, three deep
// (wk_gemm_dma.hip); macro tiles 256 x 128, 128 x 128 and 64 x 64; the fused bias + activation epilogue
// (p.ext) for op N, T.  first_tiles: launch only the first so many tiles of the tile walk (0: all), for
// a product whose other tiles run as a k-split tail.
bool gemm_f32_dma_applies(const GemmProblem &p, int bm, int bn);
// the same kernels with the work dealt to compute units x occ work-groups by k-slabs instead of by tiles
// (parts of tiles meet in p.scratch, counted on p.counters): for products whose tiles do not fill whole rounds
bool gemm_f32_dma_stream_k_applies(const GemmProblem &p, int bm, int bn);
int gemm_f32_dma_stream_k_launch(hipStream_t st, const GemmProblem &p, int bm, int bn);
bool gemm_f64_dma_stream_k_applies(const GemmProblem &p, int bm, int bn);
// rows of both f64 operands start on 16-byte boundaries
bool gemm_f64_rows_aligned(const GemmProblem &p);
// how a launch that deals k-slabs shares its work (wk_gemm_dma.hip); false: the problem does not fit
bool gemm_dma_stream_k_plan(const GemmProblem &p, int bm, int bn, int bk, int occ, unsigned &groups, uint32_t &units, uint32_t &total,
                            uint32_t &first);
int gemm_f64_dma_stream_k_launch(hipStream_t st, const GemmProblem &p, int bm, int bn);
bool gemm_dma_rows_aligned(const GemmProblem &p); // 16-byte loads (else 4-byte ones: one group of wavefronts, no fused epilogue)
int gemm_f32_dma_launch(hipStream_t st, const GemmProblem &p, int bm, int bn, uint64_t first_tiles = 0, int k_groups = 1);
// the same for f64: macro tiles 128 x 128 (k-slabs of 8) and 64 x 64 (k-slabs of 16)
bool gemm_f64_dma_applies(const GemmProblem &p, int bm, int bn);
int gemm_f64_dma_launch(hipStream_t st, const GemmProblem &p, int bm, int bn);
bool gemm_mfma_fuses(const GemmProblem &p, int variant); // variant can run p with the fused bias + activation epilogue
// f32 / f64 products with at most four rows or columns of C (wk_gemm_thin.hip)
bool gemm_thin_applies(const GemmProblem &p);
int gemm_thin_launch(hipStream_t st, const GemmProblem &p);
// f32 / f64 products with at most 32 rows or columns of C and a large other operand (wk_gemm_skinny.hip);
// every layout, and the fused bias + activation epilogue of Linear.forward in every layout
bool gemm_skinny_applies(const GemmProblem &p);
int gemm_skinny_launch(hipStream_t st, const GemmProblem &p);
int gemm_mfma_pick(const GemmProblem &p, double *cost = nullptr); // -1: not applicable; cost: the model's figure for
                                                              // the chosen tile (rounds x tile area / efficiency; times k
                                                              // proportional to the launch's time: 3.05e5 per us in f32)
const char *gemm_mfma_variant_name(int variant); // nullptr past the end
int gemm_mfma_variant_dtype(int variant);


#ifdef __HIPCC__
// activation of nn.activation.{Sigmoid,Tanh} (src/nn/activation/kernels/{sigmoid,tanh}.cl), shared by
// the element-wise kernels and the fused GEMM epilogue so that both give the same bits
template <typename T> __device__ __forceinline__ T act_forward(int kind, T x) {
    if (kind == WK_ACT_SIGMOID) return T(1) / (T(1) + exp(-x));
    if (kind == WK_ACT_TANH) return tanh(x);
    return x;
}
#endif

} // namespace wk
