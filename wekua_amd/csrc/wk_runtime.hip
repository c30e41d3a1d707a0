// Device, stream, memory and the small support kernels (fill, identity, calibration copy).
// Replaces what src/core/{context,command_queue,pipeline}.zig and src/tensor/{fill,identity,
// memory/*}.zig obtain from OpenCL.
#include "wk_internal.hpp"

#include <cstdio>
#include <cstring>
#include <cstdlib>
#include <mutex>
#include <new>
#include <unordered_map>

using namespace wk;

wk::TestOptions wk::g_test_options;

int wk_test_option(const char *name, int value) {
    if (!name) return WK_E_INVALID_VALUE;
    if (std::strcmp(name, "gemm_walk_rows") == 0) g_test_options.gemm_walk_rows = value;
    else if (std::strcmp(name, "tail_strict") == 0) g_test_options.tail_strict = value;
    else if (std::strcmp(name, "alloc_colours") == 0) g_test_options.alloc_colours = value;
    else if (std::strcmp(name, "stream_k") == 0) g_test_options.stream_k = value;
    else if (std::strcmp(name, "strips") == 0) g_test_options.strips = value;
    else if (std::strcmp(name, "skinny") == 0) g_test_options.skinny = value;
    else if (std::strcmp(name, "persistent") == 0) g_test_options.persistent = value;
    else return WK_E_INVALID_VALUE;
    return WK_OK;
}

extern "C" {

const char *wk_strerror(int code) {
    switch (code) {
    case WK_OK: return "ok";
    case WK_E_INVALID_VALUE: return "InvalidValue";
    case WK_E_INVALID_COORDINATES: return "InvalidCoordinates";
    case WK_E_INVALID_BUFFER: return "InvalidBuffer";
    case WK_E_UNQUAL_TENSORS_ATTRIBUTE: return "UnqualTensorsAttribute";
    case WK_E_UNQUAL_TENSORS_SHAPE: return "UnqualTensorsShape";
    case WK_E_UNQUAL_TENSORS_DIMENSION: return "UnqualTensorsDimension";
    case WK_E_UNQUAL_TENSORS_CONTEXT: return "UnqualTensorsContext";
    case WK_E_OUT_OF_MEMORY: return "OutOfMemory";
    case WK_E_TYPE_NOT_SUPPORTED: return "TypeNotSupported";
    case WK_E_NO_DEVICE: return "DevicesArrayEmpty";
    case WK_E_SCRATCH_TOO_SMALL: return "ScratchTooSmall: the operand exceeds the fixed scratch array of this entry point";
    default: break;
    }
    if (code >= WK_E_HIP_BASE) return hipGetErrorString(static_cast<hipError_t>(code - WK_E_HIP_BASE));
    return "unknown wekua_hip error";
}

int wk_abi_version(void) { return WK_ABI_VERSION; }

size_t wk_dtype_size(int dtype) {
    static const size_t real_size[10] = {1, 1, 2, 2, 4, 4, 8, 8, 4, 8};
    if (dtype < 0 || dtype >= WK_DTYPE_COUNT) return 0;
    return dtype >= WK_COMPLEX ? 2 * real_size[dtype - WK_COMPLEX] : real_size[dtype];
}

int wk_device_count(int *out_count) {
    if (!out_count) return WK_E_INVALID_VALUE;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        *out_count = 0;
        return e == hipErrorNoDevice ? WK_OK : hip_code(e);
    }
    *out_count = n;
    return WK_OK;
}

int wk_device_open(int ordinal, wk_device **out) {
    if (!out) return WK_E_INVALID_VALUE;
    *out = nullptr;
    int n = 0;
    int rc = wk_device_count(&n);
    if (rc) return rc;
    if (n == 0) return WK_E_NO_DEVICE;
    if (ordinal < 0 || ordinal >= n) return WK_E_INVALID_VALUE;
    wk_device *d = new (std::nothrow) wk_device;
    if (!d) return WK_E_OUT_OF_MEMORY;
    d->ordinal = ordinal;
    hipError_t e = hipGetDeviceProperties(&d->props, ordinal);
    if (e == hipSuccess) e = hipSetDevice(ordinal);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        delete d;
        return hip_code(e);
    }
    // only wk_bias_step_static needs the array: without its address that entry point reports the error
    // itself and everything else works
    (void)static_scratch_setup(ordinal);
    *out = d;
    return WK_OK;
}

void wk_device_close(wk_device *dev) { delete dev; }

int wk_device_props(wk_device *dev, wk_props *out) {
    if (!dev || !out) return WK_E_INVALID_VALUE;
    std::memset(out, 0, sizeof *out);
    std::snprintf(out->name, sizeof out->name, "%s", dev->props.name);
    std::snprintf(out->arch, sizeof out->arch, "%s", dev->props.gcnArchName);
    out->ordinal = dev->ordinal;
    out->compute_units = dev->props.multiProcessorCount;
    out->wavefront_size = dev->props.warpSize;
    out->max_work_group_size = dev->props.maxThreadsPerBlock;
    out->local_mem_bytes = dev->props.sharedMemPerBlock;
    out->global_mem_bytes = dev->props.totalGlobalMem;
    out->cache_line_size = 128;
    out->clock_mhz = dev->props.clockRate / 1000;
    return WK_OK;
}

int wk_stream_create(wk_device *dev, wk_stream **out) {
    if (!dev || !out) return WK_E_INVALID_VALUE;
    *out = nullptr;
    WK_HIP_TRY(hipSetDevice(dev->ordinal));
    wk_stream *s = new (std::nothrow) wk_stream;
    if (!s) return WK_E_OUT_OF_MEMORY;
    s->dev = dev;
    s->scratch = nullptr;
    s->scratch_bytes = 0;
    s->gemm_counters = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        delete s;
        return hip_code(e);
    }
    // the large scratch serves the k-split products; when the device cannot spare it the stream still
    // works with the small one (split plans that do not fit are simply not chosen)
    s->scratch_bytes = WK_STREAM_SCRATCH_BYTES;
    e = hipMalloc(&s->scratch, s->scratch_bytes);
    if (e == hipErrorOutOfMemory) {
        (void)hipGetLastError();
        s->scratch_bytes = WK_BIAS_STEP_SCRATCH_BYTES;
        e = hipMalloc(&s->scratch, s->scratch_bytes);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        (void)hipStreamDestroy(s->stream);
        delete s;
        return hip_code(e);
    }
    // arrival counters: zero from here on, every kernel that counts on them leaves them at zero
    e = hipMalloc(reinterpret_cast<void **>(&s->gemm_counters), WK_GEMM_COUNTERS * sizeof(uint32_t));
    // cleared on the stream itself, so that every later launch on it is ordered behind the clear
    if (e == hipSuccess) e = hipMemsetAsync(s->gemm_counters, 0, WK_GEMM_COUNTERS * sizeof(uint32_t), s->stream);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        if (s->gemm_counters) (void)hipFree(s->gemm_counters);
        (void)hipFree(s->scratch);
        (void)hipStreamDestroy(s->stream);
        delete s;
        return hip_code(e);
    }
    *out = s;
    return WK_OK;
}

void wk_stream_destroy(wk_stream *s) {
    if (!s) return;
    if (hipSetDevice(s->dev->ordinal) == hipSuccess) {
        (void)hipStreamSynchronize(s->stream);
        (void)hipStreamDestroy(s->stream);
        if (s->scratch) (void)hipFree(s->scratch);
        if (s->gemm_counters) (void)hipFree(s->gemm_counters);
    }
    (void)hipGetLastError();
    delete s;
}

int wk_stream_sync(wk_stream *s) {
    int rc = bind(s);
    if (rc) return rc;
    hipError_t e = hipStreamSynchronize(s->stream);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        reset_gemm_counters(s);
        return hip_code(e);
    }
    return WK_OK;
}

void *wk_stream_native(wk_stream *s) { return s ? static_cast<void *>(s->stream) : nullptr; }

int wk_event_create(wk_device *dev, wk_event **out) {
    if (!dev || !out) return WK_E_INVALID_VALUE;
    *out = nullptr;
    WK_HIP_TRY(hipSetDevice(dev->ordinal));
    wk_event *e = new (std::nothrow) wk_event;
    if (!e) return WK_E_OUT_OF_MEMORY;
    e->dev = dev;
    hipError_t rc = hipEventCreate(&e->event);
    if (rc != hipSuccess) {
        (void)hipGetLastError();
        delete e;
        return hip_code(rc);
    }
    *out = e;
    return WK_OK;
}

void wk_event_destroy(wk_event *e) {
    if (!e) return;
    if (hipSetDevice(e->dev->ordinal) == hipSuccess) (void)hipEventDestroy(e->event);
    (void)hipGetLastError();
    delete e;
}

int wk_event_record(wk_event *e, wk_stream *s) {
    int rc = bind(s);
    if (rc) return rc;
    if (!e) return WK_E_INVALID_VALUE;
    WK_HIP_TRY(hipEventRecord(e->event, s->stream));
    return WK_OK;
}

int wk_event_sync(wk_event *e) {
    if (!e) return WK_E_INVALID_VALUE;
    WK_HIP_TRY(hipSetDevice(e->dev->ordinal));
    WK_HIP_TRY(hipEventSynchronize(e->event));
    return WK_OK;
}

int wk_event_elapsed_ms(wk_event *start, wk_event *stop, float *out_ms) {
    if (!start || !stop || !out_ms) return WK_E_INVALID_VALUE;
    WK_HIP_TRY(hipSetDevice(start->dev->ordinal));
    WK_HIP_TRY(hipEventElapsedTime(out_ms, start->event, stop->event));
    return WK_OK;
}

// Allocation colouring.  Two streams that a kernel walks in step (x and y of AXPY) run 1.5-2.5 % faster
// on MI355X when their base addresses differ by an odd number of KiB from 3 KiB up than when they
// share their offset inside a 4 KiB block, which is what two fresh hipMalloc blocks do (measured on
// AXPY, n = 2^28 f32, over 24 base separations: same offset 6.49-6.81 TB/s, mean 6.71; +3 KiB
// 6.78-6.85, mean 6.82; +5 / +7 KiB the same; +2 KiB no gain; +4 KiB worse).  Successive large
// allocations therefore start 0, 3, 6, 9 KiB into their block, which makes every pair of neighbours
// in allocation order differ by +3 KiB or -9 KiB.  The test option "alloc_colours" = 0 turns it off.
namespace {
constexpr size_t COLOUR_MIN_BYTES = size_t(1) << 20, COLOUR_STEP = 3072;
std::mutex g_colour_mutex;
std::unordered_map<void *, void *> g_coloured; // pointer handed out -> block to free
unsigned g_next_colour = 0;
bool colouring_enabled() { return wk::g_test_options.alloc_colours != 0; }
} // namespace

int wk_malloc(wk_device *dev, size_t bytes, void **out_dptr) {
    if (!dev || !out_dptr || bytes == 0) return WK_E_INVALID_VALUE;
    *out_dptr = nullptr;
    WK_HIP_TRY(hipSetDevice(dev->ordinal));
    if (bytes < COLOUR_MIN_BYTES || !colouring_enabled()) {
        WK_HIP_TRY(hipMalloc(out_dptr, bytes));
        return WK_OK;
    }
    std::lock_guard<std::mutex> lock(g_colour_mutex);
    const size_t colour = (g_next_colour & 3u) * COLOUR_STEP;
    void *block = nullptr;
    WK_HIP_TRY(hipMalloc(&block, bytes + colour));
    ++g_next_colour;
    *out_dptr = static_cast<char *>(block) + colour;
    if (colour) g_coloured.emplace(*out_dptr, block);
    return WK_OK;
}

int wk_free(wk_device *dev, void *dptr) {
    if (!dev) return WK_E_INVALID_VALUE;
    if (!dptr) return WK_OK;
    WK_HIP_TRY(hipSetDevice(dev->ordinal));
    {
        std::lock_guard<std::mutex> lock(g_colour_mutex);
        auto it = g_coloured.find(dptr);
        if (it != g_coloured.end()) {
            dptr = it->second;
            g_coloured.erase(it);
        }
    }
    WK_HIP_TRY(hipFree(dptr));
    return WK_OK;
}

int wk_mem_info(wk_device *dev, size_t *free_bytes, size_t *total_bytes) {
    if (!dev || !free_bytes || !total_bytes) return WK_E_INVALID_VALUE;
    WK_HIP_TRY(hipSetDevice(dev->ordinal));
    WK_HIP_TRY(hipMemGetInfo(free_bytes, total_bytes));
    return WK_OK;
}

int wk_memset_async(wk_stream *s, void *dptr, int byte, size_t bytes) {
    int rc = bind(s);
    if (rc) return rc;
    if (!dptr) return WK_E_INVALID_VALUE;
    if (bytes == 0) return WK_OK;
    WK_HIP_TRY(hipMemsetAsync(dptr, byte, bytes, s->stream));
    return WK_OK;
}

// Device-to-device copy of a pitched region, one 16-byte vector per lane: blockIdx.y walks the
// rows (all slices), blockIdx.x the 16-byte columns, so no lane divides anything per element.  One
// wavefront per work-group, like the AXPY kernels: latency is hidden by the number of work-groups in flight.
__global__ __launch_bounds__(64) void rect_copy16_kernel(char *__restrict__ dst, size_t drp, size_t dsp,
                                                         const char *__restrict__ src, size_t srp, size_t ssp, size_t width16,
                                                         size_t rows, size_t total_rows) {
    for (size_t row = blockIdx.y; row < total_rows; row += gridDim.y) {
        const size_t z = row / rows, r = row % rows;
        typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 *sp = reinterpret_cast<const u32x4 *>(src + z * ssp + r * srp);
        u32x4 *dp = reinterpret_cast<u32x4 *>(dst + z * dsp + r * drp);
        for (size_t c = blockIdx.x * 64ull + threadIdx.x; c < width16; c += (size_t)gridDim.x * 64ull)
            __builtin_nontemporal_store(__builtin_nontemporal_load(&sp[c]), &dp[c]);
    }
}

static int rect_copy(wk_stream *s, void *dst, size_t drp, size_t dsp, const void *src, size_t srp, size_t ssp,
                     size_t width, size_t rows, size_t slices, hipMemcpyKind kind) {
    int rc = bind(s);
    if (rc) return rc;
    if (!dst || !src) return WK_E_INVALID_VALUE;
    if (width == 0 || rows == 0 || slices == 0) return WK_OK;
    if (drp < width || srp < width) return WK_E_INVALID_VALUE;
    if (slices > 1 && (dsp < drp * rows || ssp < srp * rows)) return WK_E_INVALID_VALUE;
    // device to device with everything on 16-byte boundaries: the streaming kernel (it outruns the
    // runtime's 2-D copy, and one launch covers all slices)
    if (kind == hipMemcpyDeviceToDevice && width % 16 == 0 && drp % 16 == 0 && srp % 16 == 0 && dsp % 16 == 0 && ssp % 16 == 0 &&
        ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u) == 0) {
        size_t w16 = width / 16, nrows = rows, nslices = slices, d_rp = drp, s_rp = srp;
        if (drp == width && srp == width && (slices == 1 || (dsp == width * rows && ssp == width * rows))) {
            w16 *= rows * slices; // fully contiguous: one long row
            nrows = nslices = 1;
            d_rp = s_rp = w16 * 16;
        }
        const size_t total_rows = nrows * nslices;
        const size_t gx = (w16 + 63) / 64;
        const unsigned grid_x = (unsigned)(gx < 1 ? 1 : (gx > (1u << 22) ? (1u << 22) : gx));
        const unsigned grid_y = (unsigned)(total_rows > 65535 ? 65535 : total_rows);
        hipLaunchKernelGGL(rect_copy16_kernel, dim3(grid_x, grid_y ? grid_y : 1), dim3(64), 0, s->stream, static_cast<char *>(dst),
                           d_rp, dsp, static_cast<const char *>(src), s_rp, ssp, w16, nrows, total_rows);
        return launch_status();
    }
    // fully contiguous on both sides: one linear copy
    if (drp == width && srp == width && (slices == 1 || (dsp == width * rows && ssp == width * rows))) {
        WK_HIP_TRY(hipMemcpyAsync(dst, src, width * rows * slices, kind, s->stream));
        return WK_OK;
    }
    for (size_t z = 0; z < slices; ++z) {
        WK_HIP_TRY(hipMemcpy2DAsync(static_cast<char *>(dst) + z * dsp, drp, static_cast<const char *>(src) + z * ssp,
                                    srp, width, rows, kind, s->stream));
    }
    return WK_OK;
}

int wk_copy_h2d_rect_async(wk_stream *s, void *dst, size_t drp, size_t dsp, const void *host_src, size_t srp,
                           size_t ssp, size_t width_bytes, size_t rows, size_t slices) {
    return rect_copy(s, dst, drp, dsp, host_src, srp, ssp, width_bytes, rows, slices, hipMemcpyHostToDevice);
}

int wk_copy_d2h_rect_async(wk_stream *s, void *host_dst, size_t drp, size_t dsp, const void *src, size_t srp,
                           size_t ssp, size_t width_bytes, size_t rows, size_t slices) {
    return rect_copy(s, host_dst, drp, dsp, src, srp, ssp, width_bytes, rows, slices, hipMemcpyDeviceToHost);
}

int wk_copy_d2d_rect_async(wk_stream *s, void *dst, size_t drp, size_t dsp, const void *src, size_t srp, size_t ssp,
                           size_t width_bytes, size_t rows, size_t slices) {
    return rect_copy(s, dst, drp, dsp, src, srp, ssp, width_bytes, rows, slices, hipMemcpyDeviceToDevice);
}

} // extern "C"

// ---- fill / identity -------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void fill_kernel(T *__restrict__ buf, uint64_t depth, uint64_t rows, uint64_t cols,
                                                   uint64_t row_pitch, uint64_t slice_pitch, T value) {
    const uint64_t total = depth * rows * cols;
    for (uint64_t idx = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t k = idx % cols;
        const uint64_t ij = idx / cols;
        const uint64_t j = ij % rows, i = ij / rows;
        buf[i * slice_pitch + j * row_pitch + k] = value;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void identity_kernel(T *__restrict__ buf, uint64_t size, uint64_t pitch_sum, T one) {
    const uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x;
    if (i < size) buf[i * pitch_sum] = one;
}

template <typename T> static T load_scalar(const void *host) {
    T v;
    std::memcpy(&v, host, sizeof(T));
    return v;
}

template <typename T> static T one_of() {
    if constexpr (elem_traits<T>::is_complex) {
        using R = typename elem_traits<T>::real;
        return T{R(1), R(0)};
    } else {
        return T(1);
    }
}

static unsigned grid_for(uint64_t total, unsigned block) {
    uint64_t g = (total + block - 1) / block;
    const uint64_t cap = 256ull * 64;
    return static_cast<unsigned>(g < cap ? (g ? g : 1) : cap);
}

extern "C" int wk_fill(wk_stream *s, int dtype, void *dptr, const uint64_t shape3[3], uint64_t row_pitch,
                       uint64_t slice_pitch, const void *host_scalar) {
    int rc = bind(s);
    if (rc) return rc;
    if (!dptr || !shape3 || !host_scalar) return WK_E_INVALID_VALUE;
    const uint64_t d = shape3[0], r = shape3[1], c = shape3[2];
    if (!d || !r || !c || row_pitch < c || (d > 1 && slice_pitch < row_pitch * r)) return WK_E_INVALID_VALUE;
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const T v = load_scalar<T>(host_scalar);
        hipLaunchKernelGGL(fill_kernel<T>, dim3(grid_for(d * r * c, 256)), dim3(256), 0, s->stream,
                           static_cast<T *>(dptr), d, r, c, row_pitch, slice_pitch, v);
        return launch_status();
    });
}

extern "C" int wk_identity(wk_stream *s, int dtype, void *dptr, uint64_t size, uint64_t pitch_sum) {
    int rc = bind(s);
    if (rc) return rc;
    if (!dptr || !size || !pitch_sum) return WK_E_INVALID_VALUE;
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        hipLaunchKernelGGL(identity_kernel<T>, dim3((unsigned)((size + 255) / 256)), dim3(256), 0, s->stream,
                           static_cast<T *>(dptr), size, pitch_sum, one_of<T>());
        return launch_status();
    });
}

// ---- calibration copy ----------------------------------------------------------------------

__global__ __launch_bounds__(256) void copy16_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src, size_t n16) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

// Launch-cost probes: the same grid, work-group size and LDS claim as a GEMM launch, with nothing (kind 0)
// or only the stores of an f32 tile per work-group (kind 1: 16 floats per thread, rows of 64 floats) inside.
extern "C" __global__ void wk_probe_kernel(int kind, float *dst, float value) {
    extern __shared__ float probe_lds[];
    if (kind == 0) return;
    float *tile = dst + (size_t)blockIdx.x * blockDim.x * 16;
#pragma unroll
    for (int r = 0; r < 16; ++r) tile[(size_t)r * blockDim.x + threadIdx.x] = value;
}

extern "C" int wk_probe_launch(wk_stream *s, int kind, unsigned work_groups, unsigned threads, size_t lds_bytes, void *dst,
                               size_t dst_bytes) {
    int rc = bind(s);
    if (rc) return rc;
    if (kind < 0 || kind > 1 || !work_groups || !threads || threads > 1024 || threads % 64 || lds_bytes > 160 * 1024) return WK_E_INVALID_VALUE;
    if (kind == 1 && (!dst || dst_bytes < (size_t)work_groups * threads * 16 * sizeof(float))) return WK_E_INVALID_VALUE;
    static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(wk_probe_kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (attr != hipSuccess) { (void)hipGetLastError(); return hip_code(attr); }
    hipLaunchKernelGGL(wk_probe_kernel, dim3(work_groups), dim3(threads), lds_bytes, s->stream, kind, static_cast<float *>(dst), 1.0f);
    return launch_status();
}

// Memory-rate probes in the shape of the AXPY stream kernel: one wavefront per work-group, one 16-byte
// vector per lane, non-temporal loads, streaming stores.  kind 0 copies src to dst (1 read + 1 write
// stream), kind 1 only reads src (1 read stream), kind 2 reads src and dst (2 read streams).  The reading
// kinds store a lane's vector only when all its words equal the sentinel the host passes, which the host
// chooses so that it never happens; the loads stay because the compiler cannot know that.
typedef unsigned u32x4_probe __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(64) void stream_probe_kernel(int kind, u32x4_probe *__restrict__ dst, const u32x4_probe *__restrict__ src,
                                                           size_t n16, unsigned sentinel) {
    const size_t i = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n16) return;
    u32x4_probe v = __builtin_nontemporal_load(src + i);
    if (kind == 0) {
        asm volatile("global_store_dwordx4 %0, %1, off nt sc0 sc1" ::"v"(dst + i), "v"(v) : "memory");
        return;
    }
    if (kind == 2) {
        const u32x4_probe w = __builtin_nontemporal_load(dst + i);
        v ^= w;
    }
    if (v.x == sentinel && v.y == sentinel && v.z == sentinel && v.w == sentinel) dst[i] = v;
}

extern "C" int wk_stream_probe(wk_stream *s, int kind, void *dst, const void *src, size_t bytes, unsigned sentinel) {
    int rc = bind(s);
    if (rc) return rc;
    if (kind < 0 || kind > 2 || !dst || !src || bytes % 16 || bytes / 16 / 64 >= 0x7fffffffull ||
        (reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 16)
        return WK_E_INVALID_VALUE;
    if (!bytes) return WK_OK;
    const size_t n16 = bytes / 16;
    hipLaunchKernelGGL(stream_probe_kernel, dim3(static_cast<unsigned>((n16 + 63) / 64)), dim3(64), 0, s->stream, kind,
                       static_cast<u32x4_probe *>(dst), static_cast<const u32x4_probe *>(src), n16, sentinel);
    return launch_status();
}

extern "C" int wk_copy_kernel(wk_stream *s, void *dst, const void *src, size_t bytes) {
    int rc = bind(s);
    if (rc) return rc;
    if (!dst || !src || bytes % 16 || (reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 16)
        return WK_E_INVALID_VALUE;
    if (!bytes) return WK_OK;
    const size_t n16 = bytes / 16;
    const size_t want = (n16 + 255) / 256;
    const unsigned grid = static_cast<unsigned>(want < 256ull * 32 ? want : 256ull * 32);
    hipLaunchKernelGGL(copy16_kernel, dim3(grid), dim3(256), 0, s->stream, static_cast<uint4 *>(dst),
                       static_cast<const uint4 *>(src), n16);
    return launch_status();
}
