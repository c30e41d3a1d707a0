// blas.axpy for gfx950: y = alpha*x + y  (src/blas/axpy.zig:93-169, kernels/axpy.cl:3-72).
//
// AXPY is pure streaming (2 loads + 1 store per element), so the only thing that matters is
// keeping HBM busy: every lane moves 16 bytes per access and a wavefront touches 1 KiB of
// consecutive addresses per access.  Measured on MI355X (f32, n = 2^28) the best shape is the
// smallest one: one wavefront per work-group, one 16-byte vector of x and of y per lane,
// non-temporal loads and stores (6.76 TB/s; 256-thread groups with 4 vectors per lane reach
// 6.1 TB/s, cached loads/stores 5.5 TB/s, an XCD-contiguous block order 6.6 TB/s).  Latency
// is hidden by occupancy (up to 32 resident waves per CU), not by unrolling.
#include "wk_internal.hpp"

#include <cmath>
#include <cstring>
#include <limits>

using namespace wk;

namespace {

enum : int { MODE_ADD = 0, MODE_SUB = 1, MODE_ALPHA = 2 };

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int AXPY_BLOCK = 64;   // stream kernel: one wavefront per work-group
constexpr int AXPY_UNROLL = 1;
constexpr int PITCHED_BLOCK = 256;

template <typename T, int MODE>
__device__ __forceinline__ T axpy_elem(T x, T y, typename elem_traits<T>::acc alpha) {
    using A = typename elem_traits<T>::acc;
    const A xa = widen<A>(x), ya = widen<A>(y);
    if constexpr (MODE == MODE_ADD) return narrow<T>(add(ya, xa));
    else if constexpr (MODE == MODE_SUB) return narrow<T>(sub(ya, xa));
    else return narrow<T>(mad(xa, alpha, ya)); // floats: one fma; complex: y + x*alpha (3-multiply product)
}

// Contiguous operands, both 16-byte aligned.  One block covers BLOCK*UNROLL vectors.
template <typename T, int MODE>
__global__ __launch_bounds__(AXPY_BLOCK) void axpy_stream_kernel(const T *__restrict__ x, T *__restrict__ y, uint64_t n,
                                                                 typename elem_traits<T>::acc alpha) {
    constexpr int VE = 16 / sizeof(T);
    const uint64_t nvec = n / VE;
    const u32x4 *xv = reinterpret_cast<const u32x4 *>(x);
    u32x4 *yv = reinterpret_cast<u32x4 *>(y);
    const uint64_t base = (uint64_t)blockIdx.x * (AXPY_BLOCK * AXPY_UNROLL) + threadIdx.x;

    u32x4 xr[AXPY_UNROLL], yr[AXPY_UNROLL];
#pragma unroll
    for (int u = 0; u < AXPY_UNROLL; ++u) {
        const uint64_t i = base + (uint64_t)u * AXPY_BLOCK;
        if (i < nvec) {
            xr[u] = __builtin_nontemporal_load(xv + i);
            yr[u] = __builtin_nontemporal_load(yv + i);
        }
    }
#pragma unroll
    for (int u = 0; u < AXPY_UNROLL; ++u) {
        const uint64_t i = base + (uint64_t)u * AXPY_BLOCK;
        if (i < nvec) {
            T xe[VE], ye[VE];
            __builtin_memcpy(xe, &xr[u], 16);
            __builtin_memcpy(ye, &yr[u], 16);
#pragma unroll
            for (int e = 0; e < VE; ++e) ye[e] = axpy_elem<T, MODE>(xe[e], ye[e], alpha);
            u32x4 out;
            __builtin_memcpy(&out, ye, 16);
            // Streaming store with system scope (nt sc0 sc1): the result goes straight out to memory.
            // Measured at n = 2^28 f32 on MI355X with non-temporal loads: this store 6.80 TB/s, a plain
            // non-temporal store 6.73, a cached store 5.98.
            asm volatile("global_store_dwordx4 %0, %1, off nt sc0 sc1" ::"v"(yv + i), "v"(out) : "memory");
        }
    }
    // the < VE leftover elements
    if (blockIdx.x == 0) {
        const uint64_t i = nvec * VE + threadIdx.x;
        if (i < n) y[i] = axpy_elem<T, MODE>(x[i], y[i], alpha);
    }
}

// Any pitches / alignment: one element per step over the logical {depth, rows, cols} region
// (the scalar build of axpy.cl:23-29).
template <typename T, int MODE>
__global__ __launch_bounds__(PITCHED_BLOCK) void axpy_pitched_kernel(const T *__restrict__ x, T *__restrict__ y, uint64_t depth,
                                                                  uint64_t rows, uint64_t cols, uint64_t xrp, uint64_t xsp,
                                                                  uint64_t yrp, uint64_t ysp,
                                                                  typename elem_traits<T>::acc alpha) {
    const uint64_t total = depth * rows * cols;
    for (uint64_t idx = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t k = idx % cols;
        const uint64_t ij = idx / cols;
        const uint64_t j = ij % rows, i = ij / rows;
        const uint64_t xi = i * xsp + j * xrp + k, yi = i * ysp + j * yrp + k;
        y[yi] = axpy_elem<T, MODE>(x[xi], y[yi], alpha);
    }
}

// Pitched rows whose starts and pitches are 16-byte aligned (every 2-D / 3-D Tensor of the host
// mirror): the same shape as the stream kernel -- one wavefront per work-group, one 16-byte vector
// per lane, streaming stores -- with blockIdx.x over the vectors of a row, blockIdx.y over the rows
// and blockIdx.z over the slices, so nothing is divided anywhere; the < VE tail of each row is done
// by element.
template <typename T, int MODE>
__global__ __launch_bounds__(AXPY_BLOCK) void axpy_rows_kernel(const T *__restrict__ x, T *__restrict__ y, uint64_t rows,
                                                               uint64_t cols, uint64_t depth, uint64_t xrp, uint64_t xsp,
                                                               uint64_t yrp, uint64_t ysp, typename elem_traits<T>::acc alpha) {
    constexpr int VE = 16 / sizeof(T);
    const uint64_t nvec = cols / VE;
    const uint64_t v = (uint64_t)blockIdx.x * AXPY_BLOCK + threadIdx.x;
    for (uint64_t i = blockIdx.z; i < depth; i += gridDim.z)
    for (uint64_t j = blockIdx.y; j < rows; j += gridDim.y) {
        const T *xr_ = x + i * xsp + j * xrp;
        T *yr_ = y + i * ysp + j * yrp;
        if (v < nvec) {
            const u32x4 *xv = reinterpret_cast<const u32x4 *>(xr_) + v;
            u32x4 *yv = reinterpret_cast<u32x4 *>(yr_) + v;
            const u32x4 xq = __builtin_nontemporal_load(xv), yq = __builtin_nontemporal_load(yv);
            T xe[VE], ye[VE];
            __builtin_memcpy(xe, &xq, 16);
            __builtin_memcpy(ye, &yq, 16);
#pragma unroll
            for (int e = 0; e < VE; ++e) ye[e] = axpy_elem<T, MODE>(xe[e], ye[e], alpha);
            u32x4 out;
            __builtin_memcpy(&out, ye, 16);
            asm volatile("global_store_dwordx4 %0, %1, off nt sc0 sc1" ::"v"(yv), "v"(out) : "memory");
        }
        if (blockIdx.x == 0) {
            const uint64_t k = nvec * VE + threadIdx.x;
            if (k < cols) yr_[k] = axpy_elem<T, MODE>(xr_[k], yr_[k], alpha);
        }
    }
}

// isSubstracting, src/blas/axpy.zig:66-91
template <typename T> bool is_subtracting(int dtype, const void *host_alpha) {
    using R = typename elem_traits<T>::real;
    R v[2] = {R(0), R(0)};
    std::memcpy(v, host_alpha, sizeof(T));
    if constexpr (elem_traits<T>::is_float) {
        const R eps = std::numeric_limits<R>::epsilon();
        if constexpr (elem_traits<T>::is_complex)
            return std::fabs(v[0] + R(1)) < eps && (std::fabs(v[1]) < eps || std::fabs(v[1] + R(1)) < eps);
        else
            return std::fabs(v[0] + R(1)) < eps;
    } else {
        if (!dtype_is_signed(dtype)) return false;
        const R minus_one = static_cast<R>(~R(0)); // two's complement -1
        if constexpr (elem_traits<T>::is_complex)
            return v[0] == minus_one && (v[1] == R(0) || v[1] == minus_one);
        else
            return v[0] == minus_one;
    }
}

template <typename T, int MODE>
int launch(wk_stream *s, const uint64_t shape3[3], const T *x, uint64_t xrp, uint64_t xsp, T *y, uint64_t yrp,
           uint64_t ysp, typename elem_traits<T>::acc alpha) {
    const uint64_t d = shape3[0], r = shape3[1], c = shape3[2];
    const uint64_t n = d * r * c;
    // Dense = the logical elements are one contiguous run.  A single-row slice may still be padded
    // (pitch > cols), so the slice pitch is held against rows * cols, not rows * row pitch.
    const bool x_dense = (r == 1 || xrp == c) && (d == 1 || xsp == r * c);
    const bool y_dense = (r == 1 || yrp == c) && (d == 1 || ysp == r * c);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
    constexpr uint64_t VE = 16 / sizeof(T);
    if (x_dense && y_dense && aligned && n >= VE) {
        const uint64_t nvec = n / VE;
        const uint64_t per_block = (uint64_t)AXPY_BLOCK * AXPY_UNROLL;
        const uint64_t blocks = (nvec + per_block - 1) / per_block;
        if (blocks > 0x7fffffffull) return WK_E_INVALID_VALUE;
        hipLaunchKernelGGL((axpy_stream_kernel<T, MODE>), dim3((unsigned)blocks), dim3(AXPY_BLOCK), 0, s->stream, x, y, n,
                           alpha);
        return launch_status();
    }
    const bool rows_aligned = aligned && xrp % VE == 0 && yrp % VE == 0 && xsp % VE == 0 && ysp % VE == 0;
    if (rows_aligned && c >= VE) {
        const uint64_t gx = (c / VE + AXPY_BLOCK - 1) / AXPY_BLOCK;
        if (gx > 0x7fffffffull) return WK_E_INVALID_VALUE;
        const uint64_t gy = r < 65535 ? r : 65535, gz = d < 65535 ? d : 65535;
        hipLaunchKernelGGL((axpy_rows_kernel<T, MODE>), dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), dim3(AXPY_BLOCK), 0, s->stream, x, y, r,
                           c, d, xrp, xsp, yrp, ysp, alpha);
        return launch_status();
    }
    const uint64_t want = (n + PITCHED_BLOCK - 1) / PITCHED_BLOCK;
    const unsigned grid = (unsigned)(want < 256ull * 64 ? want : 256ull * 64);
    hipLaunchKernelGGL((axpy_pitched_kernel<T, MODE>), dim3(grid), dim3(PITCHED_BLOCK), 0, s->stream, x, y, d, r, c, xrp, xsp,
                       yrp, ysp, alpha);
    return launch_status();
}

} // namespace

extern "C" int wk_axpy(wk_stream *s, int dtype, const uint64_t shape3[3], const void *x, uint64_t x_row_pitch,
                       uint64_t x_slice_pitch, void *y, uint64_t y_row_pitch, uint64_t y_slice_pitch,
                       const void *host_alpha) {
    int rc = bind(s);
    if (rc) return rc;
    if (!shape3 || !x || !y) return WK_E_INVALID_VALUE;
    const uint64_t d = shape3[0], r = shape3[1], c = shape3[2];
    if (!d || !r || !c) return WK_E_INVALID_VALUE;
    if (r > 1 && (x_row_pitch < c || y_row_pitch < c)) return WK_E_INVALID_VALUE;
    if (d > 1 && (x_slice_pitch < r * x_row_pitch || y_slice_pitch < r * y_row_pitch)) return WK_E_INVALID_VALUE;
    if (d > 1 && (x_slice_pitch < r * c || y_slice_pitch < r * c)) return WK_E_INVALID_VALUE;

    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        using A = typename elem_traits<T>::acc;
        const T *xp = static_cast<const T *>(x);
        T *yp = static_cast<T *>(y);
        if (!host_alpha)
            return launch<T, MODE_ADD>(s, shape3, xp, x_row_pitch, x_slice_pitch, yp, y_row_pitch, y_slice_pitch, zero_of<A>());
        if (is_subtracting<T>(dtype, host_alpha))
            return launch<T, MODE_SUB>(s, shape3, xp, x_row_pitch, x_slice_pitch, yp, y_row_pitch, y_slice_pitch, zero_of<A>());
        T a;
        std::memcpy(&a, host_alpha, sizeof(T));
        return launch<T, MODE_ALPHA>(s, shape3, xp, x_row_pitch, x_slice_pitch, yp, y_row_pitch, y_slice_pitch, widen<A>(a));
    });
}
