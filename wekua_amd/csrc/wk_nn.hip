// Element-wise and reduction kernels the MLP training step needs around gemm / axpy:
// bias add (+ activation), activation derivative, Hadamard product, bias gradient (column
// sums), MSE with its derivative, a whole-tensor sum, and an Adam update.
//
// Reference kernels restated here:  src/nn/layer/kernels/{bias,bias_step}.cl,
// src/nn/activation/kernels/{sigmoid,tanh}.cl, src/math/kernels/{dot,sum,trig}.cl,
// src/nn/loss/kernels/mse.cl.  All are HBM-bound streaming passes over row-pitched 2-D/3-D
// tensors: one 16-byte vector per lane, rows addressed through their pitch so that only the
// logical region is touched.  f32 and f64 only (what the MLP configuration uses).
#include "wk_internal.hpp"

#include <atomic>
#include <cmath>
#include <cstring>

using namespace wk;

namespace {

constexpr int EW_BLOCK = 256;

struct Region {
    uint64_t depth, rows, cols;
};

// One tensor operand of an element-wise pass.
template <typename T> struct Opnd {
    T *p;
    uint64_t rp, sp;
};

template <typename T> __device__ __forceinline__ T act_derivative(int kind, T y) {
    if (kind == WK_ACT_SIGMOID) return y * (T(1) - y);
    if (kind == WK_ACT_TANH) return T(1) - y * y;
    return T(1);
}

// Generic element-wise driver: F(idx3, element pointers...) over the logical region, VE
// elements of a row per thread when every operand allows 16-byte accesses.
// WMASK: bit i set = operand i is written back (the others are read-only inputs).
template <typename T, int NOPS, int WMASK, bool VEC, typename F>
__global__ __launch_bounds__(EW_BLOCK) void ew_kernel(Region rg, Opnd<T> o0, Opnd<T> o1, Opnd<T> o2, Opnd<T> o3, F f) {
    constexpr int VE = VEC ? 16 / sizeof(T) : 1;
    const uint64_t cols_v = (rg.cols + VE - 1) / VE;
    const uint64_t total = rg.depth * rg.rows * cols_v;
    for (uint64_t idx = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t cv = idx % cols_v;
        const uint64_t ij = idx / cols_v;
        const uint64_t j = ij % rg.rows, i = ij / rg.rows;
        const uint64_t c = cv * VE;
        T *p0 = o0.p + i * o0.sp + j * o0.rp + c;
        T *p1 = NOPS > 1 ? o1.p + i * o1.sp + j * o1.rp + c : nullptr;
        T *p2 = NOPS > 2 ? o2.p + i * o2.sp + j * o2.rp + c : nullptr;
        T *p3 = NOPS > 3 ? o3.p + i * o3.sp + j * o3.rp + c : nullptr;
        if (VEC && c + VE <= rg.cols) {
            T v0[VE], v1[VE], v2[VE], v3[VE];
            __builtin_memcpy(v0, p0, 16);
            if (NOPS > 1) __builtin_memcpy(v1, p1, 16);
            if (NOPS > 2) __builtin_memcpy(v2, p2, 16);
            if (NOPS > 3) __builtin_memcpy(v3, p3, 16);
#pragma unroll
            for (int e = 0; e < VE; ++e) f(c + e, v0[e], v1[e], v2[e], v3[e]);
            if (WMASK & 1) __builtin_memcpy(p0, v0, 16);
            if (NOPS > 1 && (WMASK & 2)) __builtin_memcpy(p1, v1, 16);
            if (NOPS > 2 && (WMASK & 4)) __builtin_memcpy(p2, v2, 16);
            if (NOPS > 3 && (WMASK & 8)) __builtin_memcpy(p3, v3, 16);
        } else {
            for (int e = 0; e < VE && c + e < rg.cols; ++e) {
                T a = p0[e], b = NOPS > 1 ? p1[e] : T(0), cc = NOPS > 2 ? p2[e] : T(0), d = NOPS > 3 ? p3[e] : T(0);
                f(c + e, a, b, cc, d);
                if (WMASK & 1) p0[e] = a;
                if (NOPS > 1 && (WMASK & 2)) p1[e] = b;
                if (NOPS > 2 && (WMASK & 4)) p2[e] = cc;
                if (NOPS > 3 && (WMASK & 8)) p3[e] = d;
            }
        }
    }
}

template <typename T> bool vec_ok(const Opnd<T> &o) {
    constexpr uint64_t VE = 16 / sizeof(T);
    return !o.p || ((reinterpret_cast<uintptr_t>(o.p) & 15u) == 0 && o.rp % VE == 0 && o.sp % VE == 0);
}

template <typename T, int NOPS, int WMASK, typename F>
int ew_launch(wk_stream *s, const Region &rg, Opnd<T> o0, Opnd<T> o1, Opnd<T> o2, Opnd<T> o3, F f) {
    const bool vec = vec_ok(o0) && vec_ok(o1) && vec_ok(o2) && vec_ok(o3);
    const uint64_t ve = vec ? 16 / sizeof(T) : 1;
    const uint64_t total = rg.depth * rg.rows * ((rg.cols + ve - 1) / ve);
    const uint64_t want = (total + EW_BLOCK - 1) / EW_BLOCK;
    const unsigned grid = (unsigned)(want < 256ull * 256 ? (want ? want : 1) : 256ull * 256);
    if (vec) hipLaunchKernelGGL((ew_kernel<T, NOPS, WMASK, true, F>), dim3(grid), dim3(EW_BLOCK), 0, s->stream, rg, o0, o1, o2, o3, f);
    else hipLaunchKernelGGL((ew_kernel<T, NOPS, WMASK, false, F>), dim3(grid), dim3(EW_BLOCK), 0, s->stream, rg, o0, o1, o2, o3, f);
    return launch_status();
}

int check_region(const uint64_t shape3[3], Region &rg) {
    if (!shape3) return WK_E_INVALID_VALUE;
    rg = {shape3[0], shape3[1], shape3[2]};
    if (!rg.depth || !rg.rows || !rg.cols) return WK_E_INVALID_VALUE;
    return WK_OK;
}

template <typename T> int check_opnd(const Region &rg, const void *p, uint64_t rp, uint64_t sp) {
    if (!p) return WK_E_INVALID_VALUE;
    if (rg.rows > 1 && rp < rg.cols) return WK_E_INVALID_VALUE;
    if (rg.depth > 1 && sp < rg.rows * rp) return WK_E_INVALID_VALUE;
    return WK_OK;
}

template <typename F> int dispatch_float(int dtype, F &&f) {
    if (dtype == WK_F32) return f.template operator()<float>();
    if (dtype == WK_F64) return f.template operator()<double>();
    return dtype >= 0 && dtype < WK_DTYPE_COUNT ? WK_E_TYPE_NOT_SUPPORTED : WK_E_TYPE_NOT_SUPPORTED;
}

// ---- column sums (bias_step.cl).  Rows are cut into `chunks` bands; a block of 64 x 4 threads
// sums 64 columns of one band (consecutive lanes read consecutive addresses of a row, four rows
// in flight per block) and writes one partial per column; a second pass runs the same kernel over
// the partials, so the order of additions is fixed and the result does not depend on scheduling. --------------------------------------------
constexpr int COLSUM_ROWS_PER_BAND = 32;
constexpr int COLSUM_MAX_BANDS = 64;

// Partials of wk_bias_step_static: part of the code object, so it exists on every device the library
// is loaded on from load time until the process ends, and no call ever allocates it.  In host code
// this name is only a handle for hipGetSymbolAddress; kernels get the per-device address below.
constexpr size_t STATIC_SCRATCH_BYTES = WK_BIAS_STEP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

constexpr int STATIC_SCRATCH_MAX_DEVICES = 64;
std::atomic<void *> g_static_scratch[STATIC_SCRATCH_MAX_DEVICES];

template <typename T>
__global__ __launch_bounds__(256) void colsum_bands_kernel(const T *__restrict__ x, uint64_t rows, uint64_t cols, uint64_t pitch,
                                                           uint64_t band_rows, T *__restrict__ partial) {
    __shared__ T part[4][64];
    const uint64_t c = blockIdx.x * 64ull + threadIdx.x;
    const uint64_t r0 = blockIdx.y * band_rows;
    const uint64_t r1 = r0 + band_rows < rows ? r0 + band_rows : rows;
    T acc = T(0);
    if (c < cols)
        for (uint64_t r = r0 + threadIdx.y; r < r1; r += 4) acc += x[r * pitch + c];
    part[threadIdx.y][threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.y == 0 && c < cols)
        partial[blockIdx.y * cols + c] = (part[0][threadIdx.x] + part[1][threadIdx.x]) + (part[2][threadIdx.x] + part[3][threadIdx.x]);
}

// ---- Linear.backward's element-wise half in one pass (linear.zig:606-640: getDerivative, math.dot,
// getBiasSensitivity): dev = act'(out), sens *= dev, and the band partials of the column sums of the
// new sens.  Same block shape and the same order of additions per column as colsum_bands_kernel
// (rows r0 + ty, r0 + ty + 4, ... per thread row ty, then (p0 + p1) + (p2 + p3)), so the bias gradient
// comes out bit for bit as from the separate passes; every lane moves VE consecutive columns.
// kind WK_ACT_NONE: dev is read, not written (the reference multiplies by the cached tensor as it is).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void sens_step_kernel(int kind, const T *__restrict__ out, uint64_t out_pitch, T *__restrict__ sens,
                                                        uint64_t sens_pitch, T *__restrict__ dev, uint64_t dev_pitch, uint64_t rows,
                                                        uint64_t cols, uint64_t band_rows, T *__restrict__ partial) {
    constexpr int VE = VEC ? 16 / sizeof(T) : 1;
    __shared__ T part[4][64][VE];
    const uint64_t c = (blockIdx.x * 64ull + threadIdx.x) * VE;
    const uint64_t r0 = blockIdx.y * band_rows;
    const uint64_t r1 = r0 + band_rows < rows ? r0 + band_rows : rows;
    T acc[VE];
#pragma unroll
    for (int e = 0; e < VE; ++e) acc[e] = T(0);
    if (c < cols) {
        const bool whole = VEC && c + VE <= cols;
        for (uint64_t r = r0 + threadIdx.y; r < r1; r += 4) {
            T *sp = sens + r * sens_pitch + c;
            T *dp = dev + r * dev_pitch + c;
            const T *op = out + r * out_pitch + c;
            T sv[VE], dv[VE], ov[VE];
            if (whole) {
                __builtin_memcpy(sv, sp, sizeof sv);
                if (kind == WK_ACT_NONE) __builtin_memcpy(dv, dp, sizeof dv);
                else __builtin_memcpy(ov, op, sizeof ov);
            } else {
                for (int e = 0; e < VE; ++e) {
                    const bool ok = c + e < cols;
                    sv[e] = ok ? sp[e] : T(0);
                    dv[e] = ok && kind == WK_ACT_NONE ? dp[e] : T(0);
                    ov[e] = ok && kind != WK_ACT_NONE ? op[e] : T(0);
                }
            }
#pragma unroll
            for (int e = 0; e < VE; ++e) {
                if (kind != WK_ACT_NONE) dv[e] = act_derivative<T>(kind, ov[e]);
                {
                    // the product is rounded before it is added (no fused multiply-add): the sum must be
                    // over the values that are stored, as in the separate passes
#pragma clang fp contract(off)
                    sv[e] = sv[e] * dv[e];
                    acc[e] = acc[e] + sv[e];
                }
            }
            if (whole) {
                if (kind != WK_ACT_NONE) __builtin_memcpy(dp, dv, sizeof dv);
                __builtin_memcpy(sp, sv, sizeof sv);
            } else {
                for (int e = 0; e < VE; ++e)
                    if (c + e < cols) {
                        if (kind != WK_ACT_NONE) dp[e] = dv[e];
                        sp[e] = sv[e];
                    }
            }
        }
    }
    if (!partial) return;
#pragma unroll
    for (int e = 0; e < VE; ++e) part[threadIdx.y][threadIdx.x][e] = acc[e];
    __syncthreads();
    if (threadIdx.y == 0 && c < cols)
#pragma unroll
        for (int e = 0; e < VE; ++e)
            if (c + e < cols)
                partial[blockIdx.y * cols + c + e] =
                    (part[0][threadIdx.x][e] + part[1][threadIdx.x][e]) + (part[2][threadIdx.x][e] + part[3][threadIdx.x][e]);
}

// One element of the Adam update.  Every product is rounded before it is added (no fused
// multiply-add), so the one-tensor and the several-tensor kernels give the same bits whatever the
// compiler makes of their surroundings.
template <typename T>
__device__ __forceinline__ void adam_update(T &w, T &m, T &v, T g, T b1, T ib1, T b2, T ib2, T step_size, T inv_sqrt_bc2, T eps) {
#pragma clang fp contract(off)
    m = b1 * m + ib1 * g;
    v = b2 * v + (ib2 * g) * g;
    w = w - step_size * m / (sqrt(v) * inv_sqrt_bc2 + eps);
}

// ---- Adam over several parameter tensors in one launch.  Blocks are dealt to the tensors in
// proportion to their size; inside its tensor a block walks 16-byte vectors with a grid stride.
constexpr int ADAM_MULTI_MAX = 8;
template <typename T> struct AdamMultiArgs {
    T *w[ADAM_MULTI_MAX], *m[ADAM_MULTI_MAX], *v[ADAM_MULTI_MAX];
    const T *g[ADAM_MULTI_MAX];
    uint64_t rows[ADAM_MULTI_MAX], cols[ADAM_MULTI_MAX]; // depth folded into rows (slices are back to back)
    uint64_t wrp[ADAM_MULTI_MAX], grp[ADAM_MULTI_MAX], mrp[ADAM_MULTI_MAX];
    uint32_t first_block[ADAM_MULTI_MAX + 1];
    int count;
    T b1, b2, ib1, ib2, step_size, inv_sqrt_bc2, eps;
};

template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void adam_multi_kernel(AdamMultiArgs<T> a) {
    constexpr int VE = 16 / sizeof(T);
    int t = 0;
    while (t + 1 < a.count && blockIdx.x >= a.first_block[t + 1]) ++t;
    const uint64_t nblocks = a.first_block[t + 1] - a.first_block[t];
    const uint64_t cols_v = (a.cols[t] + VE - 1) / VE;
    const uint64_t total = a.rows[t] * cols_v;
    for (uint64_t idx = (blockIdx.x - a.first_block[t]) * (uint64_t)EW_BLOCK + threadIdx.x; idx < total; idx += nblocks * EW_BLOCK) {
        const uint64_t r = idx / cols_v, c = (idx % cols_v) * VE;
        T *wp = a.w[t] + r * a.wrp[t] + c, *mp = a.m[t] + r * a.mrp[t] + c, *vp = a.v[t] + r * a.mrp[t] + c;
        const T *gp = a.g[t] + r * a.grp[t] + c;
        const bool whole = c + VE <= a.cols[t];
        T wv[VE], mv[VE], vv[VE], gv[VE];
        if (whole) {
            __builtin_memcpy(wv, wp, 16); __builtin_memcpy(mv, mp, 16); __builtin_memcpy(vv, vp, 16); __builtin_memcpy(gv, gp, 16);
        } else {
            for (int e = 0; e < VE; ++e) {
                const bool ok = c + e < a.cols[t];
                wv[e] = ok ? wp[e] : T(0); mv[e] = ok ? mp[e] : T(0); vv[e] = ok ? vp[e] : T(1); gv[e] = ok ? gp[e] : T(0);
            }
        }
#pragma unroll
        for (int e = 0; e < VE; ++e)
            adam_update<T>(wv[e], mv[e], vv[e], gv[e], a.b1, a.ib1, a.b2, a.ib2, a.step_size, a.inv_sqrt_bc2, a.eps);
        if (whole) {
            __builtin_memcpy(wp, wv, 16); __builtin_memcpy(mp, mv, 16); __builtin_memcpy(vp, vv, 16);
        } else {
            for (int e = 0; e < VE; ++e)
                if (c + e < a.cols[t]) { wp[e] = wv[e]; mp[e] = mv[e]; vp[e] = vv[e]; }
        }
    }
}

// ---- whole-tensor sum (math.sum + host finish, src/math/basic.zig:128-203): two fixed-shape
// passes so that the result does not depend on scheduling. ------------------------------------
constexpr int SUM_PARTIALS = 1024;

// VEC: every row starts on a 16-byte boundary (base, pitches): a thread takes 16-byte vectors, four of them in
// flight, and the < 16 bytes at the end of a row element by element; one division per vector, none when the
// region is one row (a 1-D tensor, or rows and slices that follow each other without gaps: the host then passes
// it as one row).  Which thread adds which elements is fixed by the shape alone, so the result is the same bits
// on every run.  2^28 f32: 725 us with one element and two divisions per step -> 198 us = 5.4 TB/s (f64 5.8, 8192 x 8192 pitched 5.7).
typedef unsigned int sum_u32x4 __attribute__((ext_vector_type(4)));
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void sum_pass1_kernel(const T *__restrict__ x, Region rg, uint64_t rp, uint64_t sp,
                                                        T *__restrict__ partials) {
    __shared__ T red[256];
    constexpr uint64_t THREADS = (uint64_t)SUM_PARTIALS * 256ull;
    const uint64_t tid = blockIdx.x * 256ull + threadIdx.x;
    T acc = T(0);
    if constexpr (VEC) {
        constexpr int VE = 16 / sizeof(T);
        const uint64_t nrows = rg.depth * rg.rows, nv = rg.cols / VE, total_v = nrows * nv;
        auto vector_at = [&](uint64_t v) -> const sum_u32x4 * {
            uint64_t row = 0, c = v;
            if (nrows > 1) {
                row = v / nv;
                c = v - row * nv;
            }
            const T *p = x + (row / rg.rows) * sp + (row % rg.rows) * rp + c * VE;
            return reinterpret_cast<const sum_u32x4 *>(p);
        };
        for (uint64_t v = tid; v < total_v; v += 4 * THREADS) {
            sum_u32x4 q[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (v + u * THREADS < total_v) q[u] = __builtin_nontemporal_load(vector_at(v + u * THREADS));
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (v + u * THREADS < total_v) {
                    T e[VE];
                    __builtin_memcpy(e, &q[u], 16);
#pragma unroll
                    for (int i = 0; i < VE; ++i) acc += e[i];
                }
        }
        const uint64_t tail = rg.cols - nv * VE, total_t = nrows * tail;
        for (uint64_t t = tid; t < total_t; t += THREADS) {
            const uint64_t row = t / tail, k = nv * VE + (t - row * tail);
            acc += x[(row / rg.rows) * sp + (row % rg.rows) * rp + k];
        }
    } else {
        const uint64_t total = rg.depth * rg.rows * rg.cols;
        for (uint64_t idx = tid; idx < total; idx += THREADS) {
            const uint64_t k = idx % rg.cols;
            const uint64_t ij = idx / rg.cols;
            acc += x[(ij / rg.rows) * sp + (ij % rg.rows) * rp + k];
        }
    }
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
        if ((int)threadIdx.x < st) red[threadIdx.x] += red[threadIdx.x + st];
        __syncthreads();
    }
    if (threadIdx.x == 0) partials[blockIdx.x] = red[0];
}

template <typename T>
__global__ __launch_bounds__(256) void sum_pass2_kernel(const T *__restrict__ partials, T *__restrict__ out, T scale) {
    __shared__ T red[256];
    T acc = T(0);
    for (int i = threadIdx.x; i < SUM_PARTIALS; i += 256) acc += partials[i];
    red[threadIdx.x] = acc;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) {
        if ((int)threadIdx.x < st) red[threadIdx.x] += red[threadIdx.x + st];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = red[0] * scale;
}

} // namespace

// Called by wk_device_open with `ordinal` current: every device holds its own copy of the array at
// its own address, so the address is looked up once per device and kept.
int wk::static_scratch_setup(int ordinal) {
    if (ordinal < 0 || ordinal >= STATIC_SCRATCH_MAX_DEVICES) return WK_OK; // such a device has no static entry point
    if (g_static_scratch[ordinal].load(std::memory_order_acquire)) return WK_OK;
    void *ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return hip_code(e);
    }
    if (!ptr) return WK_E_HIP_BASE + static_cast<int>(hipErrorInvalidSymbol);
    g_static_scratch[ordinal].store(ptr, std::memory_order_release);
    return WK_OK;
}

namespace {

// Column sums of a rows x cols matrix in two launches of colsum_bands_kernel: bands of rows into
// `partial_buf`, then the bands.  The number of bands depends only on (rows, cols, partial_bytes),
// so two callers with equally sized buffers add in the same order and get the same bits.
// How the rows are cut into bands: depends only on (rows, cols, element size, partial_bytes).
inline void colsum_plan(uint64_t rows, uint64_t cols, size_t esize, size_t partial_bytes, uint64_t &bands, uint64_t &band_rows) {
    bands = (rows + COLSUM_ROWS_PER_BAND - 1) / COLSUM_ROWS_PER_BAND;
    if (bands > COLSUM_MAX_BANDS) bands = COLSUM_MAX_BANDS;
    const uint64_t fit = partial_bytes / (cols * esize);
    if (bands > fit) bands = fit;
    if (bands < 2) bands = 1; // one band writes the result directly
    band_rows = (rows + bands - 1) / bands;
    bands = (rows + band_rows - 1) / band_rows;
}

template <typename T>
int colsum_two_pass(wk_stream *s, uint64_t rows, uint64_t cols, const T *sens, uint64_t pitch, T *bias_grad,
                    void *partial_buf, size_t partial_bytes) {
    uint64_t bands, band_rows;
    colsum_plan(rows, cols, sizeof(T), partial_bytes, bands, band_rows);
    T *partial = bands > 1 ? static_cast<T *>(partial_buf) : bias_grad;
    hipLaunchKernelGGL((colsum_bands_kernel<T>), dim3((unsigned)((cols + 63) / 64), (unsigned)bands), dim3(64, 4), 0,
                       s->stream, sens, rows, cols, pitch, band_rows, partial);
    int lrc = launch_status();
    if (lrc || bands == 1) return lrc;
    // second pass: the same kernel over the bands x cols matrix of partials, as one band
    hipLaunchKernelGGL((colsum_bands_kernel<T>), dim3((unsigned)((cols + 63) / 64), 1), dim3(64, 4), 0, s->stream,
                       static_cast<const T *>(partial), bands, cols, cols, bands, bias_grad);
    return launch_status();
}

} // namespace

extern "C" {

int wk_hadamard(wk_stream *s, int dtype, const uint64_t shape3[3], void *x, uint64_t xrp, uint64_t xsp, const void *y,
                uint64_t yrp, uint64_t ysp) {
    int rc = bind(s);
    if (rc) return rc;
    Region rg;
    if ((rc = check_region(shape3, rg))) return rc;
    return dispatch_float(dtype, [&]<typename T>() -> int {
        if (check_opnd<T>(rg, x, xrp, xsp) || check_opnd<T>(rg, y, yrp, ysp)) return WK_E_INVALID_VALUE;
        return ew_launch<T, 2, 1>(s, rg, Opnd<T>{(T *)x, xrp, xsp}, Opnd<T>{(T *)y, yrp, ysp}, Opnd<T>{}, Opnd<T>{},
                               [] __device__(uint64_t, T &a, T &b, T &, T &) { a *= b; });
    });
}

int wk_activation(wk_stream *s, int dtype, int kind, const uint64_t shape3[3], void *x, uint64_t xrp, uint64_t xsp) {
    int rc = bind(s);
    if (rc) return rc;
    Region rg;
    if ((rc = check_region(shape3, rg))) return rc;
    if (kind != WK_ACT_SIGMOID && kind != WK_ACT_TANH) return WK_E_INVALID_VALUE;
    return dispatch_float(dtype, [&]<typename T>() -> int {
        if (check_opnd<T>(rg, x, xrp, xsp)) return WK_E_INVALID_VALUE;
        return ew_launch<T, 1, 1>(s, rg, Opnd<T>{(T *)x, xrp, xsp}, Opnd<T>{}, Opnd<T>{}, Opnd<T>{},
                               [kind] __device__(uint64_t, T &a, T &, T &, T &) { a = act_forward<T>(kind, a); });
    });
}

int wk_activation_dev(wk_stream *s, int dtype, int kind, const uint64_t shape3[3], const void *out, uint64_t orp,
                      uint64_t osp, void *dev, uint64_t drp, uint64_t dsp) {
    int rc = bind(s);
    if (rc) return rc;
    Region rg;
    if ((rc = check_region(shape3, rg))) return rc;
    if (kind != WK_ACT_SIGMOID && kind != WK_ACT_TANH) return WK_E_INVALID_VALUE;
    return dispatch_float(dtype, [&]<typename T>() -> int {
        if (check_opnd<T>(rg, out, orp, osp) || check_opnd<T>(rg, dev, drp, dsp)) return WK_E_INVALID_VALUE;
        return ew_launch<T, 2, 1>(s, rg, Opnd<T>{(T *)dev, drp, dsp}, Opnd<T>{(T *)out, orp, osp}, Opnd<T>{}, Opnd<T>{},
                               [kind] __device__(uint64_t, T &d, T &y, T &, T &) { d = act_derivative<T>(kind, y); });
    });
}

int wk_bias_activation(wk_stream *s, int dtype, int kind, uint64_t rows, uint64_t cols, void *out, uint64_t out_pitch,
                       const void *bias) {
    int rc = bind(s);
    if (rc) return rc;
    if (!rows || !cols || !out || out_pitch < cols) return WK_E_INVALID_VALUE;
    if (kind != WK_ACT_NONE && kind != WK_ACT_SIGMOID && kind != WK_ACT_TANH) return WK_E_INVALID_VALUE;
    const Region rg{1, rows, cols};
    return dispatch_float(dtype, [&]<typename T>() -> int {
        const T *b = static_cast<const T *>(bias); // may be null: activation only
        return ew_launch<T, 1, 1>(s, rg, Opnd<T>{(T *)out, out_pitch, 0}, Opnd<T>{}, Opnd<T>{}, Opnd<T>{},
                               [kind, b] __device__(uint64_t c, T &a, T &, T &, T &) {
                                   if (b) a += b[c];
                                   a = act_forward<T>(kind, a);
                               });
    });
}

int wk_bias_step(wk_stream *s, int dtype, uint64_t rows, uint64_t cols, const void *sens, uint64_t pitch, void *bias_grad) {
    int rc = bind(s);
    if (rc) return rc;
    if (!rows || !cols || !sens || !bias_grad || pitch < cols) return WK_E_INVALID_VALUE;
    if ((cols + 63) / 64 > 0x7fffffffull) return WK_E_INVALID_VALUE;
    return dispatch_float(dtype, [&]<typename T>() -> int {
        // as many bands as its share of the stream's scratch holds partials for
        return colsum_two_pass<T>(s, rows, cols, static_cast<const T *>(sens), pitch, static_cast<T *>(bias_grad), s->scratch,
                                  s->scratch_bytes < WK_BIAS_STEP_SCRATCH_BYTES ? s->scratch_bytes : WK_BIAS_STEP_SCRATCH_BYTES);
    });
}

int wk_bias_step_static(wk_stream *s, int dtype, uint64_t rows, uint64_t cols, const void *sens, uint64_t pitch,
                        void *bias_grad) {
    int rc = bind(s);
    if (rc) return rc;
    if (!rows || !cols || !sens || !bias_grad || pitch < cols) return WK_E_INVALID_VALUE;
    if (dtype != WK_F32 && dtype != WK_F64) return WK_E_TYPE_NOT_SUPPORTED;
    const size_t esize = wk_dtype_size(dtype);
    // at least two bands of partials must fit, whatever the row count: a row is at most half the array
    if (cols > STATIC_SCRATCH_BYTES / 2 / esize) return WK_E_SCRATCH_TOO_SMALL;
    const int ordinal = s->dev->ordinal;
    void *ptr = ordinal < STATIC_SCRATCH_MAX_DEVICES ? g_static_scratch[ordinal].load(std::memory_order_acquire) : nullptr;
    if (!ptr) return WK_E_INVALID_VALUE; // the device was not opened through wk_device_open
    return dispatch_float(dtype, [&]<typename T>() -> int {
        return colsum_two_pass<T>(s, rows, cols, static_cast<const T *>(sens), pitch, static_cast<T *>(bias_grad), ptr,
                                  STATIC_SCRATCH_BYTES);
    });
}

int wk_sensitivity_step(wk_stream *s, int dtype, int kind, uint64_t rows, uint64_t cols, const void *out, uint64_t out_pitch,
                        void *sens, uint64_t sens_pitch, void *dev, uint64_t dev_pitch, void *bias_grad) {
    int rc = bind(s);
    if (rc) return rc;
    if (kind != WK_ACT_NONE && kind != WK_ACT_SIGMOID && kind != WK_ACT_TANH) return WK_E_INVALID_VALUE;
    if (dtype != WK_F32 && dtype != WK_F64) return WK_E_TYPE_NOT_SUPPORTED;
    if (!rows || !cols || !sens || !dev || sens_pitch < cols || dev_pitch < cols) return WK_E_INVALID_VALUE;
    if (kind != WK_ACT_NONE && (!out || out_pitch < cols)) return WK_E_INVALID_VALUE;
    return dispatch_float(dtype, [&]<typename T>() -> int {
        constexpr uint64_t VE = 16 / sizeof(T);
        const auto aligned = [&](const void *p, uint64_t pitch) { return !p || ((reinterpret_cast<uintptr_t>(p) & 15u) == 0 && pitch % VE == 0); };
        const bool vec = aligned(kind != WK_ACT_NONE ? out : nullptr, out_pitch) && aligned(sens, sens_pitch) && aligned(dev, dev_pitch);
        const uint64_t per_block = 64 * (vec ? VE : 1);
        if ((cols + per_block - 1) / per_block > 0x7fffffffull) return WK_E_INVALID_VALUE;
        // the bands of wk_bias_step, so that the bias gradient is the same bits as from that call
        uint64_t bands, band_rows;
        colsum_plan(rows, cols, sizeof(T), s->scratch_bytes < WK_BIAS_STEP_SCRATCH_BYTES ? s->scratch_bytes : WK_BIAS_STEP_SCRATCH_BYTES,
                    bands, band_rows);
        T *bg = static_cast<T *>(bias_grad);
        T *partial = !bg ? nullptr : bands > 1 ? static_cast<T *>(s->scratch) : bg;
        const dim3 grid((unsigned)((cols + per_block - 1) / per_block), (unsigned)bands), block(64, 4);
        if (vec)
            hipLaunchKernelGGL((sens_step_kernel<T, true>), grid, block, 0, s->stream, kind, static_cast<const T *>(out), out_pitch,
                               static_cast<T *>(sens), sens_pitch, static_cast<T *>(dev), dev_pitch, rows, cols, band_rows, partial);
        else
            hipLaunchKernelGGL((sens_step_kernel<T, false>), grid, block, 0, s->stream, kind, static_cast<const T *>(out), out_pitch,
                               static_cast<T *>(sens), sens_pitch, static_cast<T *>(dev), dev_pitch, rows, cols, band_rows, partial);
        int lrc = launch_status();
        if (lrc || !bg || bands == 1) return lrc;
        hipLaunchKernelGGL((colsum_bands_kernel<T>), dim3((unsigned)((cols + 63) / 64), 1), dim3(64, 4), 0, s->stream,
                           static_cast<const T *>(partial), bands, cols, cols, bands, bg);
        return launch_status();
    });
}

int wk_adam_step_multi(wk_stream *s, int dtype, uint32_t count, const wk_adam_tensor *host_tensors, double lr, double beta1,
                       double beta2, double eps, uint64_t step) {
    int rc = bind(s);
    if (rc) return rc;
    if (!count) return WK_OK;
    if (!host_tensors || step == 0) return WK_E_INVALID_VALUE;
    if (dtype != WK_F32 && dtype != WK_F64) return WK_E_TYPE_NOT_SUPPORTED;
    const double bc1 = 1.0 - std::pow(beta1, (double)step), bc2 = 1.0 - std::pow(beta2, (double)step);
    return dispatch_float(dtype, [&]<typename T>() -> int {
        constexpr uint64_t VE = 16 / sizeof(T);
        // every tensor is validated before anything is launched
        bool vec = true;
        for (uint32_t i = 0; i < count; ++i) {
            const wk_adam_tensor &t = host_tensors[i];
            Region rg;
            if (check_region(t.shape3, rg)) return WK_E_INVALID_VALUE;
            if (check_opnd<T>(rg, t.w, t.w_row_pitch, t.w_slice_pitch) || check_opnd<T>(rg, t.g, t.g_row_pitch, t.g_slice_pitch) ||
                check_opnd<T>(rg, t.m, t.mv_row_pitch, t.mv_slice_pitch) || check_opnd<T>(rg, t.v, t.mv_row_pitch, t.mv_slice_pitch))
                return WK_E_INVALID_VALUE;
            // the one-launch kernel wants 16-byte rows and slices that follow one another at the row pitch
            const auto ok = [&](const void *p, uint64_t rp, uint64_t sp) {
                return (reinterpret_cast<uintptr_t>(p) & 15u) == 0 && (rg.rows * rg.depth == 1 || rp % VE == 0) &&
                       (rg.depth == 1 || sp == rg.rows * rp);
            };
            vec = vec && ok(t.w, t.w_row_pitch, t.w_slice_pitch) && ok(t.g, t.g_row_pitch, t.g_slice_pitch) &&
                  ok(t.m, t.mv_row_pitch, t.mv_slice_pitch) && ok(t.v, t.mv_row_pitch, t.mv_slice_pitch);
        }
        if (!vec || count == 1) { // the same update, one launch per tensor
            for (uint32_t i = 0; i < count; ++i) {
                const wk_adam_tensor &t = host_tensors[i];
                const int r = wk_adam_step(s, dtype, t.shape3, t.w, t.w_row_pitch, t.w_slice_pitch, t.g, t.g_row_pitch, t.g_slice_pitch,
                                           t.m, t.v, t.mv_row_pitch, t.mv_slice_pitch, lr, beta1, beta2, eps, step);
                if (r) return r;
            }
            return WK_OK;
        }
        for (uint32_t first = 0; first < count; first += ADAM_MULTI_MAX) {
            AdamMultiArgs<T> a{};
            a.count = (int)(count - first < (uint32_t)ADAM_MULTI_MAX ? count - first : ADAM_MULTI_MAX);
            a.b1 = (T)beta1; a.b2 = (T)beta2; a.ib1 = (T)(1.0 - beta1); a.ib2 = (T)(1.0 - beta2);
            a.step_size = (T)(lr / bc1); a.inv_sqrt_bc2 = (T)(1.0 / std::sqrt(bc2)); a.eps = (T)eps;
            uint64_t blocks = 0;
            for (int i = 0; i < a.count; ++i) {
                const wk_adam_tensor &t = host_tensors[first + i];
                a.w[i] = static_cast<T *>(t.w); a.g[i] = static_cast<const T *>(t.g);
                a.m[i] = static_cast<T *>(t.m); a.v[i] = static_cast<T *>(t.v);
                a.rows[i] = t.shape3[0] * t.shape3[1]; a.cols[i] = t.shape3[2];
                a.wrp[i] = t.w_row_pitch; a.grp[i] = t.g_row_pitch; a.mrp[i] = t.mv_row_pitch;
                const uint64_t vecs = a.rows[i] * ((a.cols[i] + VE - 1) / VE);
                uint64_t want = (vecs + EW_BLOCK - 1) / EW_BLOCK;
                if (want > 16384) want = 16384; // grid stride beyond that
                a.first_block[i] = (uint32_t)blocks;
                blocks += want ? want : 1;
            }
            a.first_block[a.count] = (uint32_t)blocks;
            hipLaunchKernelGGL((adam_multi_kernel<T>), dim3((unsigned)blocks), dim3(EW_BLOCK), 0, s->stream, a);
            const int lrc = launch_status();
            if (lrc) return lrc;
        }
        return WK_OK;
    });
}

int wk_mse(wk_stream *s, int dtype, const uint64_t shape3[3], const void *output, uint64_t orp, uint64_t osp,
           const void *expected, uint64_t erp, uint64_t esp, void *error, uint64_t rrp, uint64_t rsp, void *dev,
           uint64_t drp, uint64_t dsp) {
    int rc = bind(s);
    if (rc) return rc;
    Region rg;
    if ((rc = check_region(shape3, rg))) return rc;
    return dispatch_float(dtype, [&]<typename T>() -> int {
        if (check_opnd<T>(rg, output, orp, osp) || check_opnd<T>(rg, expected, erp, esp) || check_opnd<T>(rg, error, rrp, rsp))
            return WK_E_INVALID_VALUE;
        if (dev) {
            if (check_opnd<T>(rg, dev, drp, dsp)) return WK_E_INVALID_VALUE;
            return ew_launch<T, 4, 3>(s, rg, Opnd<T>{(T *)error, rrp, rsp}, Opnd<T>{(T *)dev, drp, dsp},
                                   Opnd<T>{(T *)output, orp, osp}, Opnd<T>{(T *)expected, erp, esp},
                                   [] __device__(uint64_t, T &err2, T &d, T &o, T &e) {
                                       const T err = e - o;
                                       err2 = err * err;
                                       d = T(-2) * err;
                                   });
        }
        return ew_launch<T, 3, 1>(s, rg, Opnd<T>{(T *)error, rrp, rsp}, Opnd<T>{(T *)output, orp, osp},
                               Opnd<T>{(T *)expected, erp, esp}, Opnd<T>{},
                               [] __device__(uint64_t, T &err2, T &o, T &e, T &) {
                                   const T err = e - o;
                                   err2 = err * err;
                               });
    });
}

size_t wk_sum_workspace_bytes(int dtype) { return SUM_PARTIALS * wk_dtype_size(dtype); }

int wk_sum(wk_stream *s, int dtype, const uint64_t shape3[3], const void *x, uint64_t xrp, uint64_t xsp, void *workspace,
           void *dev_result, double scale) {
    int rc = bind(s);
    if (rc) return rc;
    Region rg;
    if ((rc = check_region(shape3, rg))) return rc;
    if (!workspace || !dev_result) return WK_E_INVALID_VALUE;
    return dispatch_float(dtype, [&]<typename T>() -> int {
        if (check_opnd<T>(rg, x, xrp, xsp)) return WK_E_INVALID_VALUE;
        // rows and slices that follow each other without gaps are one long row
        Region flat = rg;
        uint64_t rp = xrp, sp = xsp;
        if (rg.cols == xrp && (rg.depth == 1 || xsp == rg.rows * xrp)) {
            flat = Region{1, 1, rg.depth * rg.rows * rg.cols};
            rp = sp = flat.cols;
        }
        const bool vec = reinterpret_cast<uintptr_t>(x) % 16 == 0 && flat.cols >= 16 / sizeof(T) &&
                         (flat.depth * flat.rows == 1 || ((rp * sizeof(T)) % 16 == 0 && (sp * sizeof(T)) % 16 == 0));
        if (vec)
            hipLaunchKernelGGL((sum_pass1_kernel<T, true>), dim3(SUM_PARTIALS), dim3(256), 0, s->stream, static_cast<const T *>(x),
                               flat, rp, sp, static_cast<T *>(workspace));
        else
            hipLaunchKernelGGL((sum_pass1_kernel<T, false>), dim3(SUM_PARTIALS), dim3(256), 0, s->stream, static_cast<const T *>(x),
                               rg, xrp, xsp, static_cast<T *>(workspace));
        int lrc = launch_status();
        if (lrc) return lrc;
        hipLaunchKernelGGL((sum_pass2_kernel<T>), dim3(1), dim3(256), 0, s->stream, static_cast<const T *>(workspace),
                           static_cast<T *>(dev_result), static_cast<T>(scale));
        return launch_status();
    });
}

int wk_adam_step(wk_stream *s, int dtype, const uint64_t shape3[3], void *w, uint64_t wrp, uint64_t wsp, const void *g,
                 uint64_t grp, uint64_t gsp, void *m, void *v, uint64_t mrp, uint64_t msp, double lr, double beta1,
                 double beta2, double eps, uint64_t step) {
    int rc = bind(s);
    if (rc) return rc;
    Region rg;
    if ((rc = check_region(shape3, rg))) return rc;
    if (step == 0) return WK_E_INVALID_VALUE;
    const double bc1 = 1.0 - std::pow(beta1, (double)step), bc2 = 1.0 - std::pow(beta2, (double)step);
    return dispatch_float(dtype, [&]<typename T>() -> int {
        if (check_opnd<T>(rg, w, wrp, wsp) || check_opnd<T>(rg, g, grp, gsp) || check_opnd<T>(rg, m, mrp, msp) ||
            check_opnd<T>(rg, v, mrp, msp))
            return WK_E_INVALID_VALUE;
        const T b1 = (T)beta1, b2 = (T)beta2, ib1 = (T)(1.0 - beta1), ib2 = (T)(1.0 - beta2);
        const T step_size = (T)(lr / bc1), inv_sqrt_bc2 = (T)(1.0 / std::sqrt(bc2)), e = (T)eps;
        return ew_launch<T, 4, 7>(s, rg, Opnd<T>{(T *)w, wrp, wsp}, Opnd<T>{(T *)m, mrp, msp}, Opnd<T>{(T *)v, mrp, msp},
                               Opnd<T>{(T *)g, grp, gsp},
                               [=] __device__(uint64_t, T &wv, T &mv, T &vv, T &gv) {
                                   adam_update<T>(wv, mv, vv, gv, b1, ib1, b2, ib2, step_size, inv_sqrt_bc2, e);
                               });
    });
}

} // extern "C"
