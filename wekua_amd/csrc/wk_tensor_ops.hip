// Tensor support operations around the BLAS path: N-d transpose, random.uniform, and the
// real <-> complex conversions.
//
// Reference kernels restated here: src/tensor/kernels/transpose.cl, src/tensor/random/kernels/
// uniform.cl, src/tensor/convertions/kernels/{to_complex,to_real}.cl.  All are HBM-bound data
// movement; they address tensors through per-dimension element pitches so that only logical
// elements are touched.
#include "wk_internal.hpp"

#include <cstring>

using namespace wk;

namespace {

constexpr int MAX_DIMS = WK_MAX_DIMS;

// ---- transpose ---------------------------------------------------------------------------------
// `batch` dimensions are every dimension except the two that take part in the tile; each has an
// extent, a source pitch and a destination pitch (already permuted by the host).
struct TransposeArgs {
    int nbatch;
    uint64_t bshape[MAX_DIMS], bsrc[MAX_DIMS], bdst[MAX_DIMS];
    uint64_t rows, cols;         // extents of the two tiled source dimensions (cols: the contiguous one)
    uint64_t src_row_pitch;      // source: element (r, c) at r * src_row_pitch + c
    uint64_t dst_row_pitch;      // destination of the tiled kernel: element (r, c) lands at c * dst_row_pitch + r
    uint64_t dst_col_pitch;      // destination of the row kernel: element (r, c) lands at r * dst_row_pitch + c * 1
};

__device__ __forceinline__ void batch_offsets(const TransposeArgs &a, uint64_t b, uint64_t &so, uint64_t &dof) {
    so = 0;
    dof = 0;
    for (int x = a.nbatch - 1; x >= 0; --x) {
        const uint64_t c = b % a.bshape[x];
        b /= a.bshape[x];
        so += c * a.bsrc[x];
        dof += c * a.bdst[x];
    }
}

// The contiguous dimension takes part in the swap: T x T tiles go through LDS so that both the read
// (along source columns) and the write (along what becomes the destination's contiguous
// dimension) are runs of consecutive addresses.  With VEC every lane moves 16 bytes (VE elements)
// per access on both sides; the host grants VEC only when bases and pitches allow it.
template <typename E, int T, bool VEC>
__global__ __launch_bounds__(256) void transpose_tiled_kernel(const E *__restrict__ src, E *__restrict__ dst, TransposeArgs a,
                                                              uint64_t tiles_c) {
    constexpr int VE = VEC ? 16 / (int)sizeof(E) : 1;
    constexpr int VPR = T / VE;            // vectors per tile row
    constexpr int ITERS = T * VPR / 256;   // vectors per thread
    static_assert(T % VE == 0 && (T * VPR) % 256 == 0, "tile must split evenly over 256 threads");
    __shared__ E tile[T][T + 1];
    const uint64_t tr = blockIdx.x / tiles_c, tc = blockIdx.x % tiles_c;
    uint64_t so, dof;
    batch_offsets(a, blockIdx.y, so, dof);
    const uint64_t r0 = tr * T, c0 = tc * T;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = it * 256 + (int)threadIdx.x;
        const int r = v / VPR, c = (v % VPR) * VE;
        if (r0 + r >= a.rows) continue;
        const E *p = src + so + (r0 + r) * a.src_row_pitch + c0 + c;
        if (VEC && c0 + c + VE <= a.cols) {
            typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
            // streamed (read once, written once) for elements of up to four bytes: f32 8192^2 104 -> 95 us, u8
            // 16384^2 110 -> 103; the 8- and 16-byte types measured 4 % slower with it
            const u32x4 raw = sizeof(E) <= 4 ? __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p))
                                             : *reinterpret_cast<const u32x4 *>(p);
            E tmp[VE];
            __builtin_memcpy(tmp, &raw, 16);
#pragma unroll
            for (int e = 0; e < VE; ++e) tile[r][c + e] = tmp[e];
        } else {
            for (int e = 0; e < VE; ++e)
                if (c0 + c + e < a.cols) tile[r][c + e] = p[e];
        }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int v = it * 256 + (int)threadIdx.x;
        const int c = v / VPR, r = (v % VPR) * VE; // destination row = source column c
        if (c0 + c >= a.cols) continue;
        E *p = dst + dof + (c0 + c) * a.dst_row_pitch + r0 + r;
        if (VEC && r0 + r + VE <= a.rows) {
            E tmp[VE];
#pragma unroll
            for (int e = 0; e < VE; ++e) tmp[e] = tile[r + e][c];
            typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
            u32x4 raw;
            __builtin_memcpy(&raw, tmp, 16);
            if (sizeof(E) <= 4) __builtin_nontemporal_store(raw, reinterpret_cast<u32x4 *>(p));
            else *reinterpret_cast<u32x4 *>(p) = raw;
        } else {
            for (int e = 0; e < VE; ++e)
                if (r0 + r + e < a.rows) p[e] = tile[r + e][c];
        }
    }
}

// The contiguous dimension stays where it is: whole rows move, reads and writes both run along it.
// blockIdx.y walks (batch, row) pairs, blockIdx.x the columns.
template <typename E, bool VEC>
__global__ __launch_bounds__(256) void transpose_rows_kernel(const E *__restrict__ src, E *__restrict__ dst, TransposeArgs a,
                                                             uint64_t total_rows) {
    constexpr int VE = VEC ? 16 / (int)sizeof(E) : 1;
    const uint64_t cols_v = (a.cols + VE - 1) / VE;
    for (uint64_t br = blockIdx.y; br < total_rows; br += gridDim.y) {
        uint64_t so, dof;
        batch_offsets(a, br / a.rows, so, dof);
        const uint64_t r = br % a.rows;
        const E *sp = src + so + r * a.src_row_pitch;
        E *dp = dst + dof + r * a.dst_row_pitch;
        for (uint64_t cv = blockIdx.x * 256ull + threadIdx.x; cv < cols_v; cv += (uint64_t)gridDim.x * 256ull) {
            const uint64_t c = cv * VE;
            if (VEC && c + VE <= a.cols) {
                E tmp[VE];
                __builtin_memcpy(tmp, __builtin_assume_aligned(sp + c, 16), 16);
                __builtin_memcpy(__builtin_assume_aligned(dp + c, 16), tmp, 16);
            } else {
                for (int e = 0; e < VE && c + e < a.cols; ++e) dp[c + e] = sp[c + e];
            }
        }
    }
}

struct alignas(16) E16 {
    uint64_t lo, hi;
};

template <typename F> int dispatch_elem_size(size_t es, F &&f) {
    switch (es) {
    case 1: return f.template operator()<uint8_t>();
    case 2: return f.template operator()<uint16_t>();
    case 4: return f.template operator()<uint32_t>();
    case 8: return f.template operator()<uint64_t>();
    case 16: return f.template operator()<E16>();
    default: return WK_E_TYPE_NOT_SUPPORTED;
    }
}

// ---- random.uniform -----------------------------------------------------------------------------
// The reference's hash (uniform.cl:31-55), restated with its operator precedence: in
// `x0 ^ rotl(x0,49) ^ rotl(x0,24) * P` the product binds first, likewise in `x1 ^ ((x1>>35)+8) * P`;
// `(seed & 0xFFFFFFFF00000000) << 32` is zero in 64 bits, so the seed enters unmixed; the two
// halves of the index trade places.
__host__ __device__ inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
__host__ __device__ inline uint64_t wk_hash64(uint64_t index, uint64_t seed) {
    constexpr uint64_t P = 0x9FB21C651E98DF25ull;
    const uint64_t key = (0x7C01812CF721AD1Cull ^ 0xDED46DE9839097DBull) - seed;
    const uint64_t combined = ((index & 0xffffffffull) << 32) + (index >> 32);
    const uint64_t x0 = combined ^ key;
    const uint64_t x1 = x0 ^ rotl64(x0, 49) ^ (rotl64(x0, 24) * P);
    const uint64_t x2 = x1 ^ (((x1 >> 35) + 8) * P);
    return x2 ^ (x2 >> 28);
}

// R: storage type of one real component.  IS_FLOAT / RANGED select the branch of uniform.cl:75-180.
template <typename R, bool IS_FLOAT, bool RANGED, typename MinT>
__device__ __forceinline__ R uniform_value(uint64_t h, MinT min_value, MinT range) {
    if constexpr (RANGED) {
        const double normalized = (double)h / 18446744073709551616.0; // (double)ULONG_MAX is 2^64
        return (R)(MinT)((double)min_value + normalized * (double)range);
    } else if constexpr (IS_FLOAT) {
        return (R)h / (R)18446744073709551616.0;
    } else {
        return (R)h; // low bits; the signed types reinterpret them
    }
}

// blockIdx.y walks the rows (all slices), blockIdx.x the columns: one division per row, none per element.
template <typename R, bool CPLX, bool IS_FLOAT, bool RANGED, typename MinT>
__global__ __launch_bounds__(256) void uniform_kernel(R *__restrict__ out, uint64_t rows, uint64_t cols, uint64_t total_rows,
                                                      uint64_t row_pitch, uint64_t slice_pitch, uint64_t seed, MinT min_value,
                                                      MinT range) {
    for (uint64_t row = blockIdx.y; row < total_rows; row += gridDim.y) {
        const uint64_t off0 = (row / rows) * slice_pitch + (row % rows) * row_pitch;
        const uint64_t idx0 = row * cols;
        for (uint64_t k = blockIdx.x * 256ull + threadIdx.x; k < cols; k += (uint64_t)gridDim.x * 256ull) {
            const uint64_t idx = idx0 + k, off = off0 + k;
            if constexpr (CPLX) {
                out[2 * off] = uniform_value<R, IS_FLOAT, RANGED, MinT>(wk_hash64(idx << 1, seed), min_value, range);
                out[2 * off + 1] = uniform_value<R, IS_FLOAT, RANGED, MinT>(wk_hash64((idx << 1) + 1, seed), min_value, range);
            } else {
                out[off] = uniform_value<R, IS_FLOAT, RANGED, MinT>(wk_hash64(idx, seed), min_value, range);
            }
        }
    }
}

// grid for the row-wise kernels: x over 256-column chunks, y over rows, about 16k blocks at most
dim3 row_grid(uint64_t cols, uint64_t total_rows) {
    uint64_t gx = (cols + 255) / 256;
    if (gx < 1) gx = 1;
    if (gx > 16384) gx = 16384;
    uint64_t gy = (16384 + gx - 1) / gx;
    if (gy > total_rows) gy = total_rows;
    if (gy > 65535) gy = 65535;
    if (gy < 1) gy = 1;
    return dim3((unsigned)gx, (unsigned)gy);
}

unsigned grid_for(uint64_t total) {
    const uint64_t want = (total + 255) / 256;
    return (unsigned)(want < 1 ? 1 : (want > 65536 ? 65536 : want));
}

template <typename R, typename S, bool IS_FLOAT>
int launch_uniform(wk_stream *s, bool cplx, void *ptr, const uint64_t shape3[3], uint64_t rp, uint64_t sp, uint64_t seed,
                   const void *host_min, const void *host_range) {
    const uint64_t total_rows = shape3[0] * shape3[1];
    const dim3 grid = row_grid(shape3[2], total_rows);
    R *out = static_cast<R *>(ptr);
    S mn{}, rg{};
    if (host_min) {
        std::memcpy(&mn, host_min, sizeof(S));
        std::memcpy(&rg, host_range, sizeof(S));
    }
#define WK_U(CP, RA)                                                                                                        \
    hipLaunchKernelGGL((uniform_kernel<R, CP, IS_FLOAT, RA, S>), grid, dim3(256), 0, s->stream, out, shape3[1], shape3[2],      \
                       total_rows, rp, sp, seed, mn, rg)
    if (cplx) {
        if (host_min) WK_U(true, true);
        else WK_U(true, false);
    } else {
        if (host_min) WK_U(false, true);
        else WK_U(false, false);
    }
#undef WK_U
    return launch_status();
}

// ---- real <-> complex -------------------------------------------------------------------------
template <typename E, bool TO_COMPLEX>
__global__ __launch_bounds__(256) void complex_part_kernel(const E *__restrict__ src, E *__restrict__ dst, uint64_t rows,
                                                           uint64_t cols, uint64_t total_rows, uint64_t srp, uint64_t ssp,
                                                           uint64_t drp, uint64_t dsp, unsigned part) {
    for (uint64_t row = blockIdx.y; row < total_rows; row += gridDim.y) {
        const uint64_t i = row / rows, j = row % rows;
        const E *sp = src + (TO_COMPLEX ? 1 : 2) * (i * ssp + j * srp);
        E *dp = dst + (TO_COMPLEX ? 2 : 1) * (i * dsp + j * drp);
        for (uint64_t k = blockIdx.x * 256ull + threadIdx.x; k < cols; k += (uint64_t)gridDim.x * 256ull) {
            if constexpr (TO_COMPLEX) dp[2 * k + part] = sp[k];
            else dp[k] = sp[2 * k + part];
        }
    }
}

int check_part_args(const uint64_t shape3[3], const void *src, uint64_t srp, uint64_t ssp, const void *dst, uint64_t drp,
                    uint64_t dsp, int space) {
    if (!shape3 || !src || !dst || (space != 0 && space != 1)) return WK_E_INVALID_VALUE;
    if (!shape3[0] || !shape3[1] || !shape3[2]) return WK_E_INVALID_VALUE;
    if (shape3[1] > 1 && (srp < shape3[2] || drp < shape3[2])) return WK_E_INVALID_VALUE;
    if (shape3[0] > 1 && (ssp < shape3[1] * srp || dsp < shape3[1] * drp)) return WK_E_INVALID_VALUE;
    return WK_OK;
}

} // namespace

extern "C" {

int wk_transpose(wk_stream *s, int dtype, int ndim, const uint64_t *shape, const uint64_t *src_pitches,
                 const uint64_t *dst_pitches, int dim0, int dim1, const void *src, void *dst) {
    int rc = bind(s);
    if (rc) return rc;
    if (!shape || !src_pitches || !dst_pitches || !src || !dst || ndim < 1 || ndim > MAX_DIMS) return WK_E_INVALID_VALUE;
    if (dim0 < 0 || dim1 < 0 || dim0 >= ndim || dim1 >= ndim || dim0 == dim1) return WK_E_INVALID_VALUE;
    if (src_pitches[ndim - 1] != 1 || dst_pitches[ndim - 1] != 1) return WK_E_INVALID_VALUE;
    const size_t es = wk_dtype_size(dtype);
    if (!es) return WK_E_TYPE_NOT_SUPPORTED;
    for (int x = 0; x < ndim; ++x)
        if (!shape[x]) return WK_E_INVALID_VALUE;
    if (dim0 > dim1) {
        const int t = dim0;
        dim0 = dim1;
        dim1 = t;
    }
    // destination dimension x holds source dimension perm(x); source dimension x is therefore
    // walked with the destination pitch of perm(x)
    auto dst_pitch_of_src_dim = [&](int x) { return dst_pitches[x == dim0 ? dim1 : (x == dim1 ? dim0 : x)]; };
    const int last = ndim - 1;
    TransposeArgs a{};
    const bool tiled = dim1 == last;
    // tiled: rows = source dim0, cols = source last dim.  rows kernel: rows = second-to-last
    // source dimension that is not batch..., kept simple: rows = 1 row per batch entry unless
    // ndim >= 2, where the second-to-last dimension is the row dimension.
    int row_dim = tiled ? dim0 : (ndim >= 2 ? ndim - 2 : -1);
    a.cols = shape[last];
    a.rows = row_dim >= 0 ? shape[row_dim] : 1;
    a.src_row_pitch = row_dim >= 0 ? src_pitches[row_dim] : 0;
    a.dst_row_pitch = tiled ? dst_pitch_of_src_dim(last) : (row_dim >= 0 ? dst_pitch_of_src_dim(row_dim) : 0);
    uint64_t batches = 1;
    for (int x = 0; x < ndim; ++x) {
        if (x == last || x == row_dim) continue;
        a.bshape[a.nbatch] = shape[x];
        a.bsrc[a.nbatch] = src_pitches[x];
        a.bdst[a.nbatch] = dst_pitch_of_src_dim(x);
        batches *= shape[x];
        ++a.nbatch;
    }
    // the tiled kernel puts one batch entry on each blockIdx.y; the y dimension of a grid is limited
    if (tiled && batches > 65535) return WK_E_INVALID_VALUE;
    const bool aligned16 = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u) == 0;
    return dispatch_elem_size(es, [&]<typename E>() -> int {
        if (tiled) {
            // tile edge: at least 128 bytes of every row segment (64 elements of 4 and 8 bytes, 128 of 1 and 2, 32 of 16)
            constexpr int T = sizeof(E) == 16 ? 32 : (sizeof(E) >= 4 ? 64 : 128);
            constexpr uint64_t VE = 16 / sizeof(E);
            bool vec = aligned16 && a.src_row_pitch % VE == 0 && a.dst_row_pitch % VE == 0;
            for (int x = 0; x < a.nbatch; ++x) vec = vec && a.bsrc[x] % VE == 0 && a.bdst[x] % VE == 0;
            const uint64_t tiles_r = (a.rows + T - 1) / T, tiles_c = (a.cols + T - 1) / T;
            if (tiles_r * tiles_c > 0x7fffffffull) return WK_E_INVALID_VALUE;
            const dim3 grid((unsigned)(tiles_r * tiles_c), (unsigned)batches);
            if (vec)
                hipLaunchKernelGGL((transpose_tiled_kernel<E, T, true>), grid, dim3(256), 0, s->stream, static_cast<const E *>(src),
                                   static_cast<E *>(dst), a, tiles_c);
            else
                hipLaunchKernelGGL((transpose_tiled_kernel<E, T, false>), grid, dim3(256), 0, s->stream, static_cast<const E *>(src),
                                   static_cast<E *>(dst), a, tiles_c);
        } else {
            const uint64_t total_rows = batches * a.rows;
            constexpr uint64_t VE = 16 / sizeof(E);
            bool vec = aligned16 && a.src_row_pitch % VE == 0 && a.dst_row_pitch % VE == 0;
            for (int x = 0; x < a.nbatch; ++x) vec = vec && a.bsrc[x] % VE == 0 && a.bdst[x] % VE == 0;
            if (vec)
                hipLaunchKernelGGL((transpose_rows_kernel<E, true>), row_grid((a.cols + VE - 1) / VE, total_rows), dim3(256), 0,
                                   s->stream, static_cast<const E *>(src), static_cast<E *>(dst), a, total_rows);
            else
                hipLaunchKernelGGL((transpose_rows_kernel<E, false>), row_grid(a.cols, total_rows), dim3(256), 0, s->stream,
                                   static_cast<const E *>(src), static_cast<E *>(dst), a, total_rows);
        }
        return launch_status();
    });
}

int wk_random_uniform(wk_stream *s, int dtype, const uint64_t shape3[3], void *ptr, uint64_t row_pitch, uint64_t slice_pitch,
                      uint64_t seed, const void *host_min, const void *host_range) {
    int rc = bind(s);
    if (rc) return rc;
    if (!shape3 || !ptr || !shape3[0] || !shape3[1] || !shape3[2]) return WK_E_INVALID_VALUE;
    if ((host_min == nullptr) != (host_range == nullptr)) return WK_E_INVALID_VALUE;
    if (shape3[1] > 1 && row_pitch < shape3[2]) return WK_E_INVALID_VALUE;
    if (shape3[0] > 1 && slice_pitch < shape3[1] * row_pitch) return WK_E_INVALID_VALUE;
    if (dtype < 0 || dtype >= WK_DTYPE_COUNT) return WK_E_TYPE_NOT_SUPPORTED;
    const bool cplx = dtype >= 10;
    switch (dtype % 10) {
    case WK_I8: return launch_uniform<uint8_t, int8_t, false>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    case WK_U8: return launch_uniform<uint8_t, uint8_t, false>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    case WK_I16: return launch_uniform<uint16_t, int16_t, false>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    case WK_U16: return launch_uniform<uint16_t, uint16_t, false>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    case WK_I32: return launch_uniform<uint32_t, int32_t, false>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    case WK_U32: return launch_uniform<uint32_t, uint32_t, false>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    case WK_I64: return launch_uniform<uint64_t, int64_t, false>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    case WK_U64: return launch_uniform<uint64_t, uint64_t, false>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    case WK_F32: return launch_uniform<float, float, true>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    default: return launch_uniform<double, double, true>(s, cplx, ptr, shape3, row_pitch, slice_pitch, seed, host_min, host_range);
    }
}

uint64_t wk_random_hash(uint64_t index, uint64_t seed) { return wk_hash64(index, seed); }

int wk_to_complex(wk_stream *s, int real_dtype, const uint64_t shape3[3], const void *src, uint64_t srp, uint64_t ssp, void *dst,
                  uint64_t drp, uint64_t dsp, int space) {
    int rc = bind(s);
    if (rc) return rc;
    if ((rc = check_part_args(shape3, src, srp, ssp, dst, drp, dsp, space))) return rc;
    if (real_dtype < 0 || real_dtype >= 10) return WK_E_TYPE_NOT_SUPPORTED;
    const uint64_t total_rows = shape3[0] * shape3[1];
    return dispatch_elem_size(wk_dtype_size(real_dtype), [&]<typename E>() -> int {
        hipLaunchKernelGGL((complex_part_kernel<E, true>), row_grid(shape3[2], total_rows), dim3(256), 0, s->stream,
                           static_cast<const E *>(src), static_cast<E *>(dst), shape3[1], shape3[2], total_rows, srp, ssp, drp, dsp,
                           (unsigned)space);
        return launch_status();
    });
}

int wk_to_real(wk_stream *s, int real_dtype, const uint64_t shape3[3], const void *src, uint64_t srp, uint64_t ssp, void *dst,
               uint64_t drp, uint64_t dsp, int space) {
    int rc = bind(s);
    if (rc) return rc;
    if ((rc = check_part_args(shape3, src, srp, ssp, dst, drp, dsp, space))) return rc;
    if (real_dtype < 0 || real_dtype >= 10) return WK_E_TYPE_NOT_SUPPORTED;
    const uint64_t total_rows = shape3[0] * shape3[1];
    return dispatch_elem_size(wk_dtype_size(real_dtype), [&]<typename E>() -> int {
        hipLaunchKernelGGL((complex_part_kernel<E, false>), row_grid(shape3[2], total_rows), dim3(256), 0, s->stream,
                           static_cast<const E *>(src), static_cast<E *>(dst), shape3[1], shape3[2], total_rows, srp, ssp, drp, dsp,
                           (unsigned)space);
        return launch_status();
    });
}

} // extern "C"
