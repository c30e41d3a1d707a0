// f32 / f64 products with at most four rows or at most four columns of C: matrix-vector products in all
// but name (wekua has no gemv; blas.gemm with M = 1 or N = 1 is how its users spell one, and wk_gemm's own
// strips beyond whole tiles are such products too).  A tile kernel pads them to 64 rows and reads the long
// operand in 256-byte pieces; here the long operand is read once, along its storage order, and the thin
// one sits in LDS.
//
//   out(i, j) = sum_k X(i, k) * Y(k, j),   i < L (the long index), j < R <= 4
//
// Rows thin (M <= 4): i = column of C, X = op(B), Y(k, j) = op(A)(j, k).  Columns thin (N <= 4): i = row of C,
// X = op(A), Y = op(B).  Two kernels by the storage of X:
//   X(i, k) = X[i * ldx + k] (k-contiguous): one wavefront per i; lanes walk k (16 bytes each where the rows
//     allow it), the wavefront's partial sums meet in a butterfly, lane 0 runs the epilogue.  One launch.
//   X(i, k) = X[k * ldx + i] (i-contiguous): one thread per i and k split over blockIdx.y, so that a few
//     thousand work-groups are in flight whatever L is; the shares' partial sums go to the stream's scratch
//     and a second launch adds them in the order of the shares (the same bits on every run) and runs the
//     epilogue.
// The products are fused multiply-adds in k order per lane, so the rounding differs from the matrix
// instructions' (as theirs differs between tile shapes); option semantics as everywhere:
// src/blas/gemm.zig:500-501,591-602.
#include "wk_internal.hpp"

#include <cstring>
#include <type_traits>

using namespace wk;

namespace {

constexpr int CHUNK = 1024; // k values of Y in LDS at a time (R * CHUNK elements: at most 32 KiB)

template <typename T> struct ThinArgs {
    const T *X;
    uint64_t ldx;
    const T *Y;
    uint64_t sy_k, sy_j; // Y(k, j) = Y[k * sy_k + j * sy_j]
    T *C;
    uint64_t sc_i, sc_j; // C(i, j) = C[i * sc_i + j * sc_j]
    uint32_t L, K;
    int epi;
    T alpha, beta;
    T *partial;          // [share][j][i], i-contiguous kernel only
    uint32_t klen;       // k values per share
};

template <typename T> __device__ __forceinline__ T finish(const ThinArgs<T> &g, T v, uint64_t at) {
    if (g.epi == EPI_ALPHA) return g.alpha * v;
    if (g.epi == EPI_ALPHA_BETA) return g.alpha * v + g.beta * g.C[at];
    return v;
}

// Y's k values [k0, k0 + n) into LDS, zero beyond K
template <typename T, int R> __device__ __forceinline__ void stage_y(const ThinArgs<T> &g, T (*ys)[CHUNK], uint32_t k0, uint32_t n) {
    for (uint32_t idx = threadIdx.x; idx < R * n; idx += blockDim.x) {
        const uint32_t j = idx / n, kk = idx - j * n;
        ys[j][kk] = k0 + kk < g.K ? g.Y[(uint64_t)(k0 + kk) * g.sy_k + (uint64_t)j * g.sy_j] : T(0);
    }
}

template <typename T, int R, bool VEC>
__global__ __launch_bounds__(256) void thin_kc_kernel(ThinArgs<T> g) {
    constexpr int VE = VEC ? 16 / sizeof(T) : 1;
    __shared__ __align__(16) T ys[R][CHUNK];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t i = blockIdx.x * 4u + wave;
    const bool live = i < g.L;
    const T *xrow = g.X + (uint64_t)(live ? i : 0) * g.ldx;
    T acc[R];
#pragma unroll
    for (int j = 0; j < R; ++j) acc[j] = T(0);
    // Every work-group walks the chunks of k from a place of its own and wraps around: walking in step, the rows of
    // a long operand whose leading dimension is a multiple of the memory channels' period (8192 doubles) would
    // have their pieces in the same channels at the same time (f64 1 x 8192 x 8192 N,T: 121 us in step).
    const uint32_t chunks = (g.K + CHUNK - 1) / CHUNK, first = blockIdx.x % chunks;
    for (uint32_t c = 0; c < chunks; ++c) {
        const uint32_t k0 = (c + first < chunks ? c + first : c + first - chunks) * CHUNK;
        const uint32_t n = min((uint32_t)CHUNK, g.K - k0);
        __syncthreads();
        stage_y<T, R>(g, ys, k0, VEC ? (n + VE - 1) / VE * VE : n); // (whole vectors: zeros beyond K)
        __syncthreads();
        if (!live) continue;
        for (uint32_t kk = lane * VE; kk < n; kk += 64 * VE) {
            T x[VE];
            if (VEC && kk + VE <= n) {
                __builtin_memcpy(x, xrow + k0 + kk, sizeof x);
            } else {
#pragma unroll
                for (int e = 0; e < VE; ++e) x[e] = kk + e < n ? xrow[k0 + kk + e] : T(0);
            }
#pragma unroll
            for (int j = 0; j < R; ++j)
#pragma unroll
                for (int e = 0; e < VE; ++e) acc[j] = __builtin_fma(x[e], ys[j][kk + e], acc[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) acc[j] += __shfl_xor(acc[j], off, 64);
    if (live && lane == 0)
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint64_t at = (uint64_t)i * g.sc_i + (uint64_t)j * g.sc_j;
            g.C[at] = finish(g, acc[j], at);
        }
}

template <typename T, int R>
__global__ __launch_bounds__(256) void thin_ic_kernel(ThinArgs<T> g) {
    __shared__ T ys[R][CHUNK];
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    const uint32_t k0 = blockIdx.y * g.klen, n = min(g.klen, g.K - k0);
    stage_y<T, R>(g, ys, k0, n);
    __syncthreads();
    if (i >= g.L) return;
    const T *x = g.X + (uint64_t)k0 * g.ldx + i;
    T acc[R];
#pragma unroll
    for (int j = 0; j < R; ++j) acc[j] = T(0);
#pragma unroll 8
    for (uint32_t kk = 0; kk < n; ++kk) {
        const T xv = x[(uint64_t)kk * g.ldx];
#pragma unroll
        for (int j = 0; j < R; ++j) acc[j] = __builtin_fma(xv, ys[j][kk], acc[j]);
    }
#pragma unroll
    for (int j = 0; j < R; ++j) g.partial[((uint64_t)blockIdx.y * R + j) * g.L + i] = acc[j];
}

// The shares' partial sums, in a fixed order: 64 values of i per work-group; thread row q adds the shares
// q, q + 4, q + 8, ..., row 0 then adds the four rows' sums in order and runs the epilogue.
template <typename T, int R>
__global__ __launch_bounds__(256) void thin_sum_kernel(ThinArgs<T> g, uint32_t shares) {
    __shared__ T rows[4][R][64];
    const uint32_t ii = threadIdx.x & 63u, q = threadIdx.x >> 6;
    const uint32_t i = blockIdx.x * 64u + ii;
    T v[R];
#pragma unroll
    for (int j = 0; j < R; ++j) v[j] = T(0);
    if (i < g.L) {
#pragma unroll 4
        for (uint32_t s = q; s < shares; s += 4)
#pragma unroll
            for (int j = 0; j < R; ++j) v[j] += g.partial[((uint64_t)s * R + j) * g.L + i];
    }
#pragma unroll
    for (int j = 0; j < R; ++j) rows[q][j][ii] = v[j];
    __syncthreads();
    if (q != 0 || i >= g.L) return;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const T sum = ((rows[0][j][ii] + rows[1][j][ii]) + rows[2][j][ii]) + rows[3][j][ii];
        const uint64_t at = (uint64_t)i * g.sc_i + (uint64_t)j * g.sc_j;
        g.C[at] = finish(g, sum, at);
    }
}

// shares of the i-contiguous kernel: enough work-groups to fill the chip several times over, at least 64 k
// each, at most CHUNK
void plan_shares(uint64_t L, uint64_t K, uint32_t &shares, uint32_t &klen) {
    const uint64_t blocks_x = (L + 255) / 256;
    uint64_t want = (2048 + blocks_x - 1) / blocks_x;
    uint64_t len = (K + want - 1) / want;
    len = len < 64 ? 64 : len > (uint64_t)CHUNK ? (uint64_t)CHUNK : len;
    klen = (uint32_t)len;
    shares = (uint32_t)((K + len - 1) / len);
}

template <typename T, int R> int launch_r(hipStream_t st, const GemmProblem &p, ThinArgs<T> g, bool x_kc) {
    if (x_kc) {
        const bool vec = g.ldx % (16 / sizeof(T)) == 0 && (reinterpret_cast<uintptr_t>(g.X) & 15u) == 0;
        const dim3 grid((g.L + 3) / 4);
        if (vec) hipLaunchKernelGGL((thin_kc_kernel<T, R, true>), grid, dim3(256), 0, st, g);
        else hipLaunchKernelGGL((thin_kc_kernel<T, R, false>), grid, dim3(256), 0, st, g);
        return launch_status();
    }
    const uint32_t blocks_x = (g.L + 255) / 256;
    uint32_t shares, klen;
    plan_shares(g.L, g.K, shares, klen);
    if ((size_t)shares * R * g.L * sizeof(T) > p.scratch_bytes || !p.scratch || shares > 65535) return WK_E_SCRATCH_TOO_SMALL;
    g.klen = klen;
    g.partial = static_cast<T *>(p.scratch);
    hipLaunchKernelGGL((thin_ic_kernel<T, R>), dim3(blocks_x, shares), dim3(256), 0, st, g);
    int rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL((thin_sum_kernel<T, R>), dim3((g.L + 63) / 64), dim3(256), 0, st, g, shares);
    return launch_status();
}

template <typename T> int launch_t(hipStream_t st, const GemmProblem &p) {
    ThinArgs<T> g{};
    const T *A = static_cast<const T *>(p.A), *B = static_cast<const T *>(p.B);
    bool x_kc;
    uint32_t R;
    if (p.M <= 4) { // rows thin: the long index runs over the columns of C
        R = (uint32_t)p.M;
        g.L = (uint32_t)p.N;
        g.X = B; g.ldx = p.ldb; x_kc = p.op_b != 0;             // op(B)(k, n): B[n * ldb + k] for op T
        g.Y = A; g.sy_k = p.op_a ? p.lda : 1; g.sy_j = p.op_a ? 1 : p.lda; // op(A)(j, k)
        g.sc_i = 1; g.sc_j = p.ldc;
    } else {
        R = (uint32_t)p.N;
        g.L = (uint32_t)p.M;
        g.X = A; g.ldx = p.lda; x_kc = p.op_a == 0;             // op(A)(m, k): A[m * lda + k] for op N
        g.Y = B; g.sy_k = p.op_b ? 1 : p.ldb; g.sy_j = p.op_b ? p.ldb : 1; // op(B)(k, j)
        g.sc_i = p.ldc; g.sc_j = 1;
    }
    g.C = static_cast<T *>(p.C);
    g.K = (uint32_t)p.K;
    g.epi = p.epi;
    std::memcpy(&g.alpha, p.alpha, sizeof(T));
    std::memcpy(&g.beta, p.beta, sizeof(T));
    switch (R) {
    case 1: return launch_r<T, 1>(st, p, g, x_kc);
    case 2: return launch_r<T, 2>(st, p, g, x_kc);
    case 3: return launch_r<T, 3>(st, p, g, x_kc);
    default: return launch_r<T, 4>(st, p, g, x_kc);
    }
}

} // namespace

// At most four rows or four columns of C, the other dimension long enough to fill the chip with
// wavefronts, k long enough to be worth a launch of its own kind; the i-contiguous kernel needs the
// stream's scratch for its shares.
bool wk::gemm_thin_applies(const GemmProblem &p) {
    if ((p.dtype != WK_F32 && p.dtype != WK_F64) || p.ext) return false;
    const bool rows_thin = p.M <= 4, cols_thin = p.N <= 4;
    if (rows_thin == cols_thin) return false; // neither, or both: a handful of entries
    const uint64_t L = rows_thin ? p.N : p.M;
    if (L < 512 || L > 0x7fffffffull || p.K < 128 || p.K > 0x7fffffffull) return false;
    const bool x_kc = rows_thin ? p.op_b != 0 : p.op_a == 0;
    if (!x_kc) {
        uint32_t shares, klen;
        plan_shares(L, p.K, shares, klen);
        const uint64_t R = rows_thin ? p.M : p.N;
        if (!p.scratch || shares > 65535 || (size_t)shares * R * L * wk_dtype_size(p.dtype) > p.scratch_bytes) return false;
    }
    return true;
}

int wk::gemm_thin_launch(hipStream_t st, const GemmProblem &p) {
    if (!gemm_thin_applies(p)) return WK_E_INVALID_VALUE;
    return p.dtype == WK_F32 ? launch_t<float>(st, p) : launch_t<double>(st, p);
}
