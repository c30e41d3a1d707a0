// Generic LDS-tiled VALU GEMM for every dtype, transpose pair and shape.
//
// This is the path for the integer and complex dtypes (no f32/f64 matrix instruction applies)
// and the fallback for float shapes the MFMA kernels do not take.  Integers are computed
// in unsigned arithmetic, so sums wrap modulo 2^w whatever the order of accumulation: the
// result is bit-identical to the reference's kernels (src/blas/kernels/gemm_nxn_gpu.cl,
// gemm_nxn.cl, gemm_2x2.cl) for any input, including overflowing ones.
//
// Work-group = 256 threads = one 64x64 tile of C; thread = 4x4 outputs; k step 16.
// Tiles of op(A) and op(B) are staged through LDS as [k][m] / [k][n] with the global reads
// running along whichever index is contiguous in memory for the given transpose flag.
#include "wk_internal.hpp"

#include <cstring>

using namespace wk;

namespace {

constexpr int GB_M = 64, GB_N = 64, GB_K = 16, G_THREADS = 256;

template <typename T> struct GArgs {
    const T *A, *B;
    T *C;
    uint64_t M, N, K, lda, ldb, ldc;
    int epi;
    typename elem_traits<T>::acc alpha, beta;
};

template <typename T, bool TA, bool TB>
__global__ __launch_bounds__(G_THREADS) void gemm_tile64_kernel(GArgs<T> g) {
    using A_t = typename elem_traits<T>::acc;
    constexpr int PAD = sizeof(A_t) >= 16 ? 1 : 4;
    __shared__ A_t As[GB_K][GB_M + PAD];
    __shared__ A_t Bs[GB_K][GB_N + PAD];

    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const uint64_t m0 = (uint64_t)blockIdx.y * GB_M, n0 = (uint64_t)blockIdx.x * GB_N;

    A_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = zero_of<A_t>();

    for (uint64_t k0 = 0; k0 < g.K; k0 += GB_K) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            int mm, kk;
            if (!TA) { kk = tid & 15; mm = (tid >> 4) + 16 * r; }   // A stored M x K: k is contiguous
            else     { mm = tid & 63; kk = (tid >> 6) + 4 * r; }    // A stored K x M: m is contiguous
            const uint64_t gm = m0 + mm, gk = k0 + kk;
            A_t v = zero_of<A_t>();
            if (gm < g.M && gk < g.K) v = widen<A_t>(g.A[TA ? gk * g.lda + gm : gm * g.lda + gk]);
            As[kk][mm] = v;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            int nn, kk;
            if (!TB) { nn = tid & 63; kk = (tid >> 6) + 4 * r; }    // B stored K x N: n is contiguous
            else     { kk = tid & 15; nn = (tid >> 4) + 16 * r; }   // B stored N x K: k is contiguous
            const uint64_t gn = n0 + nn, gk = k0 + kk;
            A_t v = zero_of<A_t>();
            if (gn < g.N && gk < g.K) v = widen<A_t>(g.B[TB ? gn * g.ldb + gk : gk * g.ldb + gn]);
            Bs[kk][nn] = v;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GB_K; ++kk) {
            A_t a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = mad(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint64_t gm = m0 + ty * 4 + i;
        if (gm >= g.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint64_t gn = n0 + tx * 4 + j;
            if (gn >= g.N) continue;
            T *p = g.C + gm * g.ldc + gn;
            A_t v = acc[i][j];
            if (g.epi == EPI_ALPHA) v = mul(v, g.alpha);
            else if (g.epi == EPI_ALPHA_BETA) v = add(mul(v, g.alpha), mul(widen<A_t>(*p), g.beta));
            *p = narrow<T>(v);
        }
    }
}

template <typename T> int launch_typed(hipStream_t st, const GemmProblem &p) {
    using A_t = typename elem_traits<T>::acc;
    GArgs<T> g;
    g.A = static_cast<const T *>(p.A);
    g.B = static_cast<const T *>(p.B);
    g.C = static_cast<T *>(p.C);
    g.M = p.M; g.N = p.N; g.K = p.K; g.lda = p.lda; g.ldb = p.ldb; g.ldc = p.ldc;
    g.epi = p.epi;
    T a, b;
    std::memcpy(&a, p.alpha, sizeof(T));
    std::memcpy(&b, p.beta, sizeof(T));
    g.alpha = widen<A_t>(a);
    g.beta = widen<A_t>(b);
    const uint64_t gx = (p.N + GB_N - 1) / GB_N, gy = (p.M + GB_M - 1) / GB_M;
    if (gx > 0x7fffffffull || gy > 65535ull) return WK_E_INVALID_VALUE;
    const dim3 grid((unsigned)gx, (unsigned)gy), block(G_THREADS);
    if (!p.op_a && !p.op_b) hipLaunchKernelGGL((gemm_tile64_kernel<T, false, false>), grid, block, 0, st, g);
    else if (!p.op_a && p.op_b) hipLaunchKernelGGL((gemm_tile64_kernel<T, false, true>), grid, block, 0, st, g);
    else if (p.op_a && !p.op_b) hipLaunchKernelGGL((gemm_tile64_kernel<T, true, false>), grid, block, 0, st, g);
    else hipLaunchKernelGGL((gemm_tile64_kernel<T, true, true>), grid, block, 0, st, g);
    return launch_status();
}

} // namespace

int wk::gemm_generic_launch(hipStream_t st, const GemmProblem &p) {
    return dispatch_dtype(p.dtype, [&]<typename T>() -> int { return launch_typed<T>(st, p); });
}
