// Complex float GEMM through the real matrix-core kernels, for callers that bring a workspace
// (blas.PackedTensors, the reference's pack pass: src/blas/gemm.zig:272-357, 705-720).
//
// With interleaved storage a complex M x K matrix IS a real M x 2K matrix, and
//     C = A B   <=>   C_real (M x 2N) = A_real (M x 2K) * B~ (2K x 2N),
//     B~[2k][2n] = re b,  B~[2k][2n+1] = im b,  B~[2k+1][2n] = -im b,  B~[2k+1][2n+1] = re b      (b = B[k][n])
// because  re c = sum a_re b_re - a_im b_im  and  im c = sum a_re b_im + a_im b_re.  So the pack pass
// only has to write B~ (alpha folded in: B~ is built from alpha * b), a transposed operand is first
// turned with the tensor transpose kernel, beta scales C in place beforehand (C_old is always read and
// multiplied, as the reference's epilogue does), and the product itself is the tuned f32 / f64 kernel
// on (M, 2N, 2K): 8 M N K real flop, the same count as four real products per complex one.
// Rounding differs from the reference's three-multiplication complex product
// (wekua_cl_lib.cl:648-653) only within the stated float tolerance.
#include "wk_internal.hpp"

#include <cstring>

using namespace wk;

namespace {

constexpr int CP_BLOCK = 256;

// one thread per complex element of B (K x N, row pitch ldb complex elements)
template <typename R>
__global__ __launch_bounds__(CP_BLOCK) void expand_b_kernel(const R *__restrict__ B, uint64_t ldb, uint64_t K, uint64_t N,
                                                            R *__restrict__ Bx, bool has_alpha, R ar, R ai) {
    const uint64_t total = K * N;
    for (uint64_t idx = blockIdx.x * (uint64_t)CP_BLOCK + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * CP_BLOCK) {
        const uint64_t k = idx / N, n = idx - k * N;
        R br = B[(k * ldb + n) * 2], bi = B[(k * ldb + n) * 2 + 1];
        if (has_alpha) {
            const R tr = ar * br - ai * bi, ti = ar * bi + ai * br;
            br = tr;
            bi = ti;
        }
        R *row0 = Bx + (2 * k) * (2 * N) + 2 * n, *row1 = row0 + 2 * N;
        row0[0] = br;
        row0[1] = bi;
        row1[0] = -bi;
        row1[1] = br;
    }
}

// C = beta * C over the logical M x N complex region
template <typename R>
__global__ __launch_bounds__(CP_BLOCK) void cscale_kernel(R *__restrict__ C, uint64_t ldc, uint64_t M, uint64_t N, R br, R bi) {
    const uint64_t total = M * N;
    for (uint64_t idx = blockIdx.x * (uint64_t)CP_BLOCK + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * CP_BLOCK) {
        const uint64_t m = idx / N, n = idx - m * N;
        R *p = C + (m * ldc + n) * 2;
        const R cr = p[0], ci = p[1];
        p[0] = br * cr - bi * ci;
        p[1] = br * ci + bi * cr;
    }
}

unsigned grid_for(uint64_t total) {
    const uint64_t want = (total + CP_BLOCK - 1) / CP_BLOCK;
    return (unsigned)(want < 65536 ? (want ? want : 1) : 65536);
}

size_t align16(size_t v) { return (v + 15) & ~size_t(15); }

template <typename R>
int prepare(hipStream_t st, const GemmProblem &p, const void *b_src, uint64_t ldb, void *bx) {
    R alpha[2] = {R(1), R(0)}, beta[2] = {R(0), R(0)};
    std::memcpy(alpha, p.alpha, sizeof alpha);
    std::memcpy(beta, p.beta, sizeof beta);
    const bool has_alpha = p.epi != EPI_STORE;
    int rc = WK_OK;
    if (!p.reuse_b) {
        hipLaunchKernelGGL(expand_b_kernel<R>, dim3(grid_for(p.K * p.N)), dim3(CP_BLOCK), 0, st, static_cast<const R *>(b_src), ldb,
                           p.K, p.N, static_cast<R *>(bx), has_alpha, alpha[0], alpha[1]);
        rc = launch_status();
    }
    if (rc || p.epi != EPI_ALPHA_BETA) return rc;
    hipLaunchKernelGGL(cscale_kernel<R>, dim3(grid_for(p.M * p.N)), dim3(CP_BLOCK), 0, st, static_cast<R *>(p.C), p.ldc, p.M, p.N,
                       beta[0], beta[1]);
    return launch_status();
}

} // namespace

size_t wk::gemm_complex_packed_workspace_bytes(int dtype, uint64_t M, uint64_t N, uint64_t K) {
    if ((dtype != WK_CF32 && dtype != WK_CF64) || !M || !N || !K) return 0;
    if (M > 0x3fffffffull || N > 0x3fffffffull || K > 0x3fffffffull) return 0; // the real problem doubles N and K
    const size_t es = dtype == WK_CF32 ? 8 : 16;
    return align16(M * K * es) + align16(K * N * es) + align16(2 * K * N * es);
}

// Fills `real` with the f32 / f64 problem whose result is the complex one, after enqueueing the passes
// that build its operands in the workspace.  `transpose` turns an R x C complex matrix (row pitch ld)
// into its C x R transpose with row pitch R.
int wk::gemm_complex_packed_prepare(hipStream_t st, const GemmProblem &p, void *workspace, size_t workspace_bytes,
                                    int (*transpose)(void *ctx, int dtype, uint64_t rows, uint64_t cols, const void *src, uint64_t ld,
                                                     void *dst),
                                    void *ctx, GemmProblem &real) {
    const size_t need = gemm_complex_packed_workspace_bytes(p.dtype, p.M, p.N, p.K);
    if (!need || !workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u)) return WK_E_INVALID_VALUE;
    const size_t es = p.dtype == WK_CF32 ? 8 : 16;
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    unsigned char *at = ws, *bt = at + align16(p.M * p.K * es), *bx = bt + align16(p.K * p.N * es);

    const void *a_real = p.A;
    uint64_t lda_real = 2 * p.lda;
    if (p.op_a) { // stored K x M
        const int rc = transpose(ctx, p.dtype, p.K, p.M, p.A, p.lda, at);
        if (rc) return rc;
        a_real = at;
        lda_real = 2 * p.K;
    }
    const void *b_src = p.B;
    uint64_t ldb = p.ldb;
    if (p.op_b && !p.reuse_b) { // stored N x K
        const int rc = transpose(ctx, p.dtype, p.N, p.K, p.B, p.ldb, bt);
        if (rc) return rc;
        b_src = bt;
        ldb = p.N;
    }
    const int rc = p.dtype == WK_CF32 ? prepare<float>(st, p, b_src, ldb, bx) : prepare<double>(st, p, b_src, ldb, bx);
    if (rc) return rc;

    real = GemmProblem{};
    real.dtype = p.dtype == WK_CF32 ? WK_F32 : WK_F64;
    real.op_a = real.op_b = 0;
    real.M = p.M; real.N = 2 * p.N; real.K = 2 * p.K;
    real.A = a_real; real.lda = lda_real;
    real.B = bx; real.ldb = 2 * p.N;
    real.C = p.C; real.ldc = 2 * p.ldc;
    real.num_cus = p.num_cus;
    std::memset(real.alpha, 0, sizeof real.alpha);
    std::memset(real.beta, 0, sizeof real.beta);
    if (p.epi == EPI_ALPHA_BETA) { // C was scaled by beta already, alpha is inside B~: C = 1 * acc + 1 * C
        real.epi = EPI_ALPHA_BETA;
        if (real.dtype == WK_F32) {
            const float one = 1.f;
            std::memcpy(real.alpha, &one, 4);
            std::memcpy(real.beta, &one, 4);
        } else {
            const double one = 1.;
            std::memcpy(real.alpha, &one, 8);
            std::memcpy(real.beta, &one, 8);
        }
    } else {
        real.epi = EPI_STORE;
    }
    return WK_OK;
}
