// Complex GEMM (float and integer components) through the real matrix-core kernels, for callers that bring a workspace
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
// For the complex integer types everything is arithmetic modulo 2^width, where the identity is exact:
// the passes compute in unsigned 32-bit (64-bit components: 64-bit) and truncate (signed and unsigned share the bits), and the real
// product is the packed int8 matrix-core path on (M, 2N, 2K) in the section of the workspace behind B~.
#include "wk_internal.hpp"

#include <cstring>
#include <type_traits>

using namespace wk;

namespace {

constexpr int CP_BLOCK = 256;

// the type the passes compute in: wraparound arithmetic for the integers without promotion to signed int
template <typename R>
using Wide = std::conditional_t<std::is_integral_v<R>, std::conditional_t<sizeof(R) == 8, uint64_t, uint32_t>, R>;

// one thread per complex element of B (K x N, row pitch ldb complex elements)
template <typename R>
__global__ __launch_bounds__(CP_BLOCK) void expand_b_kernel(const R *__restrict__ B, uint64_t ldb, uint64_t K, uint64_t N,
                                                            R *__restrict__ Bx, bool has_alpha, R alpha_r, R alpha_i) {
    using W = Wide<R>;
    const W ar = alpha_r, ai = alpha_i;
    const uint64_t total = K * N;
    for (uint64_t idx = blockIdx.x * (uint64_t)CP_BLOCK + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * CP_BLOCK) {
        const uint64_t k = idx / N, n = idx - k * N;
        W br = B[(k * ldb + n) * 2], bi = B[(k * ldb + n) * 2 + 1];
        if (has_alpha) {
            const W tr = ar * br - ai * bi, ti = ar * bi + ai * br;
            br = tr;
            bi = ti;
        }
        R *row0 = Bx + (2 * k) * (2 * N) + 2 * n, *row1 = row0 + 2 * N;
        row0[0] = (R)br;
        row0[1] = (R)bi;
        row1[0] = (R)(W(0) - bi);
        row1[1] = (R)br;
    }
}

// C = beta * C over the logical M x N complex region
template <typename R>
__global__ __launch_bounds__(CP_BLOCK) void cscale_kernel(R *__restrict__ C, uint64_t ldc, uint64_t M, uint64_t N, R beta_r, R beta_i) {
    using W = Wide<R>;
    const W br = beta_r, bi = beta_i;
    const uint64_t total = M * N;
    for (uint64_t idx = blockIdx.x * (uint64_t)CP_BLOCK + threadIdx.x; idx < total; idx += (uint64_t)gridDim.x * CP_BLOCK) {
        const uint64_t m = idx / N, n = idx - m * N;
        R *p = C + (m * ldc + n) * 2;
        const W cr = p[0], ci = p[1];
        p[0] = (R)(br * cr - bi * ci);
        p[1] = (R)(br * ci + bi * cr);
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

// component type of a complex dtype this file handles, or -1
int real_of(int dtype) {
    if (dtype == WK_CF32) return WK_F32;
    if (dtype == WK_CF64) return WK_F64;
    if (dtype >= WK_COMPLEX + WK_I8 && dtype <= WK_COMPLEX + WK_U64) return dtype - WK_COMPLEX;
    return -1;
}

// bytes of the section holding the turned operands and B~
size_t section_bytes(int dtype, uint64_t M, uint64_t N, uint64_t K) {
    const size_t es = wk_dtype_size(dtype);
    return align16(M * K * es) + align16(K * N * es) + align16(2 * K * N * es);
}

} // namespace

size_t wk::gemm_complex_packed_workspace_bytes(int dtype, uint64_t M, uint64_t N, uint64_t K) {
    const int rd = real_of(dtype);
    if (rd < 0 || !M || !N || !K) return 0;
    if (M > 0x3fffffffull || N > 0x3fffffffull || K > 0x3fffffffull) return 0; // the real problem doubles N and K
    const size_t section = section_bytes(dtype, M, N, K);
    if (rd == WK_F32 || rd == WK_F64) return section;
    const size_t product = gemm_int_packed_workspace_bytes(rd, M, 2 * N, 2 * K); // digit planes of the real operands
    return product ? section + product : 0;
}

// Fills `real` with the real problem whose result is the complex one, after enqueueing the passes
// that build its operands in the workspace.  `transpose` turns an R x C complex matrix (row pitch ld)
// into its C x R transpose with row pitch R.  `rest` / `rest_bytes`: what lies behind the section
// used here (the workspace of the real integer product; empty for the float types).
int wk::gemm_complex_packed_prepare(hipStream_t st, const GemmProblem &p, void *workspace, size_t workspace_bytes,
                                    int (*transpose)(void *ctx, int dtype, uint64_t rows, uint64_t cols, const void *src, uint64_t ld,
                                                     void *dst),
                                    void *ctx, GemmProblem &real, void **rest, size_t *rest_bytes) {
    const size_t need = gemm_complex_packed_workspace_bytes(p.dtype, p.M, p.N, p.K);
    if (!need || !workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u)) return WK_E_INVALID_VALUE;
    const int rd = real_of(p.dtype);
    const size_t es = wk_dtype_size(p.dtype);
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    unsigned char *at = ws, *bt = at + align16(p.M * p.K * es), *bx = bt + align16(p.K * p.N * es);
    const size_t section = section_bytes(p.dtype, p.M, p.N, p.K);
    *rest = ws + section;
    *rest_bytes = workspace_bytes - section;

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
    int rc;
    switch (es) {
    case 2: rc = prepare<uint8_t>(st, p, b_src, ldb, bx); break;
    case 4: rc = prepare<uint16_t>(st, p, b_src, ldb, bx); break;
    case 8: rc = rd == WK_F32 ? prepare<float>(st, p, b_src, ldb, bx) : prepare<uint32_t>(st, p, b_src, ldb, bx); break;
    default: rc = rd == WK_F64 ? prepare<double>(st, p, b_src, ldb, bx) : prepare<uint64_t>(st, p, b_src, ldb, bx); break;
    }
    if (rc) return rc;

    real = GemmProblem{};
    real.dtype = rd;
    real.op_a = real.op_b = 0;
    real.M = p.M; real.N = 2 * p.N; real.K = 2 * p.K;
    real.A = a_real; real.lda = lda_real;
    real.B = bx; real.ldb = 2 * p.N;
    real.C = p.C; real.ldc = 2 * p.ldc;
    real.num_cus = p.num_cus;
    real.reuse_b = p.reuse_b;
    // the stream's scratch and tile counters, for the real kernels that split k over work-groups or deal k-slabs
    real.scratch = p.scratch; real.scratch_bytes = p.scratch_bytes;
    real.counters = p.counters; real.num_counters = p.num_counters;
    std::memset(real.alpha, 0, sizeof real.alpha);
    std::memset(real.beta, 0, sizeof real.beta);
    if (p.epi == EPI_ALPHA_BETA) { // C was scaled by beta already, alpha is inside B~: C = 1 * acc + 1 * C
        real.epi = EPI_ALPHA_BETA;
        if (rd == WK_F32) {
            const float one = 1.f;
            std::memcpy(real.alpha, &one, 4);
            std::memcpy(real.beta, &one, 4);
        } else if (rd == WK_F64) {
            const double one = 1.;
            std::memcpy(real.alpha, &one, 8);
            std::memcpy(real.beta, &one, 8);
        } else {
            real.alpha[0] = real.beta[0] = 1; // little-endian integer one of any width
        }
    } else {
        real.epi = EPI_STORE;
    }
    return WK_OK;
}
