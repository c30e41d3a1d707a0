// 64-bit integer GEMM on the int8 matrix cores, with a pack pass (the caller brings a workspace, as
// blas.PackedTensors does: src/blas/gemm.zig:272-357, 705-720).
//
// The result is only needed modulo 2^64.  Write every element in balanced digits, a = sum_i 256^i s_i
// (mod 2^64) with s_i in [-128, 127]: with c = 0x80 in every byte and t = a + c (carries and all), the
// bytes t_i of t give a = t - c = sum_i 256^i (t_i - 128), and t_i - 128 as a signed byte is t_i ^ 0x80.
// Then sum_k a b = sum_{i + j <= 7} 256^(i + j) S_ij with S_ij = sum_k s_i(a) s_j(b): 36 digit products,
// int8 x int8 accumulated in int32 by v_mfma_i32_32x32x32_i8, one accumulator per shift i + j.
// Accumulators of shift 4 and more may wrap: 256^(i+j) 2^32 vanishes modulo 2^64.  Those of shifts 0..3
// must hold their sums exactly: at most four pairs of at most 2^14 each per k, so a launch takes at most
// K_CHUNK = 2^14 values of k (4 x 2^14 x 2^14 = 2^30) and a longer product is a chain of launches through C
// (C = alpha A1 B1 + beta C, then C = alpha A2 B2 + 1 C, ...), which modulo 2^64 is the same bits.
//
//   pass 1  ipack64_kernel   reads op(A) and op(B) once, whatever their layout, and writes their digit
//                            planes in the order the matrix instruction eats them: 1 KiB blocks, one per
//                            (32 rows, 32 k, digit), lane l of a wavefront owning bytes 16 l .. 16 l + 15 =
//                            row l % 32, k 16 (l / 32) .. + 15.  Rows and k beyond the matrix are zero digits.
//   pass 2  gemm_i64_packed_kernel   128 x 64 tile, eight wavefronts of 32 x 32 (two per SIMD: eight
//                            accumulators of 16 registers each and sixteen fragments), a stage = one
//                            k-block of 32 with its eight digit blocks per 32 rows (48 KiB), three stages,
//                            brought straight from the planes into LDS (the blocks are already in the
//                            order a direct global -> LDS load lays a wavefront's 64 x 16 bytes down).
//
// Workspace: 8 bytes per element of the padded operands (256 bytes per (row, 32 k)), for at most K_CHUNK of k.
#include "wk_internal.hpp"
#include "wk_lds_dma.hpp"

#include <cstring>

using namespace wk;
using namespace wk::lds_dma;

namespace {

typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int BK = 32, BLOCK_BYTES = 1024, D = 8, GROUP_BYTES = D * BLOCK_BYTES; // one k-block of 32 rows: eight digit blocks
constexpr int BM = 128, BN = 64, A_GROUPS = BM / 32, B_GROUPS = BN / 32, GROUPS = A_GROUPS + B_GROUPS;
constexpr int STAGE_BYTES = GROUPS * GROUP_BYTES, NS = 3, WAVES = 8, LOADS = GROUPS * D / WAVES; // 1 KiB loads per wavefront and stage
constexpr uint64_t K_CHUNK = 16384;
constexpr int PACK_THREADS = 256;
constexpr uint32_t MAX_KSPLIT = 16;
static_assert(GROUPS * D % WAVES == 0, "the loads of a stage divide over the wavefronts");

struct Layout {
    uint64_t Mp, Np, KB, ksplit; // KB: k-blocks of 32 of one chunk; ksplit: k-ranges of the pack launch
    size_t planes_a, planes_b, total;
};

Layout make_layout(uint64_t M, uint64_t N, uint64_t K) {
    Layout w;
    w.Mp = (M + BM - 1) / BM * BM;
    w.Np = (N + BN - 1) / BN * BN;
    const uint64_t kc = K < K_CHUNK ? K : K_CHUNK;
    w.KB = (kc + BK - 1) / BK;
    uint64_t ks = 2048 / ((w.Mp + w.Np) / 32);
    ks = ks < 1 ? 1 : ks > MAX_KSPLIT ? MAX_KSPLIT : ks;
    if (ks > w.KB) ks = w.KB;
    w.ksplit = ks;
    w.planes_a = 0;
    w.planes_b = (size_t)w.Mp / 32 * w.KB * GROUP_BYTES;
    w.total = w.planes_b + (size_t)w.Np / 32 * w.KB * GROUP_BYTES;
    return w;
}

// 4 x 4 byte transpose: w[t] = a 32-bit word of the element at k + t -> p[d] = byte d of k + 0 .. k + 3
__device__ __forceinline__ void transpose_bytes(const uint32_t w[4], uint32_t p[4]) {
    const uint32_t ab_lo = __builtin_amdgcn_perm(w[1], w[0], 0x05010400u), ab_hi = __builtin_amdgcn_perm(w[1], w[0], 0x07030602u);
    const uint32_t cd_lo = __builtin_amdgcn_perm(w[3], w[2], 0x05010400u), cd_hi = __builtin_amdgcn_perm(w[3], w[2], 0x07030602u);
    p[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
    p[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
    p[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
    p[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
}

struct PackOperand {
    const uint64_t *src;   // element (r, k) at src[r * ld + k] (k-contiguous) or src[k * ld + r]
    uint32_t ld, rows, row_blocks; // true rows; padded rows / 32
    unsigned char *planes;
    uint32_t k_contiguous, vector_ok; // vector_ok: 16-byte loads along k are aligned
};
struct PackArgs {
    PackOperand op[2];
    uint32_t K, KB, kb_per_split; // K: the k values of this chunk
};

// blockIdx.x: row block of A, then of B; blockIdx.y: k-range.  Wave w of the work-group takes the
// k-blocks start + w, start + w + 4, ...; lane l the row l % 32 and the 16 k of half l / 32.
__global__ __launch_bounds__(PACK_THREADS) void ipack64_kernel(PackArgs g) {
    const int which = blockIdx.x >= g.op[0].row_blocks;
    const PackOperand &o = g.op[which];
    const uint64_t *__restrict__ src = o.src;
    unsigned char *__restrict__ planes = o.planes;
    const uint32_t rb = blockIdx.x - (which ? g.op[0].row_blocks : 0u);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
    const uint32_t row = rb * 32 + l32;
    const bool row_ok = row < o.rows;
    const uint32_t kb_begin = blockIdx.y * g.kb_per_split, kb_end = min(g.KB, kb_begin + g.kb_per_split);
    constexpr uint64_t CBIAS = 0x8080808080808080ull;
    for (uint32_t kb = kb_begin + wave; kb < kb_end; kb += PACK_THREADS / 64) {
        const uint32_t k0 = kb * BK + 16 * half;
        uint64_t e[16];
        if (o.k_contiguous) {
            const uint64_t *p = src + (size_t)row * o.ld + k0;
            if (row_ok && o.vector_ok && k0 + 16 <= g.K) {
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(p + 2 * q);
                    e[2 * q] = (uint64_t)v[0] | ((uint64_t)v[1] << 32);
                    e[2 * q + 1] = (uint64_t)v[2] | ((uint64_t)v[3] << 32);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 16; ++j) e[j] = row_ok && k0 + j < g.K ? p[j] : 0ull;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) e[j] = row_ok && k0 + j < g.K ? src[(size_t)(k0 + j) * o.ld + row] : 0ull;
        }
        u32x4 out[D];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t lo[4], hi[4], pl[4], ph[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint64_t x = (e[4 * q + t] + CBIAS) ^ CBIAS;
                lo[t] = (uint32_t)x;
                hi[t] = (uint32_t)(x >> 32);
            }
            transpose_bytes(lo, pl);
            transpose_bytes(hi, ph);
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                out[d][q] = pl[d];
                out[4 + d][q] = ph[d];
            }
        }
        // block (rb, kb, d) is the (kb * D + d)-th of its row block
        unsigned char *dst = planes + ((size_t)rb * g.KB + kb) * GROUP_BYTES + lane * 16;
#pragma unroll
        for (int d = 0; d < D; ++d) *reinterpret_cast<u32x4 *>(dst + d * BLOCK_BYTES) = out[d];
    }
}

struct PArgs {
    const unsigned char *planes_a, *planes_b;
    uint64_t *C;
    uint32_t M, N, KB, ldc, tiles_m, tiles_n;
    int epi;
    uint64_t alpha, beta;
    uint32_t patch_m, patch_n; // tile walk in XCD-local patches (0: groups of tile rows)
};

template <bool EDGE>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_i64_packed_kernel(PArgs g) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
    uint32_t tile_m, tile_n;
    if (g.patch_m) { // work-group b runs on XCD b % 8: the tiles an XCD holds at one time share rows of A and columns of B
        const uint32_t pid = blockIdx.x, x = pid & 7u, j = pid >> 3;
        const uint32_t per_patch = g.patch_m * g.patch_n, patch = (j / per_patch) * 8u + x, q = j % per_patch;
        const uint32_t patches_n = g.tiles_n / g.patch_n;
        tile_m = (patch / patches_n) * g.patch_m + q % g.patch_m;
        tile_n = (patch % patches_n) * g.patch_n + q / g.patch_m;
    } else {
        const uint32_t pid = blockIdx.x, group_size = 8 * g.tiles_n, group = pid / group_size, first_m = group * 8;
        const uint32_t gsz = min(g.tiles_m - first_m, 8u), in_group = pid - group * group_size;
        tile_m = first_m + in_group % gsz;
        tile_n = in_group / gsz;
    }
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    // load i of this wavefront brings block wave * LOADS + i of the stage's 48: group b / 8 (A's four row
    // groups, then B's two column groups), digit b % 8
    const unsigned char *src[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int b = wave * LOADS + i, gi = b / D, dig = b % D;
        const unsigned char *planes = gi < A_GROUPS ? g.planes_a + (size_t)(tile_m * A_GROUPS + gi) * g.KB * GROUP_BYTES
                                                   : g.planes_b + (size_t)(tile_n * B_GROUPS + gi - A_GROUPS) * g.KB * GROUP_BYTES;
        src[i] = planes + dig * BLOCK_BYTES;
    }
    const uint32_t voff = lane * 16;
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds_raw);
    auto issue = [&](uint32_t stage_bytes) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            dma16(src[i], voff, lds0 + stage_bytes + (uint32_t)(wave * LOADS + i) * BLOCK_BYTES);
            src[i] += GROUP_BYTES;
        }
    };

    i32x16 acc[D]; // one per shift i + j
#pragma unroll
    for (int s = 0; s < D; ++s)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[s][r] = 0;

    const uint32_t ktiles = g.KB;
    uint32_t st[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) st[n] = n * STAGE_BYTES;
#pragma unroll
    for (int n = 0; n < NS - 1; ++n)
        if ((uint32_t)n < ktiles) issue(st[n]);
    wait_vm_slabs<LOADS, NS - 2>(ktiles - 1);
    __builtin_amdgcn_s_barrier();

    for (uint32_t kt = 0; kt < ktiles; ++kt) {
        // stage kt + 2 goes where stage kt - 1 was: every wavefront is past the barrier that ended iteration
        // kt - 1, in front of which its matrix instructions had consumed that stage's fragments
        if (kt + NS - 1 < ktiles) issue(st[NS - 1]);
        const unsigned char *sa = lds_raw + st[0] + wm * GROUP_BYTES + lane * 16;
        const unsigned char *sb = lds_raw + st[0] + (A_GROUPS + wn) * GROUP_BYTES + lane * 16;
        i32x4 a[D], b[D];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            a[d] = *reinterpret_cast<const i32x4 *>(sa + d * BLOCK_BYTES);
            b[d] = *reinterpret_cast<const i32x4 *>(sb + d * BLOCK_BYTES);
        }
        // by shift, so that the first instructions need the fewest fragments and two instructions on one
        // accumulator are a whole shift apart
#pragma unroll
        for (int i = 0; i < D; ++i)
#pragma unroll
            for (int s = i; s < D; ++s) acc[s] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[s - i], acc[s], 0, 0, 0);
        if (kt + 1 < ktiles) {
            if (kt + NS - 1 < ktiles) wait_vm<LOADS>(); // this wavefront's loads of stage kt + 1 (those of kt + 2 may stay in flight)
            else wait_vm<0>();
            __builtin_amdgcn_s_barrier();
        }
        const uint32_t t = st[0];
#pragma unroll
        for (int n = 0; n + 1 < NS; ++n) st[n] = st[n + 1];
        st[NS - 1] = t;
    }

    // epilogue: register r of lane l is C[8 (r / 4) + 4 (l / 32) + r % 4][l % 32] of the wavefront's 32 x 32
    // block.  Shifts 0..3 hold exact sums (sign-extended), the others count modulo 2^32, which is all that is
    // left of them after the shift; everything modulo 2^64.  Option semantics of src/blas/gemm.zig:500-501,591-602.
    const uint32_t col = n0 + wn * 32 + l32, colc = EDGE ? min(col, g.N - 1) : col;
    uint64_t old[16];
    if (g.epi == EPI_ALPHA_BETA) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = m0 + wm * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
            old[r] = g.C[(size_t)(EDGE ? min(row, g.M - 1) : row) * g.ldc + colc];
        }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const uint32_t row = m0 + wm * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
        uint64_t v = 0;
#pragma unroll
        for (int s = 0; s < D; ++s) v += (uint64_t)(int64_t)acc[s][r] << (8 * s);
        if (g.epi == EPI_ALPHA) v = g.alpha * v;
        else if (g.epi == EPI_ALPHA_BETA) v = g.alpha * v + g.beta * old[r];
        if (!EDGE || ((row < g.M) & (col < g.N))) g.C[(size_t)row * g.ldc + col] = v;
    }
}

template <bool EDGE> int launch_product(hipStream_t st, PArgs g) {
    constexpr size_t lds = (size_t)NS * STAGE_BYTES;
    auto kern = gemm_i64_packed_kernel<EDGE>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) { (void)hipGetLastError(); return hip_code(attr); }
    g.patch_m = g.patch_n = 0;
    static const unsigned shapes[][2] = {{4, 8}, {2, 8}, {4, 4}, {2, 4}};
    for (const auto &sh : shapes)
        if (g.tiles_m % sh[0] == 0 && g.tiles_n % sh[1] == 0 && ((g.tiles_m / sh[0]) * (g.tiles_n / sh[1])) % 8 == 0) {
            g.patch_m = sh[0];
            g.patch_n = sh[1];
            break;
        }
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(64 * WAVES), lds, st, g);
    return launch_status();
}

} // namespace

// 0: this problem cannot take the path (dimensions of 31 bits; a row block's planes within 4 GiB offsets)
size_t wk::gemm_i64_packed_workspace_bytes(uint64_t M, uint64_t N, uint64_t K) {
    if (!M || !N || !K || M > 0x7fffffffull - BM || N > 0x7fffffffull - BN || K > 0x7fffffffull) return 0;
    return make_layout(M, N, K).total;
}

int wk::gemm_i64_packed_launch(hipStream_t st, const GemmProblem &p, void *workspace, size_t workspace_bytes) {
    const size_t need = gemm_i64_packed_workspace_bytes(p.M, p.N, p.K);
    if (!need || !workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u)) return WK_E_INVALID_VALUE;
    if (p.lda > 0x7fffffffull || p.ldb > 0x7fffffffull || p.ldc > 0x7fffffffull) return WK_E_INVALID_VALUE;
    const Layout w = make_layout(p.M, p.N, p.K);
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    const uint64_t *A = static_cast<const uint64_t *>(p.A), *B = static_cast<const uint64_t *>(p.B);
    uint64_t alpha = 1, beta = 1;
    if (p.epi != EPI_STORE) std::memcpy(&alpha, p.alpha, 8);
    if (p.epi == EPI_ALPHA_BETA) std::memcpy(&beta, p.beta, 8);
    for (uint64_t k0 = 0; k0 < p.K; k0 += K_CHUNK) {
        const uint64_t kc = p.K - k0 < K_CHUNK ? p.K - k0 : K_CHUNK;
        const uint64_t kb = (kc + BK - 1) / BK;
        PackArgs pa;
        auto operand = [&](PackOperand &o, const uint64_t *src, uint64_t ld, uint64_t rows, uint64_t rows_p, bool kc_, size_t planes) {
            o.src = src;
            o.ld = (uint32_t)ld;
            o.rows = (uint32_t)rows;
            o.row_blocks = (uint32_t)(rows_p / 32);
            o.planes = ws + planes;
            o.k_contiguous = kc_;
            o.vector_ok = kc_ && ld % 2 == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0;
        };
        // A is k-contiguous for op N (element (m, k) at A[m * lda + k]), B for op T
        operand(pa.op[0], p.op_a ? A + k0 * p.lda : A + k0, p.lda, p.M, w.Mp, !p.op_a, w.planes_a);
        operand(pa.op[1], p.op_b ? B + k0 : B + k0 * p.ldb, p.ldb, p.N, w.Np, p.op_b != 0, w.planes_b);
        pa.K = (uint32_t)kc;
        pa.KB = (uint32_t)kb;
        uint64_t ksplit = w.ksplit < kb ? w.ksplit : kb;
        pa.kb_per_split = (uint32_t)((kb + ksplit - 1) / ksplit);
        ksplit = (kb + pa.kb_per_split - 1) / pa.kb_per_split;
        // A's row blocks come first in the grid: with B's planes kept from the previous call only those are launched
        const bool keep_b = p.reuse_b && p.K <= K_CHUNK;
        const uint64_t row_blocks = (keep_b ? w.Mp : w.Mp + w.Np) / 32;
        hipLaunchKernelGGL(ipack64_kernel, dim3((unsigned)row_blocks, (unsigned)ksplit), dim3(PACK_THREADS), 0, st, pa);
        int rc = launch_status();
        if (rc) return rc;

        PArgs g;
        g.planes_a = ws + w.planes_a;
        g.planes_b = ws + w.planes_b;
        g.C = static_cast<uint64_t *>(p.C);
        g.M = (uint32_t)p.M; g.N = (uint32_t)p.N; g.KB = (uint32_t)kb;
        g.ldc = (uint32_t)p.ldc;
        g.tiles_m = (uint32_t)(w.Mp / BM);
        g.tiles_n = (uint32_t)(w.Np / BN);
        g.alpha = alpha;
        // every chunk after the first adds to what the chunks before it left in C
        g.beta = k0 == 0 ? beta : 1;
        g.epi = k0 == 0 ? p.epi : EPI_ALPHA_BETA;
        const bool edge = p.M % BM != 0 || p.N % BN != 0;
        rc = edge ? launch_product<true>(st, g) : launch_product<false>(st, g);
        if (rc) return rc;
    }
    return WK_OK;
}
