// 32-bit integer GEMM on the int8 matrix cores with a pack pass: the two-launch form of
// wk_gemm_imfma.hip, used when the caller brings a workspace (blas.PackedTensors does, as the
// reference's PackedTensors brings packed_a / packed_b and runs its pack kernel before every
// product: src/blas/gemm.zig:272-357, 705-720).
//
// The arithmetic is the same ring identity (a = S(a) + c with c = 0x80808080, ten signed-digit
// products, row and column sums; see wk_gemm_imfma.hip).  What changes is where the digits are made:
//
//   pass 1  ipack_kernel      reads op(A) and op(B) once, whatever their layout, and writes their
//                             signed-digit planes in the order the matrix instruction eats them:
//                             1 KiB blocks, one per (32 rows, 32 k, digit), lane l of a wavefront
//                             owning bytes 16 l .. 16 l + 15 = row l % 32, k 16 (l / 32) .. + 15.
//                             Rows and k beyond the matrix are zero digits.  It also leaves the row
//                             sums of the raw elements, one partial per k-range of the launch.
//   pass 2  gemm_i32_packed_kernel   128 x 128 tile, 8 waves, k-slab 32: 32 KiB of blocks per slab
//                             go global -> registers -> LDS as plain 16-byte copies, fragments come
//                             back with one conflict-free 16-byte LDS read each, and the loop is
//                             otherwise matrix instructions (20 per wave and slab).  No digit
//                             arithmetic, no edge cases (the planes are padded to the tile), one
//                             set of staging registers that fits beside the 128 accumulators.
//
// Workspace: 128 bytes per (padded row, 32 k) of each operand + the partial sums; for 2048^3 that
// is 2 x 16 MiB.  The pack pass costs what reading A and B once and writing as much costs.
#include "wk_internal.hpp"

#include <cstring>
#include <type_traits>

using namespace wk;

namespace {

typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(4))) u32x4_u { u32x4 v; };

constexpr uint32_t CBIAS = 0x80808080u;
constexpr int TILE = 128, BK = 32, BLOCK_BYTES = 1024, GROUP_BYTES = 4 * BLOCK_BYTES; // 4 digits of one (32 rows, 32 k)
constexpr int PACK_THREADS = 256;
constexpr uint32_t MAX_KSPLIT = 16;

struct Layout {
    uint64_t Mp, Np, KB, ksplit;
    size_t planes_a, planes_b, sums_a, sums_b, total; // byte offsets into the workspace
};

Layout make_layout(uint64_t M, uint64_t N, uint64_t K) {
    Layout w;
    w.Mp = (M + TILE - 1) / TILE * TILE;
    w.Np = (N + TILE - 1) / TILE * TILE;
    w.KB = (K + BK - 1) / BK;
    // enough work-groups in the pack launch to fill the chip: (Mp + Np) / 32 row blocks x ksplit
    uint64_t ks = 2048 / ((w.Mp + w.Np) / 32);
    ks = ks < 1 ? 1 : ks > MAX_KSPLIT ? MAX_KSPLIT : ks;
    if (ks > w.KB) ks = w.KB;
    w.ksplit = ks;
    w.planes_a = 0;
    w.planes_b = w.planes_a + (size_t)w.Mp / 32 * w.KB * GROUP_BYTES;
    w.sums_a = w.planes_b + (size_t)w.Np / 32 * w.KB * GROUP_BYTES;
    w.sums_b = w.sums_a + (size_t)w.ksplit * w.Mp * 4;
    w.total = w.sums_b + (size_t)w.ksplit * w.Np * 4;
    return w;
}

// 4x4 byte transpose: e[t] = element at k+t (bytes = digits 0..3) -> p[d] = digit d of k+0..k+3, signed form
__device__ __forceinline__ void digit_planes(const uint32_t e[4], uint32_t p[4]) {
    const uint32_t a = e[0] ^ CBIAS, b = e[1] ^ CBIAS, c = e[2] ^ CBIAS, d = e[3] ^ CBIAS;
    const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400u), ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602u);
    const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400u), cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602u);
    p[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
    p[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
    p[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
    p[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
}

struct PackOperand {
    const uint32_t *src;   // element (r, k) at src[r * ld + k] (k-contiguous) or src[k * ld + r]
    uint32_t ld, rows, row_blocks; // true rows; padded rows / 32
    unsigned char *planes;
    uint32_t *sums;        // [ksplit][row_blocks * 32]
    uint32_t k_contiguous, vector_ok; // vector_ok: 16-byte loads along k are aligned
};
struct PackArgs {
    PackOperand op[2];
    uint32_t K, KB, kb_per_split;
};

// blockIdx.x: row block of A, then of B; blockIdx.y: k-range.  Wave w of the work-group takes the
// k-blocks start + w, start + w + 4, ...; lane l the row l % 32 and the 16 k of half l / 32.
__global__ __launch_bounds__(PACK_THREADS) void ipack_kernel(PackArgs g) {
    __shared__ uint32_t partial[PACK_THREADS];
    const int which = blockIdx.x >= g.op[0].row_blocks;
    const PackOperand &o = g.op[which];
    const uint32_t rb = blockIdx.x - (which ? g.op[0].row_blocks : 0u);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
    const uint32_t row = rb * 32 + l32;
    const bool row_ok = row < o.rows;
    const uint32_t kb_begin = blockIdx.y * g.kb_per_split, kb_end = min(g.KB, kb_begin + g.kb_per_split);
    uint32_t sum = 0;
    for (uint32_t kb = kb_begin + wave; kb < kb_end; kb += PACK_THREADS / 64) {
        const uint32_t k0 = kb * BK + 16 * half;
        uint32_t e[16];
        if (o.k_contiguous) {
            const uint32_t *p = o.src + (size_t)row * o.ld + k0;
            if (row_ok && o.vector_ok && k0 + 16 <= g.K) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(p + 4 * q);
                    e[4 * q] = v[0]; e[4 * q + 1] = v[1]; e[4 * q + 2] = v[2]; e[4 * q + 3] = v[3];
                }
#pragma unroll
                for (int j = 0; j < 16; ++j) sum += e[j];
            } else {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const bool ok = row_ok && k0 + j < g.K;
                    const uint32_t v = ok ? p[j] : 0u;
                    sum += v;
                    e[j] = ok ? v : CBIAS; // CBIAS has all-zero signed digits
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const bool ok = row_ok && k0 + j < g.K;
                const uint32_t v = ok ? o.src[(size_t)(k0 + j) * o.ld + row] : 0u;
                sum += v;
                e[j] = ok ? v : CBIAS;
            }
        }
        u32x4 out[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t p4[4];
            digit_planes(e + 4 * q, p4);
#pragma unroll
            for (int d = 0; d < 4; ++d) out[d][q] = p4[d];
        }
        unsigned char *dst = o.planes + ((size_t)rb * g.KB + kb) * GROUP_BYTES + lane * 16;
#pragma unroll
        for (int d = 0; d < 4; ++d) *reinterpret_cast<u32x4 *>(dst + d * BLOCK_BYTES) = out[d];
    }
    partial[tid] = sum;
    __syncthreads();
    if (tid < 32) {
        uint32_t s = 0;
#pragma unroll
        for (int i = 0; i < PACK_THREADS / 32; ++i) s += partial[tid + 32 * i];
        o.sums[(size_t)blockIdx.y * o.row_blocks * 32 + rb * 32 + tid] = s;
    }
}

struct PArgs {
    const unsigned char *planes_a, *planes_b;
    const uint32_t *sums_a, *sums_b;
    uint32_t *C;
    uint32_t M, N, K, KB, Mp, Np, ksplit, ldc, tiles_m, tiles_n;
    int epi;
    uint32_t alpha, beta;
};

// BM x 128 tile, BM / 32 x 2 waves.  BM = 128 (one 8-wave work-group per CU) is what is launched.
// BM = 64 -- two independent 4-wave work-groups per CU, so that the two waves of a SIMD are not held
// in the same phase by one barrier -- was measured and is slower (8192^3: 207 against 222 TOP/s): it
// copies half as much again per matrix instruction.
template <int BM> struct PackedTile {
    static constexpr int NT = BM * 4;                       // threads
    static constexpr int GROUPS = BM / 32 + TILE / 32;      // 4 KiB groups per slab: A row blocks, then B column blocks
    static constexpr int STAGE_BYTES = GROUPS * GROUP_BYTES;
    static constexpr int GROUPS_PER_PASS = NT * 16 / GROUP_BYTES; // 1 or 2
    static constexpr int PASSES = GROUPS / GROUPS_PER_PASS;
    static constexpr size_t LDS_BYTES = 2 * STAGE_BYTES + (BM + TILE) * sizeof(uint32_t);
};

template <int BM, bool EDGE>
__global__ __launch_bounds__(BM * 4) __attribute__((amdgpu_waves_per_eu(2)))
void gemm_i32_packed_kernel(PArgs g) {
    using TL = PackedTile<BM>;
    constexpr int STAGE_BYTES = TL::STAGE_BYTES, PASSES = TL::PASSES, A_GROUPS = BM / 32;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    unsigned char *stages = lds_raw;                                              // [2][STAGE_BYTES]
    uint32_t *row_sum = reinterpret_cast<uint32_t *>(lds_raw + 2 * STAGE_BYTES);  // [BM]
    uint32_t *col_sum = row_sum + BM;                                             // [TILE]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
    uint32_t tile_m, tile_n;
    {
        const uint32_t pid = blockIdx.x, group_size = 8 * g.tiles_n, group = pid / group_size, first_m = group * 8;
        const uint32_t gsz = min(g.tiles_m - first_m, 8u), in_group = pid - group * group_size;
        tile_m = first_m + in_group % gsz;
        tile_n = in_group / gsz;
    }
    const uint32_t m0 = tile_m * BM, n0 = tile_n * TILE;

    if (tid < BM + TILE) {
        const uint32_t *src = tid < BM ? g.sums_a + m0 + tid : g.sums_b + n0 + (tid - BM);
        const uint32_t stride = tid < BM ? g.Mp : g.Np;
        uint32_t s = 0;
        for (uint32_t i = 0; i < g.ksplit; ++i) s += src[(size_t)i * stride];
        row_sum[tid] = s; // col_sum follows row_sum
    }

    i32x16 acc[4][2];
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[s][b][r] = 0;

    // Copy of one slab: GROUPS groups of 4 KiB; pass i moves group(s) i * GROUPS_PER_PASS (+ tid / 256).
    // Each group stream of this thread is a buffer resource (scalar registers) over the KB * 4 KiB of
    // that group; a load is resource + scalar slab offset + the lane's fixed 32-bit offset, so the
    // loop holds no vector address arithmetic (whose result registers the compiler would share with
    // the load destinations, waiting for every load in flight first).
    const int grp = __builtin_amdgcn_readfirstlane(tid >> 8);
    const int within = (tid & 255) * 16;
    __amdgpu_buffer_rsrc_t src[PASSES];
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
        const int gi = TL::GROUPS_PER_PASS * i + grp; // < A_GROUPS: A row blocks, then B column blocks
        const unsigned char *p = gi < A_GROUPS ? g.planes_a + (size_t)(tile_m * A_GROUPS + gi) * g.KB * GROUP_BYTES
                                               : g.planes_b + (size_t)(tile_n * 4 + gi - A_GROUPS) * g.KB * GROUP_BYTES;
        src[i] = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char *>(p), 0, (int)(g.KB * GROUP_BYTES), 0x00020000);
    }
    // Two register sets: the slab loaded in step kb is stored to LDS at the end of step kb + 1 and
    // used in step kb + 2, so a load has two slabs of matrix work to arrive.
    // (past the end the last slab is loaded again and dropped: no branch, so the loads stay where
    // they are written, ahead of the matrix work)
    u32x4 staged[2][PASSES];
    auto gload = [&](u32x4 *dst, uint32_t kb) {
        const int off = (int)(min(kb, g.KB - 1) * GROUP_BYTES);
#pragma unroll
        for (int i = 0; i < PASSES; ++i) dst[i] = __builtin_amdgcn_raw_buffer_load_b128(src[i], within, off, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto sstore = [&](const u32x4 *from, int buf) {
#pragma unroll
        for (int i = 0; i < PASSES; ++i)
            *reinterpret_cast<u32x4 *>(stages + buf * STAGE_BYTES + (TL::GROUPS_PER_PASS * i + grp) * GROUP_BYTES + within) = from[i];
    };
    auto compute = [&](int buf) {
        const unsigned char *sa = stages + buf * STAGE_BYTES + wm * GROUP_BYTES + lane * 16;
        const unsigned char *sb = stages + buf * STAGE_BYTES + (A_GROUPS + wn * 2) * GROUP_BYTES + lane * 16;
        i32x4 a[4], b[2][4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            a[d] = *reinterpret_cast<const i32x4 *>(sa + d * BLOCK_BYTES);
            b[0][d] = *reinterpret_cast<const i32x4 *>(sb + d * BLOCK_BYTES);
            b[1][d] = *reinterpret_cast<const i32x4 *>(sb + GROUP_BYTES + d * BLOCK_BYTES);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i <= s; ++i)
#pragma unroll
                for (int blk = 0; blk < 2; ++blk)
                    acc[s][blk] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[blk][s - i], acc[s][blk], 0, 0, 0);
    };
    // one step: slab kb is in LDS stage `cur`, slab kb + 1 in flight in staged[other]
    auto step = [&](uint32_t kb, auto cur_tag) {
        constexpr int cur = decltype(cur_tag)::value;
        gload(staged[cur], kb + 2);
        compute(cur);
        if (kb + 1 < g.KB) {
            sstore(staged[cur ^ 1], cur ^ 1);
            __syncthreads();
        }
    };

    gload(staged[0], 0);
    gload(staged[1], 1);
    sstore(staged[0], 0);
    __syncthreads();
    for (uint32_t kb = 0; kb < g.KB; kb += 2) {
        step(kb, std::integral_constant<int, 0>{});
        if (kb + 1 < g.KB) step(kb + 1, std::integral_constant<int, 1>{});
    }

    // epilogue: register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 block
    const uint32_t kc2 = g.K * (CBIAS * CBIAS);
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
        const uint32_t lcol = wn * 64 + blk * 32 + l32, col = n0 + lcol;
        const uint32_t csum = col_sum[lcol];
        uint32_t old[16];
        if (g.epi == EPI_ALPHA_BETA) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + wm * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                const uint32_t rowc = EDGE ? min(row, g.M - 1) : row, colc = EDGE ? min(col, g.N - 1) : col;
                old[r] = g.C[(size_t)rowc * g.ldc + colc];
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t lrow = wm * 32 + 8 * (r / 4) + 4 * lhi + (r % 4), row = m0 + lrow;
            uint32_t v = (uint32_t)acc[0][blk][r] + ((uint32_t)acc[1][blk][r] << 8) + ((uint32_t)acc[2][blk][r] << 16) +
                         ((uint32_t)acc[3][blk][r] << 24);
            v += CBIAS * (row_sum[lrow] + csum) - kc2;
            if (g.epi == EPI_ALPHA) v = g.alpha * v;
            else if (g.epi == EPI_ALPHA_BETA) v = g.alpha * v + g.beta * old[r];
            if (!EDGE || ((row < g.M) & (col < g.N))) g.C[(size_t)row * g.ldc + col] = v;
        }
    }
}

template <int BM, bool EDGE> int launch_packed(hipStream_t st, PArgs g) {
    constexpr size_t lds = PackedTile<BM>::LDS_BYTES;
    auto kern = gemm_i32_packed_kernel<BM, EDGE>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) { (void)hipGetLastError(); return hip_code(attr); }
    g.tiles_m = g.Mp / BM;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(PackedTile<BM>::NT), lds, st, g);
    return launch_status();
}

} // namespace

// 0: this problem cannot take the packed path (a group stream of KB * 4 KiB must fit the 31-bit extent
// of a buffer resource, the dimensions 31 bits)
size_t wk::gemm_i32_packed_workspace_bytes(uint64_t M, uint64_t N, uint64_t K) {
    if (!M || !N || !K || M > 0x7fffffffull || N > 0x7fffffffull || K > (0x7fffffffull / GROUP_BYTES) * BK) return 0;
    return make_layout(M, N, K).total;
}

int wk::gemm_i32_packed_launch(hipStream_t st, const GemmProblem &p, void *workspace, size_t workspace_bytes) {
    if (!gemm_i32_packed_workspace_bytes(p.M, p.N, p.K)) return WK_E_INVALID_VALUE;
    const Layout w = make_layout(p.M, p.N, p.K);
    if (!workspace || workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(workspace) & 15u)) return WK_E_INVALID_VALUE;
    unsigned char *ws = static_cast<unsigned char *>(workspace);

    PackArgs pa;
    auto operand = [&](PackOperand &o, const void *src, uint64_t ld, uint64_t rows, uint64_t rows_p, bool kc, size_t planes,
                       size_t sums) {
        o.src = static_cast<const uint32_t *>(src);
        o.ld = (uint32_t)ld;
        o.rows = (uint32_t)rows;
        o.row_blocks = (uint32_t)(rows_p / 32);
        o.planes = ws + planes;
        o.sums = reinterpret_cast<uint32_t *>(ws + sums);
        o.k_contiguous = kc;
        o.vector_ok = kc && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0;
    };
    operand(pa.op[0], p.A, p.lda, p.M, w.Mp, !p.op_a, w.planes_a, w.sums_a); // A is k-contiguous for op N
    operand(pa.op[1], p.B, p.ldb, p.N, w.Np, p.op_b != 0, w.planes_b, w.sums_b); // B for op T
    pa.K = (uint32_t)p.K;
    pa.KB = (uint32_t)w.KB;
    pa.kb_per_split = (uint32_t)((w.KB + w.ksplit - 1) / w.ksplit);
    hipLaunchKernelGGL(ipack_kernel, dim3((unsigned)((w.Mp + w.Np) / 32), (unsigned)w.ksplit), dim3(PACK_THREADS), 0, st, pa);
    int rc = launch_status();
    if (rc) return rc;

    PArgs g;
    g.planes_a = ws + w.planes_a;
    g.planes_b = ws + w.planes_b;
    g.sums_a = reinterpret_cast<const uint32_t *>(ws + w.sums_a);
    g.sums_b = reinterpret_cast<const uint32_t *>(ws + w.sums_b);
    g.C = static_cast<uint32_t *>(p.C);
    g.M = (uint32_t)p.M; g.N = (uint32_t)p.N; g.K = (uint32_t)p.K;
    g.KB = (uint32_t)w.KB; g.Mp = (uint32_t)w.Mp; g.Np = (uint32_t)w.Np; g.ksplit = (uint32_t)w.ksplit;
    g.ldc = (uint32_t)p.ldc;
    g.tiles_m = (uint32_t)(w.Mp / TILE);
    g.tiles_n = (uint32_t)(w.Np / TILE);
    g.epi = p.epi;
    std::memcpy(&g.alpha, p.alpha, 4);
    std::memcpy(&g.beta, p.beta, 4);
    const bool edge = p.M % TILE != 0 || p.N % TILE != 0;
    return edge ? launch_packed<128, true>(st, g) : launch_packed<128, false>(st, g);
}
