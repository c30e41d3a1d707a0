// 32-bit integer GEMM on the int8 matrix cores, exact modulo 2^32.
//
// The reference's integer GEMM (src/blas/kernels/gemm_*.cl with an integer `wks`) computes
// C = alpha*op(A)*op(B) + beta*C in the element width, i.e. modulo 2^32 for i32/u32.  There is no
// 32-bit integer matrix instruction, but the ring identity lets the int8 one do the work:
//
//   write every element in balanced digits,  a = sum_i 256^i s_i  (mod 2^32)  with s_i in [-128, 127]:
//   with c = 0x80808080 and t = a + c (carries and all, modulo 2^32), a = t - c = sum_i 256^i (t_i - 128)
//   over the unsigned bytes t_i of t, and t_i - 128 read as a signed byte is t_i ^ 0x80.  Then
//       sum_k a*b = sum_{i+j<=3} 256^(i+j) * sum_k s_i(a) s_j(b)              (mod 2^32)
//   (digit pairs with i+j >= 4 are multiples of 2^32).  The ten digit-pair sums are int8 x int8
//   products accumulated in int32 -- exactly v_mfma_i32_32x32x32_i8 -- and wraparound of those
//   accumulators is harmless because everything is taken modulo 2^32 anyway.  Elements of small
//   magnitude have zero upper digits, and zero padding is zero digits.  (The plain bytes of a with
//   0x80 taken off each -- no carries -- also work, with row and column sums of the elements as
//   correction terms; but then every small element has upper digits of -128 or 127, and with
//   operands that toggle all their bits the part holds a lower clock under the int8 matrix
//   instruction: 2048^3 with entries in [-100, 100] 81 against 61 us, 4096^3 536 against 390.)
//
// So one 32-bit product costs ten int8 matrix products; against the vector ALU (a 32-bit
// multiply-add per lane and clock at best) that is still several times faster.
//
// Work-group: BM/32 x 2 waves (256 or 512 threads), macro tile BM x 128 with BM = 64 or 128, wave tile 32 x 64 (two 32x32 blocks),
// four accumulator sets (one per shift i+j).  k-slab 32.  LDS holds, per operand and slab, four
// digit planes [row slot][32 bytes of k + 8 pad]; the loader XORs with c and transposes 4x4 bytes with
// v_perm_b32 so that every plane dword holds one digit of four consecutive k.
#include "wk_internal.hpp"

#include <cstring>

using namespace wk;

namespace {

typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(4))) u32x4_u { u32x4 v; };

constexpr int BN = 128, BK = 32; // BM (64 or 128) and the thread count 4 * BM are template parameters
// LDS geometry of a digit plane.  Row r of an operand lives at row slot (r % 4) * P + r / 4 and a
// slot is LDB = 40 bytes: the loader of an m/n-contiguous operand writes one dword to each of four
// ADJACENT rows per lane, lanes 16 bytes (four rows) apart, and without the regrouping those stores
// hit two banks 16 ways.  With it (found by enumerating strides and group pitches) loader stores are
// at most 2-way and the 8-byte fragment reads 2-way, which is their minimum.
constexpr int LDB = BK + 8;
// row-slot pitch of the four residue groups: 20 for a 64-row operand, 36 for a 128-row one
constexpr int group_pitch(int rows) { return rows == 64 ? 20 : 36; }
constexpr int plane_bytes(int rows) { return 4 * group_pitch(rows) * LDB; }
constexpr int slab_bytes(int bm) { return 4 * (plane_bytes(bm) + plane_bytes(BN)); }
template <int P> __device__ __forceinline__ constexpr int slot(int r) { return (r & 3) * P + (r >> 2); }
constexpr uint32_t CBIAS = 0x80808080u;

struct IArgs {
    const uint32_t *A, *B;
    uint32_t *C;
    uint32_t M, N, K, lda, ldb, ldc, tiles_m, tiles_n;
    int epi;
    uint32_t alpha, beta;
};

// 4x4 byte transpose: e[t] = element at k+t (bytes = digits 0..3); p[d] = digit d of k+0..k+3
__device__ __forceinline__ void digit_planes(const uint32_t e[4], uint32_t p[4]) {
    const uint32_t a = (e[0] + CBIAS) ^ CBIAS, b = (e[1] + CBIAS) ^ CBIAS, c = (e[2] + CBIAS) ^ CBIAS, d = (e[3] + CBIAS) ^ CBIAS;
    const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400u); // a0 b0 a1 b1
    const uint32_t ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602u); // a2 b2 a3 b3
    const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400u);
    const uint32_t cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602u);
    p[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u); // a0 b0 c0 d0
    p[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u); // a1 b1 c1 d1
    p[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
    p[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
}

// A_K / B_K: operand is k-contiguous in storage (A for op N, B for op T).  EDGE: ragged sizes or
// rows that are only element-aligned.
template <int BM, bool A_K, bool B_K, bool EDGE>
__global__ __launch_bounds__(4 * BM) __attribute__((amdgpu_waves_per_eu(2)))
void gemm_i32_mfma_kernel(IArgs g) {
    constexpr int NT = 4 * BM;               // BM/32 x 2 waves
    constexpr int P_A = group_pitch(BM), P_B = group_pitch(BN);
    constexpr int PLANE_A = plane_bytes(BM), PLANE_B = plane_bytes(BN), SLAB_BYTES = slab_bytes(BM);
    extern __shared__ __align__(16) unsigned char lds_raw[];
    unsigned char *slabs = lds_raw;                                               // [2][SLAB_BYTES]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
    // grouped walk over the tiles: 8 tile rows at a time
    uint32_t tile_m, tile_n;
    {
        const uint32_t pid = blockIdx.x, group_size = 8 * g.tiles_n, group = pid / group_size, first_m = group * 8;
        const uint32_t gsz = min(g.tiles_m - first_m, 8u), in_group = pid - group * group_size;
        tile_m = first_m + in_group % gsz;
        tile_n = in_group / gsz;
    }
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    i32x16 acc[4][2];
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[s][b][r] = 0;

    // ---- loader --------------------------------------------------------------------------------
    // k-contiguous operand of ROWS rows: vector q -> (row = q / 8, k = 4 * (q % 8)), ROWS * 8 / NT per thread.
    // otherwise a thread owns one patch of 4 k x 4 rows: patch q -> (k = 4 * (q / (ROWS/4)), row = 4 * (q % (ROWS/4)));
    // there are ROWS * 2 patches; A's go to the first threads, B's to the last, so that with 512 threads
    // two patch-loaded operands land on different threads.
    constexpr int A_NV = A_K ? BM * 8 / NT : 4, B_NV = B_K ? BN * 8 / NT : 4;
    u32x4 ra[A_NV], rb[B_NV];

    auto load_vec = [&](const uint32_t *base, uint32_t ld, uint32_t r, uint32_t r_lim, uint32_t c, uint32_t c_lim) -> u32x4 {
        const uint32_t *p = base + (size_t)r * ld + c;
        if constexpr (!EDGE) {
            return *reinterpret_cast<const u32x4 *>(p);
        } else {
            u32x4 v = {0u, 0u, 0u, 0u};
            if (r < r_lim) {
                if (c + 4 <= c_lim) {
                    v = reinterpret_cast<const u32x4_u *>(p)->v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (c + e < c_lim) v[e] = p[e];
                }
            }
            return v;
        }
    };
    auto gload = [&](u32x4 *dst, const uint32_t *base, uint32_t ld, uint32_t row0, uint32_t row_lim, uint32_t k0, auto kc_tag,
                     auto rows_tag, auto first_tag) {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        constexpr int T0 = decltype(first_tag)::value; // first thread of the patch loaders
        if constexpr (KC) {
#pragma unroll
            for (int i = 0; i < ROWS * 8 / NT; ++i) {
                const int q = tid + i * NT;
                dst[i] = load_vec(base, ld, row0 + q / 8, row_lim, k0 + 4 * (q % 8), g.K);
            }
        } else {
            const int pq = tid - T0;
            if (pq >= 0 && pq < ROWS * 2) {
                const uint32_t k = k0 + 4 * (pq / (ROWS / 4)), c = row0 + 4 * (pq % (ROWS / 4));
#pragma unroll
                for (int t = 0; t < 4; ++t) dst[t] = load_vec(base, ld, k + t, g.K, c, row_lim);
            }
        }
    };
    // registers -> digit planes in LDS
    auto sstore = [&](unsigned char *planes, const u32x4 *src, auto kc_tag, auto rows_tag, auto first_tag) {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        constexpr int T0 = decltype(first_tag)::value;
        constexpr int P = group_pitch(ROWS), plane_bytes = 4 * P * LDB;
        if constexpr (KC) {
#pragma unroll
            for (int i = 0; i < ROWS * 8 / NT; ++i) {
                const int q = tid + i * NT;
                const uint32_t e[4] = {src[i][0], src[i][1], src[i][2], src[i][3]};
                uint32_t p[4];
                digit_planes(e, p);
                const int off = slot<P>(q / 8) * LDB + 4 * (q % 8);
#pragma unroll
                for (int d = 0; d < 4; ++d) *reinterpret_cast<uint32_t *>(planes + d * plane_bytes + off) = p[d];
            }
        } else {
            const int pq = tid - T0;
            if (pq >= 0 && pq < ROWS * 2) {
                const int koff = 4 * (pq / (ROWS / 4)), row = 4 * (pq % (ROWS / 4));
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint32_t e[4] = {src[0][c], src[1][c], src[2][c], src[3][c]};
                    uint32_t p[4];
                    digit_planes(e, p);
                    const int off = slot<P>(row + c) * LDB + koff;
#pragma unroll
                    for (int d = 0; d < 4; ++d) *reinterpret_cast<uint32_t *>(planes + d * plane_bytes + off) = p[d];
                }
            }
        }
    };
    using std::integral_constant;
    constexpr int T0_A = 0, T0_B = NT - BN * 2;
    auto load_ab = [&](uint32_t k0) {
        gload(ra, g.A, g.lda, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{}, integral_constant<int, T0_A>{});
        gload(rb, g.B, g.ldb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{}, integral_constant<int, T0_B>{});
    };
    auto store_ab = [&](int buf) {
        unsigned char *s = slabs + buf * SLAB_BYTES;
        sstore(s, ra, integral_constant<bool, A_K>{}, integral_constant<int, BM>{}, integral_constant<int, T0_A>{});
        sstore(s + 4 * PLANE_A, rb, integral_constant<bool, B_K>{}, integral_constant<int, BN>{}, integral_constant<int, T0_B>{});
    };

    // ---- matrix work of one slab ----------------------------------------------------------------
    // operand of v_mfma_i32_32x32x32_i8: lane l supplies row l%32 and 16 bytes of k; which k a byte
    // position stands for is the same for both operands, so reading both with the same formula
    // (bytes 16*(l/32) .. +15 of the slab) pairs every k of A with the same k of B.
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    struct alignas(8) Frag { long lo, hi; }; // row slots are 8-byte aligned: two 8-byte reads
    auto frag = [](const unsigned char *p) -> i32x4 {
        const Frag f = *reinterpret_cast<const Frag *>(p);
        i32x4 v;
        __builtin_memcpy(&v, &f, 16);
        return v;
    };
    auto compute = [&](int buf) {
        const unsigned char *sa = slabs + buf * SLAB_BYTES + slot<P_A>(wm * 32 + l32) * LDB + 16 * lhi;
        const unsigned char *sb = slabs + buf * SLAB_BYTES + 4 * PLANE_A + slot<P_B>(wn * 64 + l32) * LDB + 16 * lhi;
        i32x4 a[4], b[2][4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            a[d] = frag(sa + d * PLANE_A);
            b[0][d] = frag(sb + d * PLANE_B);
            b[1][d] = frag(sb + d * PLANE_B + 8 * LDB); // 32 rows further: same residue group, 8 slots on
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i <= s; ++i)
#pragma unroll
                for (int blk = 0; blk < 2; ++blk)
                    acc[s][blk] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[blk][s - i], acc[s][blk], 0, 0, 0);
    };

    const uint32_t ktiles = (g.K + BK - 1) / BK;
    load_ab(0);
    store_ab(0);
    __syncthreads();
    for (uint32_t kt = 0; kt < ktiles; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < ktiles;
        if (more) load_ab((kt + 1) * BK);
        compute(cur);
        if (more) {
            store_ab(cur ^ 1); // buffer cur^1 was last read before the previous barrier
            __syncthreads();
        }
    }

    // ---- epilogue: register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 block -----
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
        const uint32_t col = n0 + wn * 64 + blk * 32 + l32;
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
            const uint32_t row = m0 + wm * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
            uint32_t v = (uint32_t)acc[0][blk][r] + ((uint32_t)acc[1][blk][r] << 8) + ((uint32_t)acc[2][blk][r] << 16) +
                         ((uint32_t)acc[3][blk][r] << 24);
            if (g.epi == EPI_ALPHA) v = g.alpha * v;
            else if (g.epi == EPI_ALPHA_BETA) v = g.alpha * v + g.beta * old[r];
            if (!EDGE || ((row < g.M) & (col < g.N))) g.C[(size_t)row * g.ldc + col] = v;
        }
    }
}

template <int BM, bool AK, bool BKC, bool EDGE> int launch_one(hipStream_t st, const GemmProblem &p) {
    constexpr int NT = 4 * BM;
    constexpr size_t lds = 2 * slab_bytes(BM);
    auto kern = gemm_i32_mfma_kernel<BM, AK, BKC, EDGE>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) { (void)hipGetLastError(); return hip_code(attr); }
    IArgs g;
    g.A = static_cast<const uint32_t *>(p.A);
    g.B = static_cast<const uint32_t *>(p.B);
    g.C = static_cast<uint32_t *>(p.C);
    g.M = (uint32_t)p.M; g.N = (uint32_t)p.N; g.K = (uint32_t)p.K;
    g.lda = (uint32_t)p.lda; g.ldb = (uint32_t)p.ldb; g.ldc = (uint32_t)p.ldc;
    g.tiles_m = (uint32_t)((p.M + BM - 1) / BM);
    g.tiles_n = (uint32_t)((p.N + BN - 1) / BN);
    g.epi = p.epi;
    std::memcpy(&g.alpha, p.alpha, 4);
    std::memcpy(&g.beta, p.beta, 4);
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(NT), lds, st, g);
    return launch_status();
}

template <int BM> int launch_bm(hipStream_t st, const GemmProblem &p, bool edge) {
    const int sel = (p.op_a ? 0 : 2) | (p.op_b ? 1 : 0); // bit1: A k-contiguous, bit0: B k-contiguous
#define WK_CASE(AK, BKC) return edge ? launch_one<BM, AK, BKC, true>(st, p) : launch_one<BM, AK, BKC, false>(st, p)
    switch (sel) {
    case 0: WK_CASE(false, false);
    case 1: WK_CASE(false, true);
    case 2: WK_CASE(true, false);
    default: WK_CASE(true, true);
    }
#undef WK_CASE
}

} // namespace

int wk::gemm_i32_mfma_launch_64(hipStream_t st, const GemmProblem &p, bool edge) { return launch_bm<64>(st, p, edge); }
int wk::gemm_i32_mfma_launch_128(hipStream_t st, const GemmProblem &p, bool edge) { return launch_bm<128>(st, p, edge); }
