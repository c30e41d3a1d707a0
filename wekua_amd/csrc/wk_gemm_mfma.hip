// f32 / f64 GEMM on the CDNA4 matrix cores (gfx950).
//
//   f32: v_mfma_f32_32x32x2_f32   -- one wavefront computes a 32x32 block per instruction,
//   f64: v_mfma_f64_16x16x4_f64   -- one wavefront computes a 16x16 block per instruction.
//
// Structure (both precisions):
//   * work-group = WAVES_M x WAVES_N wavefronts (64 lanes each), macro tile BM x BN of C,
//     k advanced in steps of BK through two LDS buffers (one barrier per step);
//   * the next k-slab is fetched from global memory into registers (16-byte loads along
//     whichever index is contiguous for the transpose flag) while the matrix cores work on
//     the current LDS buffer, then written to the other buffer;
//   * LDS layouts are chosen per operand so that both the 16-byte stores and the fragment
//     reads are bank-conflict free:
//        k-contiguous operand (A for op_a=N, B for op_b=T): [row][BK + pad], fragments are
//        one 16-byte read per lane (4 consecutive k of one row);
//        m/n-contiguous operand (A for op_a=T, B for op_b=N): [k][rows + pad], fragments
//        are 4-byte reads, 32 consecutive lanes on consecutive addresses;
//     both give lane l the k values k0 + KL*(l / ROWS) + t for t = 0..KL-1, so the two
//     operands of one instruction always agree on k;
//   * tiles are walked in groups of GROUP_M = 8 tile rows, which with the round-robin dispatch
//     of work-groups over the 8 XCDs makes all XCDs stream the same panel of B together;
//   * the epilogue applies the reference's option semantics (src/blas/gemm.zig:500-501,
//     591-602): store / alpha*acc / alpha*acc + beta*C_old.
//
// The EDGE instantiation handles ragged M, N, K and rows that are only element-aligned: tiles on
// the border of C and the slab holding the k tail bounds-check every global access, everything
// else takes unchecked element-aligned 16-byte loads.  The interior instantiation assumes
// M % BM == N % BN == K % BK == 0 and 16-byte aligned rows.
#include "wk_internal.hpp"

#include <cmath>
#include <cstdlib>
#include <algorithm>
#include <cstring>

using namespace wk;

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
// 16-byte vectors that are only element-aligned: gfx950 global loads take any dword-aligned
// address, so rows with an odd leading dimension still move 16 bytes per lane
struct __attribute__((packed, aligned(4))) f32x4_u { f32x4 v; };
struct __attribute__((packed, aligned(8))) f64x2_u { f64x2 v; };

constexpr int GROUP_M = 8;

template <typename T> struct MArgs {
    const T *A, *B;
    T *C;
    uint32_t M, N, K;
    uint32_t lda, ldb, ldc;
    uint32_t tiles_m, tiles_n;
    uint32_t xcd_remap; // 1: renumber work-groups so that each XCD gets a contiguous run of tiles
    int epi;
    T alpha, beta;
    // epilogue extension (kernels instantiated with EXT): C = act(acc + bias[col]); bias may be null
    const T *bias;
    int act;
    // k split over work-groups (kernels instantiated with SPLIT): blockIdx.y takes k values
    // [blockIdx.y * klen, min(K, (blockIdx.y + 1) * klen)) of the sum, the partial tiles meet in
    // `partials` ([share][tile][BM * BN]) and the work-group that arrives last at counters[tile] adds
    // them up.  Unused (klen 0, null pointers) by every other kernel.
    uint32_t klen;
    T *partials;
    uint32_t *counters;
    // first tile number of this launch (a product may be launched as a body of whole rounds of tiles
    // and a tail whose k is split; the tail's tile numbers follow the body's)
    uint32_t pid_offset;
};

// blockIdx.x -> (tile_m, tile_n): grouped walk, GROUP_M tile rows at a time.
// Work-groups are dealt to the 8 XCDs round-robin (work-group b runs on XCD b % 8; checked by
// reading the XCC_ID register).  Without renumbering and with GROUP_M = 8 every XCD owns one tile
// row of the group and all XCDs sweep the SAME columns of B at the same time: B is fetched from
// HBM once per sweep and served to the other XCDs from the shared 256 MB Infinity Cache, while
// the A panel of a tile row stays in that XCD's own L2.  That is the right order for launches of
// several rounds.  With renumbering (remap) each XCD gets a compact block of tiles, which wins
// when the whole launch is resident at once and lives in the L2s.  (Also measured for 8192^3: a
// compact 4 x 8 block of tiles per XCD inside each round of 8 x 32 tiles, which on paper halves the
// L2 misses, runs at the same speed and misses 18 % MORE: the work-groups of an XCD are not close
// enough in k for the 4 MB L2 to hold what they would share.)
__device__ __forceinline__ void tile_coords(uint32_t tiles_m, uint32_t tiles_n, uint32_t &tm, uint32_t &tn, uint32_t remap = 0,
                                            uint32_t pid_offset = 0) {
    uint32_t pid = blockIdx.x;
    if (remap && (gridDim.x % 8) == 0) pid = (pid % 8) * (gridDim.x / 8) + pid / 8;
    pid += pid_offset;
    const uint32_t group_size = GROUP_M * tiles_n;
    const uint32_t group = pid / group_size;
    const uint32_t first_m = group * GROUP_M;
    const uint32_t gsz = min(tiles_m - first_m, (uint32_t)GROUP_M);
    const uint32_t in_group = pid - group * group_size;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

// ------------------------------------------------------------------------------------ f32 ---

// LDS geometry of one operand slab (ROWS rows of the m or n index, BK values of k)
template <int ROWS, int BK, bool KCONTIG> struct Slab {
    static constexpr int LD = KCONTIG ? BK + 4 : ROWS + 8; // floats per LDS row
    static constexpr int SIZE = KCONTIG ? ROWS * LD : BK * LD;
};

// KS > 1: KS groups of WAVES_M x WAVES_N wavefronts share the macro tile and split every k-slab of
// KS * BK values between them (group kg multiplies the k values kg * BK .. kg * BK + BK - 1 of the
// slab); their accumulators are added through LDS before the epilogue.  For launches that put a
// single small work-group on a CU this doubles the wavefronts a SIMD can switch between.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int OCC, bool A_K, bool B_K, bool EDGE, bool EXT = false, int KS = 1, int LSEL = -1,
          bool SPLIT = false>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64 * KS) __attribute__((amdgpu_waves_per_eu(OCC)))
void gemm_f32_mfma_kernel(MArgs<float> g) {
    static_assert(!SPLIT || KS == 1, "k is split over work-groups or inside one, not both");
    constexpr int NT = WAVES_M * WAVES_N * 64 * KS;
    constexpr int BKT = BK * KS; // k values per LDS slab
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int FM = WM / 32, FN = WN / 32;
    static_assert(WM % 32 == 0 && WN % 32 == 0 && BK % 8 == 0, "tile shape");
    using SA = Slab<BM, BKT, A_K>;
    using SB = Slab<BN, BKT, B_K>;
    constexpr int A_V4 = BM * BKT / 4 / NT, B_V4 = BN * BKT / 4 / NT; // 16-byte loads per thread per slab
    static_assert(A_V4 * NT * 4 == BM * BKT && B_V4 * NT * 4 == BN * BKT, "slab must divide over the threads");

    extern __shared__ __align__(16) float lds[];
    float *As = lds;                     // [2][SA::SIZE]
    float *Bs = lds + 2 * SA::SIZE;      // [2][SB::SIZE]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = (tid >> 6) % (WAVES_M * WAVES_N), kg = (tid >> 6) / (WAVES_M * WAVES_N);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    uint32_t tile_m, tile_n;
    tile_coords(g.tiles_m, g.tiles_n, tile_m, tile_n, g.xcd_remap, SPLIT ? g.pid_offset : 0u); // only a split tail starts past tile 0
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    if constexpr (SPLIT) { // this work-group's share of k; from here on the kernel sees a shorter product
        const uint32_t k_begin = blockIdx.y * g.klen;
        const uint32_t k_end = min(g.K, k_begin + g.klen);
        g.A += A_K ? (size_t)k_begin : (size_t)k_begin * g.lda;
        g.B += B_K ? (size_t)k_begin : (size_t)k_begin * g.ldb;
        g.K = k_end - k_begin;
    }
    // one solo iteration = FM*FN*BK/2 matrix instructions of 64 clocks = FM*FN*BK/4 sleep units

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // Which spelling of the main loop (described below); the bounds-checked instantiation has the
    // peeled ones only.
    // Staging registers, global -> LDS: one set.  (LOOP 2 on the small tile keeps two and requests
    // slab kt+2 while slab kt is computed: with one or two 64x64 tiles on a CU a slab's matrix work is
    // shorter than the latency of a global load.  LOOP 3 gets the same lead from one set.)
    constexpr int LOOP_WANTED = LSEL >= 0 ? LSEL : (BM * BN <= 128 * 128) ? 3 : B_K ? 3 : (A_K ? 0 : 5);
    constexpr int LOOP = (EDGE && LOOP_WANTED < 2) ? 2 : LOOP_WANTED;
    constexpr int PF = (BM * BN <= 64 * 64 && LOOP == 2) ? 2 : 1;
    f32x4 ra[PF][A_V4], rb[PF][B_V4];

    // ---- global -> registers -----------------------------------------------------------
    // KCONTIG: slab is ROWS x BK, q -> (row = q / (BK/4), c4 = q % (BK/4)), address row*ld + k0 + 4*c4
    // else   : slab is BK x ROWS, q -> (k = q / (ROWS/4), c4 = q % (ROWS/4)), address (k0+k)*ld + 4*c4
    // CHECK: bounds-check every access (edge tiles and the k tail); otherwise the slab lies inside
    // the operand and only the alignment of the 16-byte load differs between the instantiations.
    auto gload = [&](f32x4 *dst, const float *__restrict__ base, uint32_t ld, uint32_t row0, uint32_t row_lim,
                     uint32_t k0, auto kc_tag, auto rows_tag, auto nv_tag, auto check_tag) {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        constexpr int NV = decltype(nv_tag)::value;
        constexpr bool CHECK = decltype(check_tag)::value;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int q = tid + i * NT;
            uint32_t r, c;     // r: index along the row-of-storage direction, c: first of 4 contiguous
            uint32_t r_lim, c_lim;
            if constexpr (KC) {
                r = row0 + q / (BKT / 4); c = k0 + 4 * (q % (BKT / 4));
                r_lim = row_lim; c_lim = g.K;
            } else {
                r = k0 + q / (ROWS / 4); c = row0 + 4 * (q % (ROWS / 4));
                r_lim = g.K; c_lim = row_lim;
            }
            const float *p = base + (size_t)r * ld + c;
            if constexpr (!EDGE) {
                dst[i] = *reinterpret_cast<const f32x4 *>(p);
            } else if constexpr (!CHECK) {
                dst[i] = reinterpret_cast<const f32x4_u *>(p)->v;
            } else {
                // Clamp the address into the operand and load one raw vector; nothing here depends
                // on the loaded value, so the request stays in flight across the matrix work.  The
                // lanes that do not exist are sorted out when the vector is stored to LDS (fixup).
                const uint32_t rr = r < r_lim ? r : r_lim - 1;
                const uint32_t cc = c + 4 <= c_lim ? c : (c_lim >= 4 ? c_lim - 4 : 0);
                const float *q = base + (size_t)rr * ld + cc;
                f32x4 v;
                if (c_lim >= 4) { // uniform: operands narrower than one vector are read by element
                    v = reinterpret_cast<const f32x4_u *>(q)->v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = (uint32_t)e < c_lim ? q[e] : 0.f;
                }
                dst[i] = v;
            }
        }
    };
    // ---- registers -> LDS ------------------------------------------------------------------
    // FIX: the vectors came from the clamped loads of a checked slab: element e of the vector
    // that should start at column c sits at index (c - cc) + e of what was loaded, if it exists.
    auto sstore = [&](float *slab, const f32x4 *src, uint32_t row0, uint32_t row_lim, uint32_t k0, auto kc_tag, auto rows_tag,
                      auto nv_tag, auto fix_tag) {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        constexpr int NV = decltype(nv_tag)::value;
        constexpr bool FIX = decltype(fix_tag)::value;
        constexpr int LD = Slab<ROWS, BKT, KC>::LD;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int q = tid + i * NT;
            int off;
            if constexpr (KC) off = (q / (BKT / 4)) * LD + 4 * (q % (BKT / 4));
            else off = (q / (ROWS / 4)) * LD + 4 * (q % (ROWS / 4));
            f32x4 v = src[i];
            if constexpr (FIX) {
                // keeps the compiler from folding this path into the unchecked one as selects, which
                // would charge every interior slab for the lane sorting
                asm volatile("" ::: "memory");
                uint32_t r, c, r_lim, c_lim;
                if constexpr (KC) {
                    r = row0 + q / (BKT / 4); c = k0 + 4 * (q % (BKT / 4));
                    r_lim = row_lim; c_lim = g.K;
                } else {
                    r = k0 + q / (ROWS / 4); c = row0 + 4 * (q % (ROWS / 4));
                    r_lim = g.K; c_lim = row_lim;
                }
                const uint32_t cc = c + 4 <= c_lim ? c : (c_lim >= 4 ? c_lim - 4 : 0);
                const uint32_t shift = c - cc;
                const f32x4 t = v;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const uint32_t idx = shift + e;
                    float x = t[3];
                    x = idx == 2 ? t[2] : x;
                    x = idx == 1 ? t[1] : x;
                    x = idx == 0 ? t[0] : x;
                    const bool ok = (r < r_lim) & (c + e < c_lim);
                    v[e] = ok ? x : 0.f;
                }
            }
            *reinterpret_cast<f32x4 *>(slab + off) = v;
        }
    };

    using std::integral_constant;
    // In the bounds-checked instantiation most work is still interior: a tile that lies inside C
    // needs checks only on the slab that holds the k tail.  The choice is uniform over the work-group.
    const bool tile_inside = !EDGE || (m0 + BM <= g.M && n0 + BN <= g.N);
    const uint32_t k_inside = g.K - g.K % BKT; // slabs starting below this are complete
    // An edge tile away from the k tail needs less than the full treatment: rows and columns beyond
    // the matrix only feed entries of C that are never stored, so the clamped loads (which keep the
    // addresses inside the operand and deliver copies of valid data) can go to LDS as they are.  The
    // one exception is a vector that straddles the end of a row of storage, whose valid elements
    // arrive shifted: that happens only when the contiguous extent is not a multiple of the vector.
    const bool fix_a_always = !A_K && g.M % 4 != 0, fix_b_always = !B_K && g.N % 4 != 0;
    // How a slab is treated is a compile-time flavour of the loop that handles it, so that the loops
    // over complete slabs carry no trace of the checked paths:
    //   PLAIN    the slab lies inside both operands (the only flavour of the unchecked instantiation)
    //   CLAMPED  edge tile, complete slab: clamped loads, stored as they are unless a row end is straddled
    //   ANY      decided per slab at run time (the iterations that touch the k tail)
    enum { PLAIN = 0, CLAMPED = 1, ANY = 2 };
    // W: which operands (bit 0: A, bit 1: B)
    auto load_sel = [&](uint32_t k0, f32x4 *ra, f32x4 *rb, auto flavour_tag, auto which_tag) {
        constexpr int FL = decltype(flavour_tag)::value;
        constexpr int W = decltype(which_tag)::value;
        if (FL == PLAIN || (FL == ANY && tile_inside && k0 < k_inside)) {
            if constexpr (W & 1)
                gload(ra, g.A, g.lda, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{},
                      integral_constant<int, A_V4>{}, std::false_type{});
            if constexpr (W & 2)
                gload(rb, g.B, g.ldb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{},
                      integral_constant<int, B_V4>{}, std::false_type{});
        } else {
            if constexpr (W & 1)
                gload(ra, g.A, g.lda, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{},
                      integral_constant<int, A_V4>{}, std::true_type{});
            if constexpr (W & 2)
                gload(rb, g.B, g.ldb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{},
                      integral_constant<int, B_V4>{}, std::true_type{});
        }
    };
    auto store_sel = [&](int buf, uint32_t k0, const f32x4 *ra, const f32x4 *rb, auto flavour_tag, auto which_tag) {
        constexpr int FL = decltype(flavour_tag)::value;
        constexpr int W = decltype(which_tag)::value;
        const bool complete = FL != ANY || k0 < k_inside;
        const bool plain = FL == PLAIN || (FL == ANY && tile_inside && complete);
        if constexpr (W & 1) {
            if (plain || (complete && !fix_a_always))
                sstore(As + buf * SA::SIZE, ra, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{},
                       integral_constant<int, A_V4>{}, std::false_type{});
            else
                sstore(As + buf * SA::SIZE, ra, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{},
                       integral_constant<int, A_V4>{}, std::true_type{});
        }
        if constexpr (W & 2) {
            if (plain || (complete && !fix_b_always))
                sstore(Bs + buf * SB::SIZE, rb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{},
                       integral_constant<int, B_V4>{}, std::false_type{});
            else
                sstore(Bs + buf * SB::SIZE, rb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{},
                       integral_constant<int, B_V4>{}, std::true_type{});
        }
    };
    auto load_ab = [&](uint32_t k0, f32x4 *ra, f32x4 *rb, auto flavour_tag) {
        load_sel(k0, ra, rb, flavour_tag, integral_constant<int, 3>{});
    };
    auto store_ab = [&](int buf, uint32_t k0, const f32x4 *ra, const f32x4 *rb, auto flavour_tag) {
        store_sel(buf, k0, ra, rb, flavour_tag, integral_constant<int, 3>{});
    };
    using AnyFlavour = integral_constant<int, EDGE ? ANY : PLAIN>;

    const uint32_t ktiles = (g.K + BKT - 1) / BKT;
    constexpr int S = BK / 8; // fragment steps per k-slab (8 values of k each)

    // fragments of step s of LDS buffer `buf`: lane holds k = 8*s + 4*lhi + t, t = 0..3
    auto read_frags = [&](int buf, int s, f32x4 *af, f32x4 *bf) {
        const float *as = As + buf * SA::SIZE + (A_K ? (wm * WM + l32) * SA::LD : wm * WM + l32);
        const float *bs = Bs + buf * SB::SIZE + (B_K ? (wn * WN + l32) * SB::LD : wn * WN + l32);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if constexpr (A_K) {
                af[i] = *reinterpret_cast<const f32x4 *>(as + i * 32 * SA::LD + kg * BK + 8 * s + 4 * lhi);
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t) af[i][t] = as[(kg * BK + 8 * s + 4 * lhi + t) * SA::LD + i * 32];
            }
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            if constexpr (B_K) {
                bf[j] = *reinterpret_cast<const f32x4 *>(bs + j * 32 * SB::LD + kg * BK + 8 * s + 4 * lhi);
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t) bf[j][t] = bs[(kg * BK + 8 * s + 4 * lhi + t) * SB::LD + j * 32];
            }
        }
    };

    load_ab(0, ra[0], rb[0], AnyFlavour{});
    store_ab(0, 0, ra[0], rb[0], AnyFlavour{});
    if (PF == 2 && ktiles > 1) load_ab(BKT, ra[PF - 1], rb[PF - 1], AnyFlavour{});
    if (LOOP >= 3 && ktiles > 1) // the operands that are stored early are requested a slab ahead
        load_sel(BKT, ra[0], rb[0], AnyFlavour{}, integral_constant<int, LOOP == 3 ? 3 : LOOP == 4 ? 1 : 2>{});
    __syncthreads();

    // Fragment registers are double-buffered: the LDS reads for step s+1 are issued before the
    // matrix instructions of step s, and the slab hand-over (LDS store of the next slab, barrier,
    // first fragment reload) sits in front of the last step's matrix instructions, so that LDS
    // latency and barrier skew are covered by matrix work of the same wavefront.
    // With one staging set slab kt+1 is requested from global memory at the top of iteration kt
    // (requesting it a whole iteration earlier was measured on the large tiles and changes nothing);
    // with two sets slab kt+2 is requested there and slab kt+1, requested an iteration ago, is the
    // one handed over.
    //
    // The loop exists in four spellings, three of the same schedule and one that stores early.  How two co-resident work-groups
    // interleave on a CU depends on the instruction order the compiler derives from the spelling,
    // and the rate moves by up to 10 % with it; each tile (for 256x128: each operand layout) uses the one that measured fastest on
    // MI355X (same box, same process, f32, alpha and beta given):
    //   LOOP 0  `if (more)` around the hand-over, written out      256x128: NN 143.0, NT 133.7, TN 130.6, TT 131.7
    //   LOOP 1  the same inside a lambda                            256x128: NN 129.3, NT 131.6, TN 128.6
    //   LOOP 2  last slab peeled, hand-over fenced                  256x128: NN 134.7, NT 135.2, TN 133.3, TT 133.0
    //           (sched_barrier) so that matrix instructions
    //           are not hoisted above the barrier
    //   LOOP 3  LOOP 2 with an early store: slab kt+1, requested    256x128: NN 133.6, NT 144.0, TN 128.6, TT 142.3;
    //           a whole iteration ago, goes to the free LDS        the loop of the 128x128 and 64x64 tiles
    //           buffer at the top of iteration kt and slab kt+2
    //           is requested into the same registers
    //   LOOP 4 / 5  LOOP 3 for A only / for B only, the other     256x128: LOOP 4 NN 139.7, NT 143.3, TN 132.6, TT 135.9;
    //           operand stored late as in LOOP 2                    LOOP 5 NN 135.9, NT 143.9, TN 136.1, TT 138.5
    // (8192^3, alpha and beta given, TFLOP/s, one process on one box.)  The ranking is not stable under
    // changes elsewhere in the kernel: one more scalar kernel argument read by every instantiation (a
    // tile-number offset) took N,N under LOOP 0 from 143 to 132.6 while LOOP 4 stayed at 139 -- the offset
    // is therefore read by the split-k instantiations only, and bench.py holds a floor under the headline
    // rate.
    // (the bounds-checked instantiation takes LOOP 2 and up, whose iterations exist per flavour)
    f32x4 af[2][FM], bf[2][FN];
    read_frags(0, 0, af[0], bf[0]);

    auto mfma_step = [&](int s) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[s & 1][i][t], bf[s & 1][j][t], acc[i][j], 0, 0, 0);
    };

    if constexpr (LOOP == 0) {
        for (uint32_t kt = 0; kt < ktiles; ++kt) {
            const int cur = kt & 1;
            const bool more = kt + 1 < ktiles;
            if (more) load_ab((kt + 1) * BKT, ra[0], rb[0], AnyFlavour{});
#pragma unroll
            for (int s = 0; s < S; ++s) {
                if (s + 1 < S) {
                    read_frags(cur, s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
                } else if (more) {
                    store_ab(cur ^ 1, (kt + 1) * BKT, ra[0], rb[0], AnyFlavour{});
                    __syncthreads();
                    read_frags(cur ^ 1, 0, af[(s + 1) & 1], bf[(s + 1) & 1]);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < FM; ++i)
#pragma unroll
                        for (int j = 0; j < FN; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[s & 1][i][t], bf[s & 1][j][t], acc[i][j], 0, 0, 0);
            }
        }
    } else if constexpr (LOOP == 1) {
        auto iteration = [&](uint32_t kt) {
            const int cur = kt & 1;
            const bool more = kt + 1 < ktiles;
            if (more) load_ab((kt + 1) * BKT, ra[0], rb[0], AnyFlavour{});
#pragma unroll
            for (int s = 0; s < S; ++s) {
                if (s + 1 < S) {
                    read_frags(cur, s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
                } else if (more) {
                    store_ab(cur ^ 1, (kt + 1) * BKT, ra[0], rb[0], AnyFlavour{});
                    __syncthreads();
                    read_frags(cur ^ 1, 0, af[(s + 1) & 1], bf[(s + 1) & 1]);
                }
                mfma_step(s);
            }
        };
        for (uint32_t kt = 0; kt < ktiles; ++kt) iteration(kt);
    } else {
        // LOOP 2 and 3: one iteration that hands over to slab kt+1; P = parity of kt, a compile-time
        // constant so that the staging sets stay in registers.  EARLY (LOOP 3): slab kt+1 was requested
        // an iteration ago and goes to the free LDS buffer at the top of iteration kt, slab kt+2 is then
        // requested into the same registers, and only the barrier and the first fragment reads of the
        // next slab sit between the matrix instructions of two slabs.
        constexpr bool EARLY = LOOP >= 3;
        constexpr int EW = LOOP == 3 ? 3 : LOOP == 4 ? 1 : LOOP == 5 ? 2 : 0; // operands stored early (bit 0: A, bit 1: B)
        using Early = integral_constant<int, EW>;
        using Late = integral_constant<int, 3 - EW>;
        constexpr int LEAD = (PF == 2 || EARLY) ? 2 : 1; // iteration kt requests slab kt + LEAD
        auto iteration = [&](uint32_t kt, auto parity_tag, auto flavour_tag) __attribute__((always_inline)) {
            constexpr int P = decltype(parity_tag)::value;
            const int cur = kt & 1;
            if constexpr (EARLY) {
                store_sel(cur ^ 1, (kt + 1) * BKT, ra[0], rb[0], flavour_tag, Early{});
                if (kt + 2 < ktiles) load_sel((kt + 2) * BKT, ra[0], rb[0], flavour_tag, Early{});
                if constexpr (EW != 3) load_sel((kt + 1) * BKT, ra[0], rb[0], flavour_tag, Late{});
            } else if constexpr (PF == 1) {
                load_ab((kt + 1) * BKT, ra[0], rb[0], flavour_tag);
            } else {
                if (kt + 2 < ktiles) load_ab((kt + 2) * BKT, ra[P], rb[P], flavour_tag); // set P held slab kt, already in LDS
            }
            constexpr int NEXT = PF == 1 ? 0 : 1 - P; // the set holding slab kt+1
#pragma unroll
            for (int s = 0; s < S; ++s) {
                if (s + 1 < S) {
                    read_frags(cur, s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
                } else {
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (!EARLY) store_ab(cur ^ 1, (kt + 1) * BKT, ra[NEXT], rb[NEXT], flavour_tag);
                    else if constexpr (EW != 3) store_sel(cur ^ 1, (kt + 1) * BKT, ra[0], rb[0], flavour_tag, Late{});
                    __syncthreads();
                    read_frags(cur ^ 1, 0, af[(s + 1) & 1], bf[(s + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                mfma_step(s);
            }
        };
        // iterations kt .. end-1 in one flavour, two per trip; with two staging sets the set index is
        // the parity of kt
        auto run = [&](uint32_t &kt, uint32_t end, auto flavour_tag) __attribute__((always_inline)) {
            if constexpr (PF == 1 && !EARLY) {
                for (; kt < end; ++kt) iteration(kt, integral_constant<int, 0>{}, flavour_tag);
            } else {
                if ((kt & 1) && kt < end) {
                    iteration(kt, integral_constant<int, 1>{}, flavour_tag);
                    ++kt;
                }
                for (; kt + 1 < end; kt += 2) {
                    iteration(kt, integral_constant<int, 0>{}, flavour_tag);
                    iteration(kt + 1, integral_constant<int, 1>{}, flavour_tag);
                }
                if (kt < end) {
                    iteration(kt, integral_constant<int, 0>{}, flavour_tag);
                    ++kt;
                }
            }
        };
        uint32_t kt = 0;
        if constexpr (!EDGE) {
            if constexpr (PF == 1 && !EARLY) {
                for (; kt + 1 < ktiles; ++kt) iteration(kt, integral_constant<int, 0>{}, AnyFlavour{});
            } else {
                for (; kt + 2 < ktiles; kt += 2) {
                    iteration(kt, integral_constant<int, 0>{}, AnyFlavour{});
                    iteration(kt + 1, integral_constant<int, 1>{}, AnyFlavour{});
                }
                if (kt + 1 < ktiles) {
                    iteration(kt, integral_constant<int, 0>{}, AnyFlavour{});
                    ++kt;
                }
            }
        } else {
            // Iteration kt stores slab kt + 1 and requests slab kt + LEAD: the iterations before
            // `main_end` touch complete slabs only and run in a flavour fixed for the tile.
            const bool has_tail = g.K % BKT != 0;
            const uint32_t hand_overs = ktiles - 1;
            const uint32_t main_end = has_tail ? (hand_overs > (uint32_t)LEAD ? hand_overs - LEAD : 0u) : hand_overs;
            if (tile_inside) run(kt, main_end, integral_constant<int, PLAIN>{});
            else run(kt, main_end, integral_constant<int, CLAMPED>{});
            run(kt, hand_overs, integral_constant<int, ANY>{});
        }
        {   // last slab: nothing to hand over
            const int cur = kt & 1;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                if (s + 1 < S) read_frags(cur, s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
                mfma_step(s);
            }
        }
    }

    if constexpr (KS > 1) {
        // the groups' partial tiles meet in LDS (the slabs are done with): [group - 1][wave][i][j][r][lane]
        static_assert((KS - 1) * BM * BN <= 2 * (SA::SIZE + SB::SIZE), "partial tiles must fit the slab buffers");
        __syncthreads();
        if (kg > 0) {
            float *dst = lds + (size_t)((kg - 1) * WAVES_M * WAVES_N + wave) * FM * FN * 16 * 64 + lane;
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) dst[((i * FN + j) * 16 + r) * 64] = acc[i][j][r];
        }
        __syncthreads();
        if (kg > 0) return;
#pragma unroll
        for (int q = 1; q < KS; ++q) {
            const float *src = lds + (size_t)((q - 1) * WAVES_M * WAVES_N + wave) * FM * FN * 16 * 64 + lane;
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] += src[((i * FN + j) * 16 + r) * 64];
        }
    }

    if constexpr (SPLIT) {
        // The shares' partial tiles meet in memory in accumulator-register order (register q of thread
        // t at q * NT + t: coalesced).  The work-group that arrives last at the tile's counter adds
        // them up, always in the order of the shares and its own read back like the others, so the
        // result does not depend on which one that is; it leaves the counter at zero for the next
        // launch.
        // Work-groups of one tile may sit on different XCDs, behind different L2s.  The partial tiles
        // are therefore written and read with device-scope accesses (relaxed atomics: they go through
        // to the memory side and are read from there), a wavefront waits for its stores to be
        // acknowledged before the barrier in front of the count, and the count itself is a
        // device-scope atomic.  This orders everything that matters without release / acquire fences,
        // which on this part write back and invalidate a whole L2 per work-group (measured: with
        // fences the split launch was no faster than the unsplit one).
        __shared__ uint32_t s_last;
        constexpr size_t TILE = (size_t)BM * BN;
        float *mine = g.partials + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * TILE + tid;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    __hip_atomic_store(mine + (size_t)((i * FN + j) * 16 + r) * NT, acc[i][j][r], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const uint32_t before = __hip_atomic_fetch_add(&g.counters[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t last = before == gridDim.y - 1 ? 1u : 0u;
            if (last) __hip_atomic_store(&g.counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = last;
        }
        __syncthreads();
        if (!s_last) return;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        for (uint32_t z = 0; z < gridDim.y; ++z) {
            const float *part = g.partials + ((size_t)z * gridDim.x + blockIdx.x) * TILE + tid;
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    float v[16]; // one 32x32 block's worth of loads in flight
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        v[r] = __hip_atomic_load(part + (size_t)((i * FN + j) * 16 + r) * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] += v[r];
                }
        }
    }

    // ---- epilogue: acc register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 block.
    // The reads of C_old (beta given) are issued for a whole 32x32 block before any is used; in the
    // bounds-checked instantiation their addresses are clamped into C instead of being skipped, so
    // that they stay one batch of independent loads (a load inside a branch is waited for on the spot).
    const float alpha = g.alpha, beta = g.beta;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const uint32_t col = n0 + wn * WN + j * 32 + l32;
            const uint32_t colc = EDGE ? min(col, g.N - 1) : col;
            float bias_v = 0.f;
            if constexpr (EXT) {
                if (g.bias) bias_v = g.bias[colc];
            }
            float old[16];
            if (g.epi == EPI_ALPHA_BETA) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                    const uint32_t rowc = EDGE ? min(row, g.M - 1) : row;
                    old[r] = g.C[(size_t)rowc * g.ldc + colc];
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                float v = acc[i][j][r];
                if (g.epi == EPI_ALPHA) v = alpha * v;
                else if (g.epi == EPI_ALPHA_BETA) v = alpha * v + beta * old[r];
                if constexpr (EXT) {
                    if (g.bias) v += bias_v;
                    v = act_forward<float>(g.act, v);
                }
                if (!EDGE || ((row < g.M) & (col < g.N))) g.C[(size_t)row * g.ldc + col] = v;
            }
        }
}

// ------------------------------------------------------------------------------------ f64 ---
// Same structure with v_mfma_f64_16x16x4_f64: lane l supplies A[l%16][l/16] and B[l/16][l%16];
// result register r of lane l is C[4*r + l/16][l%16] of the 16x16 block.
// LDS element = double, "vectors" are 2 doubles (16 bytes).

template <int ROWS, int BK, bool KCONTIG> struct SlabD {
    static constexpr int LD = KCONTIG ? BK + 2 : ROWS + 4; // doubles per LDS row
    static constexpr int SIZE = KCONTIG ? ROWS * LD : BK * LD;
};

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int OCC, bool A_K, bool B_K, bool EDGE, bool EXT = false, int KS = 1,
          bool SPLIT = false>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64 * KS) __attribute__((amdgpu_waves_per_eu(OCC)))
void gemm_f64_mfma_kernel(MArgs<double> g) {
    static_assert(!SPLIT || KS == 1, "k is split over work-groups or inside one, not both");
    constexpr int NT = WAVES_M * WAVES_N * 64 * KS; // KS groups of wavefronts split each slab, as in the f32 kernel
    constexpr int BKT = BK * KS;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int FM = WM / 16, FN = WN / 16;
    static_assert(WM % 16 == 0 && WN % 16 == 0 && BK % 8 == 0, "tile shape");
    using SA = SlabD<BM, BKT, A_K>;
    using SB = SlabD<BN, BKT, B_K>;
    constexpr int A_V2 = BM * BKT / 2 / NT, B_V2 = BN * BKT / 2 / NT;
    static_assert(A_V2 * NT * 2 == BM * BKT && B_V2 * NT * 2 == BN * BKT, "slab must divide over the threads");

    extern __shared__ __align__(16) float lds[];
    double *As = reinterpret_cast<double *>(lds);
    double *Bs = As + 2 * SA::SIZE;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = (tid >> 6) % (WAVES_M * WAVES_N), kg = (tid >> 6) / (WAVES_M * WAVES_N);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l16 = lane & 15, lq = lane >> 4; // lq = 0..3

    uint32_t tile_m, tile_n;
    tile_coords(g.tiles_m, g.tiles_n, tile_m, tile_n, g.xcd_remap, SPLIT ? g.pid_offset : 0u); // only a split tail starts past tile 0
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    if constexpr (SPLIT) { // this work-group's share of k, as in the f32 kernel
        const uint32_t k_begin = blockIdx.y * g.klen;
        const uint32_t k_end = min(g.K, k_begin + g.klen);
        g.A += A_K ? (size_t)k_begin : (size_t)k_begin * g.lda;
        g.B += B_K ? (size_t)k_begin : (size_t)k_begin * g.ldb;
        g.K = k_end - k_begin;
    }
    // one solo iteration = FM*FN*BK/4 matrix instructions of 64 clocks = FM*FN*BK/8 sleep units

    f64x4 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0;

    // two staging sets for the small tile, as in the f32 kernel
    constexpr int PF = (BM * BN <= 64 * 64) ? 2 : 1;
    f64x2 ra[PF][A_V2], rb[PF][B_V2];

    auto gload = [&](f64x2 *dst, const double *__restrict__ base, uint32_t ld, uint32_t row0, uint32_t row_lim,
                     uint32_t k0, auto kc_tag, auto rows_tag, auto nv_tag, auto check_tag) {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        constexpr int NV = decltype(nv_tag)::value;
        constexpr bool CHECK = decltype(check_tag)::value;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int q = tid + i * NT;
            uint32_t r, c, r_lim, c_lim;
            if constexpr (KC) {
                r = row0 + q / (BKT / 2); c = k0 + 2 * (q % (BKT / 2));
                r_lim = row_lim; c_lim = g.K;
            } else {
                r = k0 + q / (ROWS / 2); c = row0 + 2 * (q % (ROWS / 2));
                r_lim = g.K; c_lim = row_lim;
            }
            const double *p = base + (size_t)r * ld + c;
            if constexpr (!EDGE) {
                dst[i] = *reinterpret_cast<const f64x2 *>(p);
            } else if constexpr (!CHECK) {
                dst[i] = reinterpret_cast<const f64x2_u *>(p)->v;
            } else {
                // clamped raw load; the fixup happens at the LDS store, as in the f32 kernel
                const uint32_t rr = r < r_lim ? r : r_lim - 1;
                const uint32_t cc = c + 2 <= c_lim ? c : (c_lim >= 2 ? c_lim - 2 : 0);
                const double *q = base + (size_t)rr * ld + cc;
                f64x2 v;
                if (c_lim >= 2) {
                    v = reinterpret_cast<const f64x2_u *>(q)->v;
                } else {
                    v[0] = q[0];
                    v[1] = 0.0;
                }
                dst[i] = v;
            }
        }
    };
    auto sstore = [&](double *slab, const f64x2 *src, uint32_t row0, uint32_t row_lim, uint32_t k0, auto kc_tag, auto rows_tag,
                      auto nv_tag, auto fix_tag) {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        constexpr int NV = decltype(nv_tag)::value;
        constexpr bool FIX = decltype(fix_tag)::value;
        constexpr int LD = SlabD<ROWS, BKT, KC>::LD;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int q = tid + i * NT;
            int off;
            if constexpr (KC) off = (q / (BKT / 2)) * LD + 2 * (q % (BKT / 2));
            else off = (q / (ROWS / 2)) * LD + 2 * (q % (ROWS / 2));
            f64x2 v = src[i];
            if constexpr (FIX) {
                asm volatile("" ::: "memory"); // as in the f32 kernel: keep this a branch, not selects
                uint32_t r, c, r_lim, c_lim;
                if constexpr (KC) {
                    r = row0 + q / (BKT / 2); c = k0 + 2 * (q % (BKT / 2));
                    r_lim = row_lim; c_lim = g.K;
                } else {
                    r = k0 + q / (ROWS / 2); c = row0 + 2 * (q % (ROWS / 2));
                    r_lim = g.K; c_lim = row_lim;
                }
                const uint32_t cc = c + 2 <= c_lim ? c : (c_lim >= 2 ? c_lim - 2 : 0);
                const uint32_t shift = c - cc;
                const f64x2 t = v;
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const double x = shift + e == 0 ? t[0] : t[1];
                    const bool ok = (r < r_lim) & (c + e < c_lim);
                    v[e] = ok ? x : 0.0;
                }
            }
            *reinterpret_cast<f64x2 *>(slab + off) = v;
        }
    };

    using std::integral_constant;
    // interior tiles of the bounds-checked instantiation check only the slab with the k tail
    const bool tile_inside = !EDGE || (m0 + BM <= g.M && n0 + BN <= g.N);
    const uint32_t k_inside = g.K - g.K % BKT;
    // slab flavours as in the f32 kernel: PLAIN inside both operands, CLAMPED for complete slabs of an
    // edge tile (stored as loaded unless a 2-element vector straddles a row end), ANY decided per slab
    const bool fix_a_always = !A_K && g.M % 2 != 0, fix_b_always = !B_K && g.N % 2 != 0;
    enum { PLAIN = 0, CLAMPED = 1, ANY = 2 };
    auto load_ab = [&](uint32_t k0, f64x2 *ra, f64x2 *rb, auto flavour_tag) {
        constexpr int FL = decltype(flavour_tag)::value;
        if (FL == PLAIN || (FL == ANY && tile_inside && k0 < k_inside)) {
            gload(ra, g.A, g.lda, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{},
                  integral_constant<int, A_V2>{}, std::false_type{});
            gload(rb, g.B, g.ldb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{},
                  integral_constant<int, B_V2>{}, std::false_type{});
        } else {
            gload(ra, g.A, g.lda, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{},
                  integral_constant<int, A_V2>{}, std::true_type{});
            gload(rb, g.B, g.ldb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{},
                  integral_constant<int, B_V2>{}, std::true_type{});
        }
    };
    auto store_ab = [&](int buf, uint32_t k0, const f64x2 *ra, const f64x2 *rb, auto flavour_tag) {
        constexpr int FL = decltype(flavour_tag)::value;
        const bool complete = FL != ANY || k0 < k_inside;
        const bool plain = FL == PLAIN || (FL == ANY && tile_inside && complete);
        if (plain || (complete && !fix_a_always))
            sstore(As + buf * SA::SIZE, ra, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{},
                   integral_constant<int, A_V2>{}, std::false_type{});
        else
            sstore(As + buf * SA::SIZE, ra, m0, g.M, k0, integral_constant<bool, A_K>{}, integral_constant<int, BM>{},
                   integral_constant<int, A_V2>{}, std::true_type{});
        if (plain || (complete && !fix_b_always))
            sstore(Bs + buf * SB::SIZE, rb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{},
                   integral_constant<int, B_V2>{}, std::false_type{});
        else
            sstore(Bs + buf * SB::SIZE, rb, n0, g.N, k0, integral_constant<bool, B_K>{}, integral_constant<int, BN>{},
                   integral_constant<int, B_V2>{}, std::true_type{});
    };
    using AnyFlavour = integral_constant<int, EDGE ? ANY : PLAIN>;

    const uint32_t ktiles = (g.K + BKT - 1) / BKT;
    constexpr int S = BK / 8;

    // fragments of step s: lane holds k = 8*s + 2*lq + t, t = 0..1 (two instructions per 8 k)
    auto read_frags = [&](int buf, int s, f64x2 *af, f64x2 *bf) {
        const double *as = As + buf * SA::SIZE + (A_K ? (wm * WM + l16) * SA::LD : wm * WM + l16);
        const double *bs = Bs + buf * SB::SIZE + (B_K ? (wn * WN + l16) * SB::LD : wn * WN + l16);
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if constexpr (A_K) {
                af[i] = *reinterpret_cast<const f64x2 *>(as + i * 16 * SA::LD + kg * BK + 8 * s + 2 * lq);
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t) af[i][t] = as[(kg * BK + 8 * s + 2 * lq + t) * SA::LD + i * 16];
            }
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            if constexpr (B_K) {
                bf[j] = *reinterpret_cast<const f64x2 *>(bs + j * 16 * SB::LD + kg * BK + 8 * s + 2 * lq);
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t) bf[j][t] = bs[(kg * BK + 8 * s + 2 * lq + t) * SB::LD + j * 16];
            }
        }
    };

    load_ab(0, ra[0], rb[0], AnyFlavour{});
    store_ab(0, 0, ra[0], rb[0], AnyFlavour{});
    if (PF == 2 && ktiles > 1) load_ab(BKT, ra[PF - 1], rb[PF - 1], AnyFlavour{});
    __syncthreads();

    // Same schedule as the f32 kernel: double-buffered fragments, hand-over in front of the last
    // step's matrix instructions.  The large tiles request slab kt+1 at the top of iteration kt
    // around an `if (more)`; the small tile requests slab kt+2 there (two staging sets), runs its
    // last slab after the loop and fences the hand-over against reordering.
    f64x2 af[2][FM], bf[2][FN];
    read_frags(0, 0, af[0], bf[0]);

    auto mfma_step = [&](int s) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[s & 1][i][t], bf[s & 1][j][t], acc[i][j], 0, 0, 0);
    };

    if constexpr (PF == 1 && !EDGE) {
        for (uint32_t kt = 0; kt < ktiles; ++kt) {
            const int cur = kt & 1;
            const bool more = kt + 1 < ktiles;
            if (more) load_ab((kt + 1) * BKT, ra[0], rb[0], AnyFlavour{});
#pragma unroll
            for (int s = 0; s < S; ++s) {
                if (s + 1 < S) {
                    read_frags(cur, s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
                } else if (more) {
                    store_ab(cur ^ 1, (kt + 1) * BKT, ra[0], rb[0], AnyFlavour{});
                    __syncthreads();
                    read_frags(cur ^ 1, 0, af[(s + 1) & 1], bf[(s + 1) & 1]);
                }
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int i = 0; i < FM; ++i)
#pragma unroll
                        for (int j = 0; j < FN; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[s & 1][i][t], bf[s & 1][j][t], acc[i][j], 0, 0, 0);
            }
        }
    } else {
        // (the bounds-checked instantiation of every tile takes this loop, whose iterations exist per flavour)
        auto iteration = [&](uint32_t kt, auto parity_tag, auto flavour_tag) __attribute__((always_inline)) {
            constexpr int P = decltype(parity_tag)::value;
            const int cur = kt & 1;
            if constexpr (PF == 1) {
                load_ab((kt + 1) * BKT, ra[0], rb[0], flavour_tag);
            } else {
                if (kt + 2 < ktiles) load_ab((kt + 2) * BKT, ra[P], rb[P], flavour_tag);
            }
            constexpr int NEXT = PF == 1 ? 0 : 1 - P;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                if (s + 1 < S) {
                    read_frags(cur, s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
                } else {
                    __builtin_amdgcn_sched_barrier(0);
                    store_ab(cur ^ 1, (kt + 1) * BKT, ra[NEXT], rb[NEXT], flavour_tag);
                    __syncthreads();
                    read_frags(cur ^ 1, 0, af[(s + 1) & 1], bf[(s + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                mfma_step(s);
            }
        };
        auto run = [&](uint32_t &kt, uint32_t end, auto flavour_tag) __attribute__((always_inline)) {
            if constexpr (PF == 1) {
                for (; kt < end; ++kt) iteration(kt, integral_constant<int, 0>{}, flavour_tag);
            } else {
                if ((kt & 1) && kt < end) {
                    iteration(kt, integral_constant<int, 1>{}, flavour_tag);
                    ++kt;
                }
                for (; kt + 1 < end; kt += 2) {
                    iteration(kt, integral_constant<int, 0>{}, flavour_tag);
                    iteration(kt + 1, integral_constant<int, 1>{}, flavour_tag);
                }
                if (kt < end) {
                    iteration(kt, integral_constant<int, 0>{}, flavour_tag);
                    ++kt;
                }
            }
        };
        uint32_t kt = 0;
        if constexpr (!EDGE) {
            for (; kt + 2 < ktiles; kt += 2) {
                iteration(kt, integral_constant<int, 0>{}, AnyFlavour{});
                iteration(kt + 1, integral_constant<int, 1>{}, AnyFlavour{});
            }
            if (kt + 1 < ktiles) {
                iteration(kt, integral_constant<int, 0>{}, AnyFlavour{});
                ++kt;
            }
        } else {
            const bool has_tail = g.K % BKT != 0;
            const uint32_t hand_overs = ktiles - 1;
            const uint32_t main_end = has_tail ? (hand_overs > (uint32_t)PF ? hand_overs - PF : 0u) : hand_overs;
            if (tile_inside) run(kt, main_end, integral_constant<int, PLAIN>{});
            else run(kt, main_end, integral_constant<int, CLAMPED>{});
            run(kt, hand_overs, integral_constant<int, ANY>{});
        }
        const int cur = kt & 1; // last slab: nothing to hand over
#pragma unroll
        for (int s = 0; s < S; ++s) {
            if (s + 1 < S) read_frags(cur, s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
            mfma_step(s);
        }
    }

    if constexpr (KS > 1) {
        // partial tiles of the groups through LDS: [group - 1][wave][i][j][r][lane]
        static_assert((KS - 1) * BM * BN <= 2 * (SA::SIZE + SB::SIZE), "partial tiles must fit the slab buffers");
        double *red = reinterpret_cast<double *>(lds);
        __syncthreads();
        if (kg > 0) {
            double *dst = red + (size_t)((kg - 1) * WAVES_M * WAVES_N + wave) * FM * FN * 4 * 64 + lane;
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r) dst[((i * FN + j) * 4 + r) * 64] = acc[i][j][r];
        }
        __syncthreads();
        if (kg > 0) return;
#pragma unroll
        for (int q = 1; q < KS; ++q) {
            const double *src = red + (size_t)((q - 1) * WAVES_M * WAVES_N + wave) * FM * FN * 4 * 64 + lane;
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[i][j][r] += src[((i * FN + j) * 4 + r) * 64];
        }
    }

    if constexpr (SPLIT) {
        // partial tiles of the shares through memory, added by the last arrival in the order of the
        // shares; device-scope accesses and a wait for the stores instead of fences (see the f32 kernel)
        __shared__ uint32_t s_last;
        constexpr int Q = FM * FN * 4;
        constexpr size_t TILE = (size_t)BM * BN;
        double *mine = g.partials + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * TILE + tid;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    __hip_atomic_store(mine + (size_t)((i * FN + j) * 4 + r) * NT, acc[i][j][r], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) {
            const uint32_t before = __hip_atomic_fetch_add(&g.counters[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t last = before == gridDim.y - 1 ? 1u : 0u;
            if (last) __hip_atomic_store(&g.counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_last = last;
        }
        __syncthreads();
        if (!s_last) return;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0;
        for (uint32_t z = 0; z < gridDim.y; ++z) {
            const double *part = g.partials + ((size_t)z * gridDim.x + blockIdx.x) * TILE + tid;
            double v[Q];
#pragma unroll
            for (int q = 0; q < Q; ++q) v[q] = __hip_atomic_load(part + (size_t)q * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[i][j][r] += v[(i * FN + j) * 4 + r];
        }
    }

    const double alpha = g.alpha, beta = g.beta;
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const uint32_t col = n0 + wn * WN + j * 16 + l16;
            const uint32_t colc = EDGE ? min(col, g.N - 1) : col;
            double bias_v = 0.;
            if constexpr (EXT) {
                if (g.bias) bias_v = g.bias[colc];
            }
            double old[4];
            if (g.epi == EPI_ALPHA_BETA) { // batched, clamped reads of C_old (see the f32 kernel)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t row = m0 + wm * WM + i * 16 + 4 * r + lq;
                    const uint32_t rowc = EDGE ? min(row, g.M - 1) : row;
                    old[r] = g.C[(size_t)rowc * g.ldc + colc];
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t row = m0 + wm * WM + i * 16 + 4 * r + lq;
                double v = acc[i][j][r];
                if (g.epi == EPI_ALPHA) v = alpha * v;
                else if (g.epi == EPI_ALPHA_BETA) v = alpha * v + beta * old[r];
                if constexpr (EXT) {
                    if (g.bias) v += bias_v;
                    v = act_forward<double>(g.act, v);
                }
                if (!EDGE || ((row < g.M) & (col < g.N))) g.C[(size_t)row * g.ldc + col] = v;
            }
        }
}

// ------------------------------------------------------------------------------ dispatch ---

template <typename T> MArgs<T> make_args(const GemmProblem &p, int bm, int bn) {
    MArgs<T> g{}; // every field starts at zero / null; a split launch fills klen, partials and counters itself
    g.A = static_cast<const T *>(p.A);
    g.B = static_cast<const T *>(p.B);
    g.C = static_cast<T *>(p.C);
    g.M = (uint32_t)p.M; g.N = (uint32_t)p.N; g.K = (uint32_t)p.K;
    g.lda = (uint32_t)p.lda; g.ldb = (uint32_t)p.ldb; g.ldc = (uint32_t)p.ldc;
    g.tiles_m = (uint32_t)((p.M + bm - 1) / bm);
    g.tiles_n = (uint32_t)((p.N + bn - 1) / bn);
    // Small launches (every tile resident at once) run out of the per-XCD L2: give each XCD a
    // compact run of tiles.  Large launches stream from the shared Infinity Cache: keep the XCDs on
    // the same B panel (see tile_coords).  Measured: 1024^3 f32 48 -> 62 TFLOP/s with the
    // renumbering, 8192^3 138 -> 131 with it.
    g.xcd_remap = (uint64_t)g.tiles_m * g.tiles_n <= 4ull * (p.num_cus ? p.num_cus : 256u) ? 1u : 0u;
    g.epi = p.epi;
    std::memcpy(&g.alpha, p.alpha, sizeof(T));
    std::memcpy(&g.beta, p.beta, sizeof(T));
    g.bias = static_cast<const T *>(p.ext_bias);
    g.act = p.ext_act;
    return g;
}

template <typename K> int set_lds(K kernel, size_t bytes) {
    if (bytes > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) { (void)hipGetLastError(); return hip_code(e); }
    }
    return WK_OK;
}

// Fills the split-k fields of the kernel arguments from a plan and checks, on the host, everything the
// kernel takes for granted: memory for the partial tiles and a counter for every tile.
template <typename T> int apply_split(MArgs<T> &g, const GemmProblem &p, const GemmSplitPlan &plan, int bm, int bn) {
    if (plan.shares < 2 || plan.klen == 0) return WK_E_INVALID_VALUE;
    if (!p.scratch || !p.counters) return WK_E_INVALID_VALUE;
    // the launch covers tiles first_tile .. first_tile + tiles - 1 of C
    if (plan.tiles == 0 || plan.first_tile + plan.tiles != (uint64_t)g.tiles_m * g.tiles_n || plan.tiles > p.num_counters)
        return WK_E_INVALID_VALUE;
    if ((uint64_t)plan.shares * plan.tiles * bm * bn * sizeof(T) > p.scratch_bytes) return WK_E_INVALID_VALUE;
    if ((uint64_t)plan.klen * (plan.shares - 1) >= p.K || (uint64_t)plan.klen * plan.shares < p.K) return WK_E_INVALID_VALUE;
    if (plan.shares > 65535) return WK_E_INVALID_VALUE;
    g.klen = plan.klen;
    g.partials = static_cast<T *>(p.scratch);
    g.counters = p.counters;
    g.pid_offset = (uint32_t)plan.first_tile;
    g.xcd_remap = 0; // blockIdx.x is the tile's counter index and its place among the partial tiles
    return WK_OK;
}

template <int BM, int BN, int BK, int WMS, int WNS, int OCC, bool AK, bool BKC, bool EDGE, bool EXT = false, int KS = 1, int LSEL = -1,
          bool SPLIT = false>
int launch_f32_one(hipStream_t st, const GemmProblem &p, const GemmSplitPlan *plan = nullptr) {
    constexpr size_t lds = 2 * (Slab<BM, BK * KS, AK>::SIZE + Slab<BN, BK * KS, BKC>::SIZE) * sizeof(float);
    auto kern = gemm_f32_mfma_kernel<BM, BN, BK, WMS, WNS, OCC, AK, BKC, EDGE, EXT, KS, LSEL, SPLIT>;
    static int attr_rc = set_lds(kern, lds);
    if (attr_rc) return attr_rc;
    MArgs<float> g = make_args<float>(p, BM, BN);
    unsigned shares = 1;
    if constexpr (SPLIT) {
        if (!plan) return WK_E_INVALID_VALUE;
        const int rc = apply_split(g, p, *plan, BM, BN);
        if (rc) return rc;
        shares = plan->shares;
    }
    uint32_t grid_x = g.tiles_m * g.tiles_n;
    if constexpr (SPLIT) grid_x = (uint32_t)plan->tiles;
    else if (plan) { // the body of a product whose tail is launched separately: the first tiles only
        if (plan->first_tile == 0 || plan->first_tile >= grid_x) return WK_E_INVALID_VALUE;
        grid_x = (uint32_t)plan->first_tile;
        g.xcd_remap = 0;
    }
    hipLaunchKernelGGL(kern, dim3(grid_x, shares), dim3(WMS * WNS * 64 * KS), lds, st, g);
    return launch_status();
}

// BK: k values one group of wavefronts multiplies per slab; KS groups share a slab of BK * KS
template <int BM, int BN, int BK, int WMS, int WNS, int OCC, int KS = 1, int LSEL = -1>
int launch_f32(hipStream_t st, const GemmProblem &p, bool edge) {
    const int sel = (p.op_a ? 0 : 2) | (p.op_b ? 1 : 0); // bit1: A k-contiguous, bit0: B k-contiguous
    if (p.ext) { // fused bias + activation: instantiated for op N, T only (see gemm_mfma_fuses)
        if (sel != 3) return WK_E_INVALID_VALUE;
        return edge ? launch_f32_one<BM, BN, BK, WMS, WNS, OCC, true, true, true, true, KS, LSEL>(st, p)
                    : launch_f32_one<BM, BN, BK, WMS, WNS, OCC, true, true, false, true, KS, LSEL>(st, p);
    }
#define WK_CASE(AK, BKC)                                                                                   \
    return edge ? launch_f32_one<BM, BN, BK, WMS, WNS, OCC, AK, BKC, true, false, KS, LSEL>(st, p)                          \
                : launch_f32_one<BM, BN, BK, WMS, WNS, OCC, AK, BKC, false, false, KS, LSEL>(st, p)
    switch (sel) {
    case 0: WK_CASE(false, false);
    case 1: WK_CASE(false, true);
    case 2: WK_CASE(true, false);
    default: WK_CASE(true, true);
    }
#undef WK_CASE
}

template <int BM, int BN, int BK, int WMS, int WNS, int OCC, bool AK, bool BKC, bool EDGE, bool EXT = false, int KS = 1,
          bool SPLIT = false>
int launch_f64_one(hipStream_t st, const GemmProblem &p, const GemmSplitPlan *plan = nullptr) {
    constexpr size_t lds = 2 * (SlabD<BM, BK * KS, AK>::SIZE + SlabD<BN, BK * KS, BKC>::SIZE) * sizeof(double);
    auto kern = gemm_f64_mfma_kernel<BM, BN, BK, WMS, WNS, OCC, AK, BKC, EDGE, EXT, KS, SPLIT>;
    static int attr_rc = set_lds(kern, lds);
    if (attr_rc) return attr_rc;
    MArgs<double> g = make_args<double>(p, BM, BN);
    unsigned shares = 1;
    if constexpr (SPLIT) {
        if (!plan) return WK_E_INVALID_VALUE;
        const int rc = apply_split(g, p, *plan, BM, BN);
        if (rc) return rc;
        shares = plan->shares;
    }
    uint32_t grid_x = g.tiles_m * g.tiles_n;
    if constexpr (SPLIT) grid_x = (uint32_t)plan->tiles;
    else if (plan) {
        if (plan->first_tile == 0 || plan->first_tile >= grid_x) return WK_E_INVALID_VALUE;
        grid_x = (uint32_t)plan->first_tile;
        g.xcd_remap = 0;
    }
    hipLaunchKernelGGL(kern, dim3(grid_x, shares), dim3(WMS * WNS * 64 * KS), lds, st, g);
    return launch_status();
}

template <int BM, int BN, int BK, int WMS, int WNS, int OCC, int KS = 1>
int launch_f64(hipStream_t st, const GemmProblem &p, bool edge) {
    const int sel = (p.op_a ? 0 : 2) | (p.op_b ? 1 : 0);
    if (p.ext) {
        if (sel != 3) return WK_E_INVALID_VALUE;
        return edge ? launch_f64_one<BM, BN, BK, WMS, WNS, OCC, true, true, true, true, KS>(st, p)
                    : launch_f64_one<BM, BN, BK, WMS, WNS, OCC, true, true, false, true, KS>(st, p);
    }
#define WK_CASE(AK, BKC)                                                                                   \
    return edge ? launch_f64_one<BM, BN, BK, WMS, WNS, OCC, AK, BKC, true, false, KS>(st, p)                               \
                : launch_f64_one<BM, BN, BK, WMS, WNS, OCC, AK, BKC, false, false, KS>(st, p)
    switch (sel) {
    case 0: WK_CASE(false, false);
    case 1: WK_CASE(false, true);
    case 2: WK_CASE(true, false);
    default: WK_CASE(true, true);
    }
#undef WK_CASE
}

// ---- k split over work-groups ------------------------------------------------------------------
// A product with few tiles of C and a long k leaves most compute units without work (512 x 512 x 8192
// is 64 tiles of 64 x 64 on 256 units).  These variants give every tile to `shares` work-groups, each
// summing a contiguous range of k; the partial tiles meet in the stream's scratch memory and the
// work-group that arrives last at the tile's counter adds them in the order of the shares, so the
// result is the same bits on every run.
//   The plan: only when the tiles leave at least half the compute units idle, as many shares as put
//   four (f64: two) work-groups on every unit (a power of two, at most 64), each share at least eight
//   slabs long.  Where that gives none, a forced variant (tests) falls back to the relaxed plan: split
//   whenever k holds two slabs, up to four shares.  (Launches used to take the relaxed plan always:
//   512 x 512 x 8192 52 -> 47 us, 256 x 256 x 8192 51 -> 31, 128 x 128 x 16384 94 -> 38, f64 256 x 256 x 8192 89 -> 50.)
bool plan_split(const GemmProblem &p, int bm, int bn, int bkt, size_t elem, bool relaxed, GemmSplitPlan &plan) {
    plan = GemmSplitPlan{};
    plan.tiles = ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn);
    const uint64_t slabs = (p.K + bkt - 1) / bkt;
    uint64_t shares = 1;
    if (relaxed) {
        shares = slabs >= 4 ? 4 : slabs;
    } else {
        // up to `occ` work-groups per compute unit (what the tile's registers and LDS allow): co-resident
        // work-groups are what hides the slab hand-overs of one another
        const uint64_t cus = p.num_cus ? p.num_cus : 256;
        const uint64_t occ = elem == 8 ? 2 : 4;
        if (plan.tiles * 2 > cus) return false;
        while (shares < 64 && plan.tiles * shares * 2 <= cus * occ && slabs / (shares * 2) >= 8) shares *= 2;
    }
    if (shares < 2) return false;
    const uint64_t klen = (slabs + shares - 1) / shares * bkt; // whole slabs per share
    shares = (p.K + klen - 1) / klen;                           // the last share may have vanished
    if (shares < 2) return false;
    plan.shares = (uint32_t)shares;
    plan.klen = (uint32_t)klen;
    plan.bytes = (size_t)(shares * plan.tiles * bm * bn * elem);
    return p.scratch && p.counters && plan.bytes <= p.scratch_bytes && plan.tiles <= p.num_counters;
}

// The 64 x 64 tiles with k split over work-groups; without a feasible plan (short k, no scratch, the
// fused epilogue) the plain tile runs.
int launch_f32_split64(hipStream_t st, const GemmProblem &p, bool edge) {
    constexpr int BM = 64, BN = 64, BK = 32;
    GemmSplitPlan plan;
    // the plan of the automatic choice where it exists (as many shares as fill the units), else the forced variant's
    if (p.ext || !(plan_split(p, BM, BN, BK, sizeof(float), false, plan) || plan_split(p, BM, BN, BK, sizeof(float), true, plan)))
        return launch_f32<BM, BN, BK, 2, 2, 4>(st, p, edge);
    const int sel = (p.op_a ? 0 : 2) | (p.op_b ? 1 : 0);
#define WK_CASE(AK, BKC)                                                                                                \
    return edge ? launch_f32_one<BM, BN, BK, 2, 2, 4, AK, BKC, true, false, 1, -1, true>(st, p, &plan)                    \
                : launch_f32_one<BM, BN, BK, 2, 2, 4, AK, BKC, false, false, 1, -1, true>(st, p, &plan)
    switch (sel) {
    case 0: WK_CASE(false, false);
    case 1: WK_CASE(false, true);
    case 2: WK_CASE(true, false);
    default: WK_CASE(true, true);
    }
#undef WK_CASE
}

int launch_f64_split64(hipStream_t st, const GemmProblem &p, bool edge) {
    constexpr int BM = 64, BN = 64, BK = 32;
    GemmSplitPlan plan;
    if (p.ext || !(plan_split(p, BM, BN, BK, sizeof(double), false, plan) || plan_split(p, BM, BN, BK, sizeof(double), true, plan)))
        return launch_f64<BM, BN, BK, 2, 2, 2>(st, p, edge);
    const int sel = (p.op_a ? 0 : 2) | (p.op_b ? 1 : 0);
#define WK_CASE(AK, BKC)                                                                                                \
    return edge ? launch_f64_one<BM, BN, BK, 2, 2, 2, AK, BKC, true, false, 1, true>(st, p, &plan)                        \
                : launch_f64_one<BM, BN, BK, 2, 2, 2, AK, BKC, false, false, 1, true>(st, p, &plan)
    switch (sel) {
    case 0: WK_CASE(false, false);
    case 1: WK_CASE(false, true);
    case 2: WK_CASE(true, false);
    default: WK_CASE(true, true);
    }
#undef WK_CASE
}

// forced tail variants plan relaxed (tests reach the tail path on small shapes); the test option
// "tail_strict" makes them plan like the automatic choice (benchmarks of the choice itself)
inline bool tail_relaxed() { return g_test_options.tail_strict == 0; }

// ---- a tail of tiles with k split --------------------------------------------------------------
// A launch whose tiles do not fill whole rounds ends with a few compute units finishing the
// left-over tiles while the rest idle (4097 x 4095 is 544 tiles of 256 x 128 on 256 units: two
// rounds and 32 tiles more, which take as long as a third round).  These variants launch the whole
// rounds as they are and the left-over tiles as a second launch with k split over work-groups, so
// that the tail occupies every unit for a fraction of a tile's time.
//   relaxed (forced variant, tests): every left-over tile is a tail tile, up to four shares; a product
//   of less than one round is all tail.
//   otherwise: at least one whole round in the body, a tail of at most half a round, as many shares
//   as fill the units once (a power of two, at most 64), each at least eight slabs long.
bool plan_tail(const GemmProblem &p, int bm, int bn, int bkt, size_t elem, int occ, bool relaxed, GemmSplitPlan &plan) {
    plan = GemmSplitPlan{};
    const uint64_t tiles = ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn);
    // a round = as many tiles as are resident at once: `occ` work-groups on every compute unit
    const uint64_t round = (p.num_cus ? p.num_cus : 256) * (uint64_t)(occ > 0 ? occ : 1);
    const uint64_t rem = tiles % round, body = tiles - rem;
    const uint64_t slabs = (p.K + bkt - 1) / bkt;
    if (rem == 0) return false;
    uint64_t shares = 1;
    if (relaxed) {
        shares = slabs >= 4 ? 4 : slabs;
    } else {
        if (body == 0) return false;
        while (shares < 64 && rem * shares * 2 <= round && slabs / (shares * 2) >= 8) shares *= 2;
    }
    if (shares < 2) return false;
    const uint64_t klen = (slabs + shares - 1) / shares * bkt;
    shares = (p.K + klen - 1) / klen;
    if (shares < 2) return false;
    plan.shares = (uint32_t)shares;
    plan.klen = (uint32_t)klen;
    plan.tiles = rem;
    plan.first_tile = body;
    plan.bytes = (size_t)(shares * rem * bm * bn * elem);
    return p.scratch && p.counters && plan.bytes <= p.scratch_bytes && plan.tiles <= p.num_counters;
}

template <int BM, int BN, int BK, int WMS, int WNS, int OCC>
int launch_f32_tail(hipStream_t st, const GemmProblem &p, bool edge) {
    GemmSplitPlan plan;
    if (p.ext || !plan_tail(p, BM, BN, BK, sizeof(float), OCC, tail_relaxed(), plan)) return launch_f32<BM, BN, BK, WMS, WNS, OCC>(st, p, edge);
    const int sel = (p.op_a ? 0 : 2) | (p.op_b ? 1 : 0);
    int rc = WK_OK;
    if (plan.first_tile > 0 && gemm_f32_dma_applies(p, BM, BN)) {
        rc = gemm_f32_dma_launch(st, p, BM, BN, plan.first_tile); // the whole rounds on the direct-to-LDS kernel
        if (rc) return rc;
    } else if (plan.first_tile > 0) { // the whole rounds, as the plain variant would run them
#define WK_CASE(AK, BKC)                                                                                                \
    rc = edge ? launch_f32_one<BM, BN, BK, WMS, WNS, OCC, AK, BKC, true>(st, p, &plan)                                   \
              : launch_f32_one<BM, BN, BK, WMS, WNS, OCC, AK, BKC, false>(st, p, &plan);                                 \
    break
        switch (sel) {
        case 0: WK_CASE(false, false);
        case 1: WK_CASE(false, true);
        case 2: WK_CASE(true, false);
        default: WK_CASE(true, true);
        }
#undef WK_CASE
        if (rc) return rc;
    }
#define WK_CASE(AK, BKC)                                                                                                \
    return edge ? launch_f32_one<BM, BN, BK, WMS, WNS, OCC, AK, BKC, true, false, 1, -1, true>(st, p, &plan)              \
                : launch_f32_one<BM, BN, BK, WMS, WNS, OCC, AK, BKC, false, false, 1, -1, true>(st, p, &plan)
    switch (sel) {
    case 0: WK_CASE(false, false);
    case 1: WK_CASE(false, true);
    case 2: WK_CASE(true, false);
    default: WK_CASE(true, true);
    }
#undef WK_CASE
}

// the direct-to-LDS kernels where they apply, the register-staged tile of the same size elsewhere
template <int BM, int BN, int BK, int OCC> int launch_f32_dma(hipStream_t st, const GemmProblem &p, bool edge) {
    if (gemm_f32_dma_applies(p, BM, BN)) return gemm_f32_dma_launch(st, p, BM, BN); // (checks everything it needs itself)
    return launch_f32<BM, BN, BK, 2, 2, OCC>(st, p, edge);
}

// two groups of wavefronts per tile on the direct-to-LDS kernel; elsewhere the k-split twin of the staged tile
template <int BM, int BN> int launch_f32_dma2(hipStream_t st, const GemmProblem &p, bool edge) {
    if (!p.ext && gemm_f32_dma_applies(p, BM, BN)) return gemm_f32_dma_launch(st, p, BM, BN, 0, 2);
    if (BM == 128) return launch_f32<128, 128, 16, 2, 2, 2, 2>(st, p, edge);
    return launch_f32<64, 64, 16, 2, 2, 4, 4>(st, p, edge);
}

// the direct-to-LDS kernel with its left-over tiles dealt by k-slabs (see gemm_f32_dma_kernel); where that does not
// apply, by tiles
template <int BM, int BN, int OCC> int launch_f32_stream_k(hipStream_t st, const GemmProblem &p, bool edge) {
    if (gemm_f32_dma_stream_k_applies(p, BM, BN)) return gemm_f32_dma_stream_k_launch(st, p, BM, BN);
    if constexpr (BM == 64) return launch_f32_dma<64, 64, 32, 4>(st, p, edge);
    else return launch_f32_dma<BM, BN, 16, OCC>(st, p, edge);
}

template <int BM, int BN, int BK, int OCC> int launch_f64_dma(hipStream_t st, const GemmProblem &p, bool edge) {
    if (gemm_f64_dma_applies(p, BM, BN)) return gemm_f64_dma_launch(st, p, BM, BN);
    return launch_f64<BM, BN, BK, 2, 2, OCC>(st, p, edge);
}

// f64 with the left-over tiles dealt by k-slabs; where that does not apply, by tiles
template <int BM, int BN, int BK, int OCC> int launch_f64_stream_k(hipStream_t st, const GemmProblem &p, bool edge) {
    if (gemm_f64_dma_stream_k_applies(p, BM, BN)) return gemm_f64_dma_stream_k_launch(st, p, BM, BN);
    return launch_f64_dma<BM, BN, BK, OCC>(st, p, edge);
}

struct VariantDesc {
    const char *name;
    int dtype, bm, bn, bk; // bk: k values per LDS slab
    double efficiency; // fraction of the matrix peak this tile shape sustains over many rounds (0: never chosen by cost)
    double fill;       // start-up and drain of a launch, in units of one round of tiles
    int (*launch)(hipStream_t, const GemmProblem &, bool);
    // k-split twins of this tile (more wavefronts per work-group, each slab shared between groups of
    // them): the variant to take instead when the launch is one round of tiles / at most two
    const char *one_round = nullptr, *two_rounds = nullptr;
    // and the quarter-size tile (one wavefront's 32x32, k split over four of them) for launches
    // whose tiles of this size would leave a quarter of the CUs or more without work
    const char *sparse = nullptr;
    // and the same tile with k split over work-groups, for few tiles and a long k (plan_split)
    const char *split = nullptr;
    // and the same tile with its left-over tiles launched as a tail with k split (plan_tail)
    const char *tail = nullptr;
    int occ = 0; // work-groups of this tile that share a compute unit (0: not needed)
};
bool is_dma_variant(const char *name) { // ...d: k-slabs straight into LDS
    const size_t n = std::strlen(name);
    return n && name[n - 1] == 'd';
}
enum { SPLIT_NONE = 0, SPLIT_ALL = 1, SPLIT_TAIL = 2 };
int split_kind_of(const char *name) { // by the name's suffix: ...z splits every tile's k, ...t the tail's
    const size_t n = std::strlen(name);
    return n && name[n - 1] == 'z' ? SPLIT_ALL : n && name[n - 1] == 't' ? SPLIT_TAIL : SPLIT_NONE;
}

const VariantDesc k_variants[] = {
    {"mfma_f32_256x128", WK_F32, 256, 128, 16, 0.940, 0.19, &launch_f32<256, 128, 16, 2, 2, 2>, nullptr, nullptr, nullptr, nullptr,
     "mfma_f32_256x128t", 2},
    // slabs straight into LDS, three deep; 16-byte aligned rows only (the cost loop skips it elsewhere):
    // 147.5 against 142.5 TFLOP/s at 8192^3, T,N 145.5 against 136
    {"mfma_f32_256x128d", WK_F32, 256, 128, 16, 0.943, 0.08, &launch_f32_dma<256, 128, 16, 2>, nullptr, nullptr, nullptr, nullptr,
     "mfma_f32_256x128t", 2},
    // 2048 x 4096 x 4096: N,T 143.0 (staged 139.6), N,N 141.8 (132.0); 4096^3 144
    {"mfma_f32_128x128d", WK_F32, 128, 128, 16, 0.922, 0.08, &launch_f32_dma<128, 128, 16, 3>, "mfma_f32_128x128d2", nullptr, nullptr, nullptr,
     "mfma_f32_128x128t", 3},
    // 3072^3 129.7 (staged 120.4), 2048 x 1024 x 4096 132 (126), 1024^3 103.7 (101.5 with four k-groups)
    {"mfma_f32_64x64d", WK_F32, 64, 64, 32, 0.84, 0.10, &launch_f32_dma<64, 64, 32, 4>, "mfma_f32_64x64d2", nullptr, "mfma_f32_32x32s4",
     "mfma_f32_64x64z"},
    // eight wavefronts per tile in two k-groups, for launches of one round (see gemm_f32_dma_kernel).  Measured
    // against the one-group kernels (N,N / N,T / T,N / T,T, TFLOP/s): 2048^3 129.5 / 132.6 / 122.9 / 129.7 ->
    // 133.7 / 137.2 / 129.1 / 133.2, 1024 x 4096 x 2048 T,N 123.9 -> 128.0; 64 x 64: 1024^3 102 / 101 / 105 / 102 ->
    // 105 / 106 / 97 / 103, 1024 x 1024 x 4096 121 / 120 / 124 / 119 -> 124 / 127 / 120 / 123: not for T,N there
    {"mfma_f32_128x128d2", WK_F32, 128, 128, 32, 0.0, 0.08, &launch_f32_dma2<128, 128>},
    {"mfma_f32_64x64d2", WK_F32, 64, 64, 32, 0.0, 0.10, &launch_f32_dma2<64, 64>},
    // the same kernels with the work dealt by k-slabs (see gemm_f32_dma_kernel), for tiles that do not fill whole rounds
    {"mfma_f32_256x128k", WK_F32, 256, 128, 16, 0.0, 0.08, &launch_f32_stream_k<256, 128, 2>, nullptr, nullptr, nullptr, nullptr, nullptr, 2},
    {"mfma_f32_128x128k", WK_F32, 128, 128, 16, 0.0, 0.08, &launch_f32_stream_k<128, 128, 3>, nullptr, nullptr, nullptr, nullptr, nullptr, 3},
    {"mfma_f32_64x64k", WK_F32, 64, 64, 32, 0.0, 0.10, &launch_f32_stream_k<64, 64, 3>, nullptr, nullptr, nullptr, nullptr, nullptr, 3},
    {"mfma_f32_256x128t", WK_F32, 256, 128, 16, 0.0, 0.25, &launch_f32_tail<256, 128, 16, 2, 2, 2>, nullptr, nullptr, nullptr, nullptr,
     nullptr, 2}, // whole rounds + a k-split tail
    {"mfma_f32_128x128", WK_F32, 128, 128, 16, 0.897, 0.19, &launch_f32<128, 128, 16, 2, 2, 3>, nullptr, nullptr, nullptr, nullptr,
     "mfma_f32_128x128t", 3},
    {"mfma_f32_128x128t", WK_F32, 128, 128, 16, 0.0, 0.25, &launch_f32_tail<128, 128, 16, 2, 2, 3>, nullptr, nullptr, nullptr, nullptr,
     nullptr, 3},
    {"mfma_f32_128x128s2", WK_F32, 128, 128, 32, 0.0, 0.25, &launch_f32<128, 128, 16, 2, 2, 2, 2>}, // 2 groups x 16 k, see pick
    {"mfma_f32_64x64", WK_F32, 64, 64, 32, 0.813, 0.13, &launch_f32<64, 64, 32, 2, 2, 4>, "mfma_f32_64x64s4", "mfma_f32_64x64s2",
     "mfma_f32_32x32s4", "mfma_f32_64x64z"},
    {"mfma_f32_64x64z", WK_F32, 64, 64, 32, 0.0, 0.10, &launch_f32_split64}, // k split over work-groups
    {"mfma_f32_64x64s2", WK_F32, 64, 64, 32, 0.0, 0.10, &launch_f32<64, 64, 16, 2, 2, 4, 2>}, // 2 groups x 16 k
    {"mfma_f32_64x64s4", WK_F32, 64, 64, 64, 0.0, 0.10, &launch_f32<64, 64, 16, 2, 2, 4, 4>}, // 4 groups x 16 k
    {"mfma_f32_32x32s4", WK_F32, 32, 32, 64, 0.0, 0.10, &launch_f32<32, 32, 16, 1, 1, 4, 4>}, // one wavefront's tile, 4 groups
    {"mfma_f64_128x128", WK_F64, 128, 128, 16, 0.908, 0.20, &launch_f64<128, 128, 16, 2, 2, 2>},
    {"mfma_f64_64x64", WK_F64, 64, 64, 32, 0.840, 0.05, &launch_f64<64, 64, 32, 2, 2, 2>, "mfma_f64_64x64s2", nullptr,
     "mfma_f64_32x32s4", "mfma_f64_64x64z"},
    // slabs straight into LDS, three deep (wk_gemm_dma.hip), interior shapes: 4096^3 70.2 against 68.5 TFLOP/s
    {"mfma_f64_128x128d", WK_F64, 128, 128, 16, 0.94, 0.10, &launch_f64_dma<128, 128, 16, 2>},
    // 8192 x 256 x 8192 69.6 (staged 62.2), 2048^3 68 (61.7), 4096^3 69-70.5
    {"mfma_f64_64x64d", WK_F64, 64, 64, 32, 0.89, 0.05, &launch_f64_dma<64, 64, 32, 2>, nullptr, nullptr, "mfma_f64_32x32s4", "mfma_f64_64x64z"},
    {"mfma_f64_64x64z", WK_F64, 64, 64, 32, 0.0, 0.05, &launch_f64_split64}, // k split over work-groups
    // the direct-to-LDS kernels with the left-over tiles dealt by k-slabs (see gemm_f64_dma_kernel)
    {"mfma_f64_128x128k", WK_F64, 128, 128, 16, 0.0, 0.10, &launch_f64_stream_k<128, 128, 16, 2>, nullptr, nullptr, nullptr, nullptr, nullptr, 2},
    {"mfma_f64_64x64k", WK_F64, 64, 64, 32, 0.0, 0.05, &launch_f64_stream_k<64, 64, 32, 2>, nullptr, nullptr, nullptr, nullptr, nullptr, 3},
    {"mfma_f64_64x64s2", WK_F64, 64, 64, 64, 0.0, 0.05, &launch_f64<64, 64, 32, 2, 2, 2, 2>}, // 2 groups x 32 k
    // (two wavefronts per SIMD: with a 128-register budget its staging sets and fragments spill and it
    // runs several times slower than the 64x64 tile)
    {"mfma_f64_32x32s4", WK_F64, 32, 32, 64, 0.0, 0.05, &launch_f64<32, 32, 16, 1, 1, 2, 4>},
    {"mfma_f64_128x64", WK_F64, 128, 64, 16, 0.863, 0.25, &launch_f64<128, 64, 16, 2, 2, 3>},
    // 32-bit integers through the int8 matrix cores (wk_gemm_imfma.hip); same kernel for both signs
    // (efficiency here is relative between the two integer tiles: 196-202 against 155-192 TOP/s)
    {"mfma_i32_64x128", WK_I32, 64, 128, 32, 0.88, 0.25, &gemm_i32_mfma_launch_64},
    {"mfma_u32_64x128", WK_U32, 64, 128, 32, 0.88, 0.25, &gemm_i32_mfma_launch_64},
    {"mfma_i32_128x128", WK_I32, 128, 128, 32, 1.0, 0.25, &gemm_i32_mfma_launch_128},
    {"mfma_u32_128x128", WK_U32, 128, 128, 32, 1.0, 0.25, &gemm_i32_mfma_launch_128},
};
constexpr int k_num_variants = sizeof(k_variants) / sizeof(k_variants[0]);

} // namespace

// The fused epilogue is instantiated for the f32 / f64 kernels of this file and for op N, T only
// (x * W^T, the product Linear.forward makes).
bool wk::gemm_mfma_fuses(const GemmProblem &p, int variant) {
    if (variant < 0 || variant >= k_num_variants) return false;
    const VariantDesc &v = k_variants[variant];
    return (v.dtype == WK_F32 || v.dtype == WK_F64) && v.dtype == p.dtype && !p.op_a && p.op_b;
}

namespace {

bool needs_edge(const GemmProblem &p, const VariantDesc &v) {
    const size_t es = p.dtype == WK_F64 ? 8 : 4;
    const uint64_t vec = 16 / es;
    if (p.M % v.bm || p.N % v.bn || p.K % v.bk) return true;
    if (p.lda % vec || p.ldb % vec) return true;
    if ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15u) return true;
    return false;
}

} // namespace

const char *wk::gemm_mfma_variant_name(int variant) {
    return (variant >= 0 && variant < k_num_variants) ? k_variants[variant].name : nullptr;
}

int wk::gemm_mfma_variant_dtype(int variant) {
    return (variant >= 0 && variant < k_num_variants) ? k_variants[variant].dtype : -1;
}

// Kernel choice by a small cost model.  The matrix pipes of a CU are saturated by the work-groups
// resident on it, so a launch takes about (tiles on the busiest CU + a start-up/drain share) x
// (tile area / efficiency):
//     cost = (ceil(tiles / CUs) + fill) * BM * BN / efficiency
// `efficiency` and `fill` are fitted per macro tile to times measured on MI355X over launches of
// one to sixteen rounds (f32 256x128: 123 TFLOP/s at one tile per CU, 130 at two, 143.6 at eight;
// 128x128: 112 / 128 / 137 at one / two / sixteen; f64 alike).  This picks big tiles for big
// problems, the next size down while the big one would run a single round (a lone work-group per
// CU has nothing to overlap its hand-overs and epilogue with), small tiles when the others would
// leave CUs idle (1024^3, tall-skinny) or quantise badly (4097 x 4095: 544 tiles of 256x128 put
// three tiles on some CUs and two on the rest).
// The 64x64 tiles use k-slabs of 32: with one or two small tiles per CU the matrix work of a slab
// is shorter than the latency of the global loads behind it, and the deeper slab halves the number
// of such waits (f32 1024^3: 76 -> 84 TFLOP/s, 2048x1024x4096: 116 -> 130; f64 8192x256x8192:
// 56 -> 60); the larger tiles measured no better with it.
bool wk::gemm_mfma_split_plan(const GemmProblem &p, int variant, bool forced, GemmSplitPlan &plan) {
    plan = GemmSplitPlan{};
    if (variant < 0 || variant >= k_num_variants || p.ext) return false;
    const VariantDesc &v = k_variants[variant];
    const size_t elem = v.dtype == WK_F64 ? 8 : 4;
    switch (split_kind_of(v.name)) {
    case SPLIT_ALL: return plan_split(p, v.bm, v.bn, v.bk, elem, false, plan) || (forced && plan_split(p, v.bm, v.bn, v.bk, elem, true, plan));
    case SPLIT_TAIL: return plan_tail(p, v.bm, v.bn, v.bk, elem, v.occ, forced && tail_relaxed(), plan);
    default: return false;
    }
}

namespace {
// Splitting k costs a write and a read of every partial tile and one more pass of additions.  Measured
// on MI355X against the quarter-size tile with k split inside the work-group, the next best choice for
// few tiles: f32 512 x 512 x 8192 57 -> 52 us, 256 x 256 x 8192 54 -> 45, 1024 x 512 x 4096 43.5 -> 42,
// but 512 x 512 x 2048 14.4 -> 18.6; f64 512 x 512 x 8192 111 -> 89 us, 256 x 256 x 8192 111 -> 89,
// 512 x 512 x 2048 32 -> 30.
bool split_pays(const GemmProblem &p, const GemmSplitPlan &plan) {
    // (a thin strip -- a handful of rows or columns -- reads the whole other operand whatever the tile: there the
    // shares pay from half that length on, 1 x 4095 x 4093 47.5 -> 35.6 us, 4096 x 1 x 4093 76 -> 51)
    const bool strip = p.dtype == WK_F32 && (p.M <= 64 || p.N <= 64);
    return plan.shares >= 2 && p.K >= (p.dtype == WK_F64 || strip ? 2048u : 4096u);
}
} // namespace

namespace {
// cost of a k-split tail in rounds of its tile: launch gap, hand-overs without a co-resident
// work-group and the addition of the partial tiles (fixed part), plus the tile's time over the shares.
// Measured with the direct-to-LDS body (time of the whole launch minus the body's rounds, in tile times): 0.34
// at 4 shares (8292 x 8192 x 4096), 0.39 at 5 (4200^3) and at 8 (8191 x 8193 x 8190), 0.35 at 16 (4096 x 4160 x
// 4096): from five shares on it does not shrink any further (TAIL_FLOOR).
constexpr double TAIL_FIXED = 0.06, TAIL_PER_SHARE = 1.52, TAIL_FLOOR = 0.36;
} // namespace

int wk::gemm_mfma_pick(const GemmProblem &p, double *cost_out) {
    if (p.dtype != WK_F32 && p.dtype != WK_F64 && p.dtype != WK_I32 && p.dtype != WK_U32) return -1;
    if (p.M > 0x7fffffffull || p.N > 0x7fffffffull || p.K > 0x7fffffffull || p.lda > 0x7fffffffull ||
        p.ldb > 0x7fffffffull || p.ldc > 0x7fffffffull)
        return -1;
    const double cus = p.num_cus ? (double)p.num_cus : 256.0;
    int best = -1;
    double best_cost = 0.0;
    for (int v = 0; v < k_num_variants; ++v) {
        const VariantDesc &d = k_variants[v];
        if (d.dtype != p.dtype || d.efficiency <= 0.0) continue;
        if (is_dma_variant(d.name) && !(d.dtype == WK_F64 ? gemm_f64_dma_applies(p, d.bm, d.bn) : gemm_f32_dma_applies(p, d.bm, d.bn)))
            continue;
        const double tiles = (double)((p.M + d.bm - 1) / d.bm) * (double)((p.N + d.bn - 1) / d.bn);
        // Whole rounds: the big tiles (two or three work-groups per unit) pay for a started round in
        // full, the small tile (four per unit, short) for about two thirds of it.
        const double whole = (double)(uint64_t)((tiles + cus - 1.0) / cus);
        const double rounds = tiles / cus + (d.bm <= 64 ? 0.65 : 1.0) * (whole - tiles / cus);
        // the bounds-checked instantiation runs slower than the interior one (8191 x 8193 x 8190 against
        // 8192^3 on the 256 x 128 tile: 126 against 142 TFLOP/s with the tail split off)
        // (the direct-to-LDS kernels run ragged shapes in the same loop: their cost is in the tile count)
        const bool slower_edge = needs_edge(p, d) && !is_dma_variant(d.name);
        const double eff = d.efficiency * (slower_edge ? (d.bm >= 256 ? 0.86 : d.bm >= 128 ? 0.944 : 0.93) : 1.0);
        const double cost = (rounds + d.fill) * d.bm * d.bn / eff;
        if (best < 0 || cost < best_cost) {
            best = v;
            best_cost = cost;
        }
        // the same tile with its left-over tiles as a k-split tail: the whole rounds, then a second
        // launch that keeps every unit busy for a fraction of a tile's time (tail_rounds fitted to
        // measured launches)
        GemmSplitPlan tp;
        if (d.tail && !p.ext && plan_tail(p, d.bm, d.bn, d.bk, 4, d.occ, false, tp)) {
            const double tail_rounds = std::max(TAIL_FIXED + TAIL_PER_SHARE / tp.shares, TAIL_FLOOR);
            const double tcost = ((double)tp.first_tile / cus + d.fill + tail_rounds * tp.tiles * tp.shares / cus) * d.bm * d.bn / eff;
            if (tcost < best_cost)
                for (int w = 0; w < k_num_variants; ++w)
                    if (!std::strcmp(k_variants[w].name, d.tail)) {
                        best = w;
                        best_cost = tcost;
                    }
        }
    }
    // Tiles that do not come out even over the compute units: the whole rounds of tiles run whole and the k-slabs of
    // the tiles that are left are dealt to one more work-group per unit (the "...k" kernels, wk_gemm_dma.hip), so
    // that every unit has the same amount of matrix work, where that beats what was found above by more than the
    // model's error.  Fitted on cubes from 2200 to 6000 and six other shapes (N,N): the time is that of tiles / units
    // tile times at an efficiency of 0.90 (128 x 128) / 0.933 (256 x 128) plus 15 / 36 us per launch (the dealt
    // work-groups are done early, and their parts are added while the whole tiles are still being multiplied;
    // with every tile dealt, as at first, the exchange stood at the end of the launch and cost 22 us).
    // Measured against the choice without it, N,N, TFLOP/s: 2200^3 100 -> 118, 2300^3 112 -> 130, 2500^3 113 -> 127,
    // 2700^3 113 -> 126, 3000^3 122 -> 132, 3200^3 126 -> 140, 3500^3 124 -> 132, 3700^3 123 -> 138, 4000^3 130 -> 137,
    // 4500^3 129 -> 135, 5000^3 133 -> 136, 6000^3 134 -> 141, 3000 x 3000 x 8192 124 -> 136, 2500 x 3500 x 4096 123 ->
    // 133, 3333 x 3333 x 1111 105 -> 123; nothing to gain where the tiles are whole rounds (2048 x 4096 x 1024).
    // (f64, fitted the same way on cubes from 1100 to 4300: 64 x 64 0.887 and 12 us, 128 x 128 0.897 and 20 us; 1100^3
    // 37 -> 50 TFLOP/s, 1536^3 51 -> 66, 1792^3 52 -> 66, 2300^3 58 -> 68, 2500^3 59 -> 65, 3456^3 51 -> 70, 4300^3 63 -> 69)
    if ((p.dtype == WK_F32 || p.dtype == WK_F64) && best >= 0 && p.K >= 256 && g_test_options.stream_k) {
        const double cost_per_us = p.dtype == WK_F32 ? 3.05e5 : 1.525e5;
        static const struct { const char *name; int dtype, bm, bn; double eff, fixed_us; uint64_t min_k; } dealt[] = {
            {"mfma_f32_128x128k", WK_F32, 128, 128, 0.90, 15.0, 256}, {"mfma_f32_256x128k", WK_F32, 256, 128, 0.933, 36.0, 1024},
            {"mfma_f32_64x64k", WK_F32, 64, 64, 0.83, 6.0, 256},
            {"mfma_f64_128x128k", WK_F64, 128, 128, 0.897, 20.0, 1024}, {"mfma_f64_64x64k", WK_F64, 64, 64, 0.887, 12.0, 256}};
        // Below k = 1024 the figure found above leaves out what a tile costs whatever its k (filling the stages, the
        // epilogue: about 300 values of k in f32, 250 in f64, fitted on 1536 x 1536 x 256 ... 512), which the dealt
        // kernels' own constant holds; for the comparison it is put back.  (Automatic choice against the best forced
        // variant over 16 shapes x k = 256 ... 512 x N,N / T,N before: 7.8 % behind on average in f32, 6.4 % in f64.)
        const double short_k = p.K < 1024 ? 1.0 + (p.dtype == WK_F32 ? 300.0 : 250.0) / (double)p.K : 1.0;
        const double plain_cost = best_cost * short_k;
        double bar = plain_cost; // the figure to beat: the plain choice's, then that of the dealt kernel taken so far
        for (const auto &d : dealt) {
            if (d.dtype != p.dtype || p.K < d.min_k) continue;
            const double tiles = (double)((p.M + d.bm - 1) / d.bm) * (double)((p.N + d.bn - 1) / d.bn);
            const bool applies = p.dtype == WK_F32 ? gemm_f32_dma_stream_k_applies(p, d.bm, d.bn) : gemm_f64_dma_stream_k_applies(p, d.bm, d.bn);
            if (!applies) continue;
            bool by_rule = false;
            if (tiles <= cus) {
                // At most one tile per unit: the small tile with every tile's k-slabs dealt over all the work-groups
                // that are resident, where k is long and the tiles (or the shares the k-split kernels would cut
                // them into) do not come out even over the units.  Measured against the choice without it, N,N /
                // T,N, TFLOP/s: f64 768 x 768 x 4096 36 / 35 -> 57 / 57, 832^2 x 4096 42 / 41 -> 58 / 57, 640^2 x 4096 44 / 42 ->
                // 51 / 52, 384^2 x 16384 32 -> 44, 960^2 x 2048 49 / 47 -> 53 / 54, 1024^2 x 8192 59 / 56 -> 66 / 66 (x 1024: 52 -> 48,
                // not taken); 512^2 and 512 x 1024 (64 and 128 tiles: whole shares per unit) and 256^2 x 65536 within
                // +-5 % or worse, not taken.  f32 768^2 x 4096 80 / 77 -> 107 / 99, x 2048 75 / 72 -> 86 / 83, 832^2 x 4096 93 / 90 -> 107 /
                // 103, 640^2 x 4096 75 -> 91 (x 2048: 72 -> 68, not taken), 512^2 x 8192 90 -> 96, 384^2 x 16384 75 -> 85, 512 x
                // 1024 x 8192 111 / 106 -> 117 / 119; a full round (1024^2) is the two-group kernel's: 130 against 121-125.
                if (d.bm != 64 || p.K < 2048) continue;
                const uint64_t t = (uint64_t)tiles, units = (uint64_t)cus;
                // (N,T is the layout the plain kernels read best: a nearly full round of it stays theirs in f64, 0.91-0.96
                // of their rate dealt, and so does k < 4096 in f32; f32 below 42 tiles loses: 256 x 384 x 4096 20 -> 32 us)
                const bool nt = !p.op_a && p.op_b;
                const bool take = p.dtype == WK_F64 ? t >= 32 && (t == units || units % t != 0) && !(nt && 10 * t > 8 * units)
                                                    : 10 * t <= 9 * units && t >= 42 && (p.K >= 4096 || (2 * t > units && !nt));
                if (!take) continue;
                by_rule = true; // (the model above has no figure for a single round that these measurements bear out)
            } else if (std::fmod(tiles, cus) == 0.0) {
                continue;
            }
            const double cost = tiles / cus * d.bm * d.bn / d.eff + d.fixed_us * cost_per_us / (double)p.K;
            if (by_rule || (cost < 0.98 * plain_cost && cost < bar))
                for (int w = 0; w < k_num_variants; ++w)
                    if (!std::strcmp(k_variants[w].name, d.name)) {
                        best = w;
                        best_cost = cost;
                        bar = cost;
                    }
        }
    }
    // f64 with a short k: the small tile, whose epilogue and stage fill are a quarter of the large one's per work-group
    // and overlap three to a unit (4096 x 2048 x 256 82 -> 74 us, 2048 x 6144 x 256 122 -> 109, 8192 x 1024 x 384 111 -> 103,
    // 2048 x 6144 x 640 258 -> 238; from k = 1000 on the large tile is level or ahead
    // -- up to four rounds of the large tile; beyond, it is the better one again: 7000 x 7000 x 512 T,N 798 us against 888)
    if (p.dtype == WK_F64 && p.K < 768 && best >= 0 && !std::strcmp(k_variants[best].name, "mfma_f64_128x128d") &&
        (double)((p.M + 127) / 128) * (double)((p.N + 127) / 128) <= 4.0 * cus && gemm_f64_dma_applies(p, 64, 64))
        for (int w = 0; w < k_num_variants; ++w)
            if (!std::strcmp(k_variants[w].name, "mfma_f64_64x64d")) best = w;
    if (cost_out) *cost_out = best_cost;
    // f32 problems that are one nearly full round of 128x128 tiles: that tile with two k-groups (eight
    // wavefronts per CU) beats the four rounds of 64x64 the cost model would take -- 2048^3 126 / 132 /
    // 120 / 126 -> 130 / 136 / 126 / 131 TFLOP/s (NN / NT / TN / TT), 2048x2048x4096 128 -> 134.  With
    // fewer tiles (1536^3) or more than one round (3072^3) the 64x64 tile wins.
    const bool best_dealt = best >= 0 && k_variants[best].name[std::strlen(k_variants[best].name) - 1] == 'k';
    if (p.dtype == WK_F32 && p.K >= 512) {
        const double tiles128 = (double)((p.M + 127) / 128) * (double)((p.N + 127) / 128);
        // (where the small tile dealt by k-slabs was found cheaper, it is, unless the round is all but full:
        // 1800^3 118 against 100 TFLOP/s, 1900^3 121 against 110, 2000^3 126 / 124, 2048^3 134 / 134.5)
        if (tiles128 <= cus && tiles128 >= (best_dealt ? 0.97 : 0.85) * cus) {
            // (the direct-to-LDS kernel of that tile where it applies: 2048^3 N,N 131 against 128.5)
            const char *want = !gemm_f32_dma_applies(p, 128, 128) ? "mfma_f32_128x128s2"
                               : (p.K >= 1024 && !p.ext && gemm_dma_rows_aligned(p)) ? "mfma_f32_128x128d2"
                                                                   : "mfma_f32_128x128d";
            // Since launches of between one and two rounds of the 64 x 64 tile take their tiles in turn (three
            // work-groups per unit: more than 768 and fewer than 1536 tiles), that tile is the faster one here up to
            // k = 2048, except with a k-contiguous B beside an A that is too (N,T), which the two-group kernel reads
            // best.  NN / NT / TN / TT, TFLOP/s, two-group 128 x 128 against 64 x 64: 2048^3 130 / 136 / 128 / 129 against
            // 134 / 131 / 132 / 131, 2048 x 2048 x 1024 121 / 125 / 119 / 120 against 127 / 125 / 126 / 126, 2048 x 2048 x 512
            // 105 / 108 / 104 / 104 against 113 / 115 / 111 / 112, 4096 x 1024 x 2048 130 / 136 / 128 / 129 against 133 /
            // 132 / 132 / 132; 2048 x 2048 x 4096 137 / 142 / 134 / 135 against 136 / 135 / 136 / 137: not from there on.
            const double tiles64 = (double)((p.M + 63) / 64) * (double)((p.N + 63) / 64);
            if (!p.ext && g_test_options.persistent && tiles64 > 3.0 * cus && tiles64 < 6.0 * cus && p.K <= 2048 &&
                (p.K <= 512 || p.op_a || !p.op_b) && gemm_f32_dma_applies(p, 64, 64) && gemm_dma_rows_aligned(p))
                want = "mfma_f32_64x64d";
            for (int v = 0; v < k_num_variants; ++v)
                if (!std::strcmp(k_variants[v].name, want)) return v;
        }
    }
    // A launch of one round (f32: up to two) of the small tile leaves each SIMD one or two wavefronts,
    // which stall together at every hand-over: the k-split twin of the tile gives it two to four.
    // Measured on MI355X, f32: 1024^3 90.8 -> 101.8 TFLOP/s, 1000^3 64 -> 76, 1024x1024x4096 102 -> 119,
    // 2048x1024x1024 (two rounds) 108 -> 113; f64: 1024^3 47 -> 53, 1000^3 36.6 -> 42.9.  From three
    // rounds on, and for short k, the plain tile is as fast or faster.
    // Below three quarters of a round the quarter-size tile spreads the work over the idle CUs
    // (f32 512^3: 13.1 -> 6.9 us, 512x512x2048: 43.5 -> 15.7 us, 768^3: 18.5 -> 14.8 us; at 1024^3 it loses).
    if (best >= 0 && p.K >= 64) {
        const VariantDesc &d = k_variants[best];
        const double tiles = (double)((p.M + d.bm - 1) / d.bm) * (double)((p.N + d.bn - 1) / d.bn);
        const char *twin = nullptr;
        GemmSplitPlan plan;
        if (d.split && !p.ext && plan_split(p, d.bm, d.bn, d.bk, p.dtype == WK_F64 ? 8 : 4, false, plan) &&
            split_pays(p, plan))
            twin = d.split;
        else if (tiles <= 0.75 * cus && d.sparse) twin = d.sparse; // (f64 512^3: 21.5 -> 10.3 us, 512x512x2048: 74 -> 32 us)
        else if (p.K >= 256) twin = tiles <= cus ? d.one_round : (tiles <= 2.0 * cus ? d.two_rounds : nullptr);
        if (twin && twin == d.one_round && is_dma_variant(d.name)) { // the two-group direct-to-LDS kernels: not fused
            if (p.ext || !gemm_dma_rows_aligned(p) || p.K < (d.bm == 64 ? 512u : 1024u)) twin = nullptr; // (below: equal)
            else if (d.bm == 64 && p.op_a && !p.op_b) twin = nullptr;       // 64 x 64, T,N: the one-group kernel is faster
        }
        for (int v = 0; twin && v < k_num_variants; ++v)
            if (!std::strcmp(k_variants[v].name, twin)) return v;
    }
    return best;
}

int wk::gemm_mfma_launch(hipStream_t st, const GemmProblem &p, int variant) {
    if (variant < 0 || variant >= k_num_variants || k_variants[variant].dtype != p.dtype) return WK_E_INVALID_VALUE;
    // the kernels index with 32 bits per dimension; automatic selection never gets here with more
    // (gemm_mfma_pick declines), a forced variant is turned away
    if (p.M > 0x7fffffffull || p.N > 0x7fffffffull || p.K > 0x7fffffffull || p.lda > 0x7fffffffull ||
        p.ldb > 0x7fffffffull || p.ldc > 0x7fffffffull)
        return WK_E_INVALID_VALUE;
    const VariantDesc &v = k_variants[variant];
    const uint64_t tiles = ((p.M + v.bm - 1) / v.bm) * ((p.N + v.bn - 1) / v.bn);
    if (tiles > 0x7fffffffull) return WK_E_INVALID_VALUE;
    return v.launch(st, p, needs_edge(p, v));
}
