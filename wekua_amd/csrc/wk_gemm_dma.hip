// f32 GEMM on the CDNA4 matrix cores with k-slabs brought from global memory straight into LDS
// (gfx950's 16-byte-per-lane global_load_lds), three slabs deep.
//
// Same tiling and matrix-instruction mapping as the kernels of wk_gemm_mfma.hip
// (v_mfma_f32_32x32x2_f32, 2 x 2 wavefronts, macro tiles 256 x 128 and 128 x 128 with k-slabs of 16, 64 x 64 with 32),
// for operands whose rows start on 16-byte boundaries (any M, N, K).  What differs is how a slab gets into LDS and how the work-group hands over from one
// slab to the next:
//   * no staging registers and no LDS stores: every lane names 16 bytes of global memory and the
//     load unit writes them to LDS at (wave-uniform base) + 16 * lane.  The lane -> address map is
//     free, the LDS side is not, so padding is replaced by swizzling: the lane that fills LDS
//     chunk p of a row fetches the chunk that belongs there;
//   * unpadded slabs of the 256 x 128 tile are 24 KB (A 16 KB + B 8 KB), so three of them fit twice
//     on a compute unit (144 of 160 KB; 128 x 128: 3 x 16 KB three times; 64 x 64 with k-slabs of 32: 3 x 16 KB three times).  Slab kt+2 is requested at the top of iteration kt, a whole iteration and a
//     half before it is read, and the only thing between the matrix instructions of two slabs is
//     one barrier (every wavefront first waits for its own share of slab kt+1 to have landed).
//
// LDS layouts (floats):
//   k-contiguous operand (A for op_a = N, B for op_b = T): [row][16], four 16-byte chunks per row,
//     chunk c of row r stored at chunk position c ^ ((r >> 2) & 3).  A fragment is one 16-byte read
//     per lane (row = lane % 32, k = 8 s + 4 (lane / 32) + 0..3); sixteen consecutive rows at one
//     logical chunk cover all 64 banks once.
//   m/n-contiguous operand (A for op_a = T, B for op_b = N): [k][ROWS], element (k, m) stored at
//     m ^ (32 * ((k >> 2) & 1)).  Fragments are 4-byte reads; the two half-wavefronts read rows k
//     and k + 4, which the swizzle puts on disjoint banks.
//
// The loads are issued through inline assembly: the compiler's wait-count pass treats a direct-to-LDS
// load it knows about as a store that any later LDS read may alias and would wait for all of them in
// front of every fragment read, which serialises exactly what this kernel overlaps.  The waits that
// are needed are written out instead (vmcnt before the barrier that publishes a slab).
#include "wk_internal.hpp"
#include "wk_lds_dma.hpp"

#include <cstdlib>
#include <cstring>

using namespace wk;
using namespace wk::lds_dma;

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int GROUP_M = 8;

// In front of every tile (or part of a tile) of a work-group that may run several: `again` false for the first.
// The counted wait is one the compiler sees, and it is on every path: without it the compiler's wait-count pass
// carries loads of the tile before (C_old, partial tiles) as possibly pending into the next tile's main loop and,
// where the register allocation happens to reuse their registers for fragments, puts a vmcnt(0) into that loop,
// which drains the slab pipeline in every iteration (128 x 128 N,N: 111 against 129 TFLOP/s at 2300^3).  The barrier:
// every wavefront is done with the LDS stages of the tile before.
__device__ __forceinline__ void next_tile(bool again) {
    __builtin_amdgcn_s_waitcnt(0);
    if (again) __syncthreads();
}

struct DArgs {
    const float *A, *B;
    float *C;
    uint32_t M, N, K;
    uint32_t lda, ldb, ldc;
    uint32_t tiles_m, tiles_n;
    int epi;
    float alpha, beta;
    const float *bias; // kernels instantiated with EXT: C = act(acc + bias[col]); bias may be null
    int act;
    uint32_t patch_m, patch_n; // tile walk in XCD-local patches of patch_m x patch_n tiles (0: rows of groups)
    // kernels instantiated with SK (work dealt by k-slabs, not by tiles): k-slabs per work-group, k-slabs in all
    // (tiles x slabs per tile), memory for two partial tiles per work-group and one arrival counter per tile
    // sk_first: the tiles before that one are run whole, one work-group each (work-groups sk_groups ... of the
    // launch); the k-slabs of the tiles from it on are dealt to work-groups 0 ... sk_groups - 1
    uint32_t sk_units, sk_total, sk_first, sk_groups;
    // tiles of this launch (one work-group each, or fewer work-groups that take every gridDim.x-th tile in turn)
    uint32_t tiles_run;
    float *partials;
    uint32_t *counters;
};

// KS: groups of 2 x 2 wavefronts on the same tile (1 or 2).  A launch of one round of tiles leaves every SIMD
// a single wavefront, which stands still at every wait; with KS = 2 all eight wavefronts bring the slabs
// in, group kg multiplies steps kg * S / KS ... of every slab, and the two partial tiles are added
// through LDS (the stages, free by then) before group 0 runs the epilogue.
// VB: bytes per lane and load.  16 for operands whose rows start on 16-byte boundaries; 4 for any other (every
// lane then fetches one float into the same place of the same LDS layout: SUB = 4 loads per KiB instead of one,
// nothing read beyond the end of a row).
// SK: for products whose tiles do not come out even over the compute units.  The first sk_groups work-groups of
// the launch are dealt k-slabs instead of tiles: the slabs of the tiles from sk_first on are numbered in tile-walk
// order and work-group b takes [b' U, (b' + 1) U) of them (b' numbers the work-groups of one XCD consecutively); every
// later work-group runs one whole tile, as ever.  With one dealt work-group per unit beside the whole tiles every
// unit has the same amount of matrix work (gemm_dma_stream_k_plan below; with fewer tiles than units every tile
// is dealt, to as many work-groups as are resident).  A dealt range that holds a whole tile runs it as ever; a
// part of a tile (at most two per work-group: the end of one tile at the start of its range, the start of
// another at its end) goes to memory as a partial tile, and the work-group that arrives last at the tile's
// counter adds the parts up in the order of k, so the bits do not depend on who that is (the part that starts the
// tile stays in its registers when it is the last to arrive: 0 + p0 + p1 ... and p0 + p1 ... are the same
// bits), and runs the epilogue.  The same hand-over as the k-split kernels of wk_gemm_mfma.hip (device-scope stores
// and loads, a wait for the stores in front of the count).
template <int BM, int BN, int BK, int NS, int OCC, bool A_K, bool B_K, bool EXT, int KS = 1, int VB = 16, bool SK = false>
__global__ __launch_bounds__(256 * KS) __attribute__((amdgpu_waves_per_eu(OCC)))
void gemm_f32_dma_kernel(DArgs g) {
    static_assert(VB == 16 || VB == 4, "bytes per lane");
    static_assert(!SK || KS == 1, "work dealt by k-slabs: one group of wavefronts");
    constexpr int SUB = 16 / VB;
    __shared__ uint32_t s_last;
    auto run = [&](const uint32_t pid, const uint32_t kb, const uint32_t ke, const uint32_t bq) __attribute__((always_inline)) {
    constexpr int WM = BM / 2, WN = BN / 2, FM = WM / 32, FN = WN / 32;
    constexpr int S = BK / 8;   // fragment steps per slab (8 values of k each: four matrix instructions per block)
    constexpr int CPR = BK / 4; // 16-byte chunks per row of a k-contiguous slab
    constexpr int A_FLOATS = BM * BK, B_FLOATS = BN * BK, STAGE = A_FLOATS + B_FLOATS;
    constexpr int WAVES = 4 * KS;
    constexpr int SG = S / KS; // steps of a slab per group of wavefronts
    constexpr int A_LOADS = BM * BK / (256 * WAVES), B_LOADS = BN * BK / (256 * WAVES); // 1 KB per wavefront and load
    static_assert(BM % 64 == 0 && BN % 64 == 0 && (BK == 16 || BK == 32) && NS >= 2, "tile shape");
    static_assert((KS == 1 || KS == 2) && SG >= 2 && SG % 2 == 0 && A_LOADS >= 1 && B_LOADS >= 1, "k-groups");

    extern __shared__ __align__(16) float lds[]; // [NS][STAGE]: A then B

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // the same in every lane: kept in a scalar register
    const int kg = wave >> 2;                                  // k-group of this wavefront
    const int wm = (wave >> 1) & 1, wn = wave & 1;
    const int l32 = lane & 31, lhi = lane >> 5;

    // tile walk: groups of GROUP_M tile rows, as in wk_gemm_mfma.hip (every XCD sweeps the same panel of B)
    uint32_t tile_m, tile_n;
    if (g.patch_m) {
        // work-group b runs on XCD b % 8: the j-th work-group of an XCD takes tile j % (patch) of that
        // XCD's patch j / (patch), so the tiles that share an L2 at one time share rows of A and columns of B
        const uint32_t x = pid & 7u, j = pid >> 3;
        const uint32_t per_patch = g.patch_m * g.patch_n;
        const uint32_t patch = (j / per_patch) * 8u + x, q = j % per_patch;
        const uint32_t patches_n = g.tiles_n / g.patch_n;
        tile_m = (patch / patches_n) * g.patch_m + q % g.patch_m;
        tile_n = (patch % patches_n) * g.patch_n + q / g.patch_m;
    } else {
        const uint32_t group_size = GROUP_M * g.tiles_n;
        const uint32_t group = pid / group_size;
        const uint32_t first_m = group * GROUP_M;
        const uint32_t gsz = min(g.tiles_m - first_m, (uint32_t)GROUP_M);
        const uint32_t in_group = pid - group * group_size;
        tile_m = first_m + in_group % gsz;
        tile_n = in_group / gsz;
    }
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    // position of a 16-byte chunk inside its row of a k-contiguous slab: chunk number ^ swizzle(row)
    auto swizzle = [](uint32_t row) -> uint32_t { return CPR == 4 ? (row >> 2) & 3u : (row >> 1) & 7u; };

    // ---- global side: scalar bases (advance by one slab per iteration) and per-lane byte offsets ----
    const float *a_base = A_K ? g.A + (size_t)m0 * g.lda : g.A + m0;
    const float *b_base = B_K ? g.B + (size_t)n0 * g.ldb : g.B + n0;
    const size_t a_step = A_K ? (size_t)BK : (size_t)BK * g.lda; // floats per slab
    const size_t b_step = B_K ? (size_t)BK : (size_t)BK * g.ldb;
    if constexpr (SK) { // this range starts at slab kb of the tile
        a_base += kb * a_step;
        b_base += kb * b_step;
    }
    uint32_t a_off[A_LOADS * SUB], b_off[B_LOADS * SUB];
    // loads i * SUB ... of this wavefront fill the 1 KB group i * 4 + wave of the operand's slab: sixteen rows of a
    // k-contiguous operand, 256 / ROWS rows of k of an m-contiguous one
    // Rows (columns) of the tile beyond the matrix are fetched from its last row (column): they only feed
    // entries of C that are never stored.  A 16-byte chunk whose first float exists is fetched as it is:
    // bases and leading dimensions are multiples of 16 bytes, so the chunk cannot leave the page of
    // that float.  `last` = index of the last existing row (column) counted from the tile's origin.
    // With one float per lane (VB = 4) lane l of load q of a group fetches the float that belongs at float
    // 64 q + l of the group.
    auto lane_offset = [&](int grp, int q, uint32_t ld, uint32_t last, auto kc_tag, auto rows_tag) -> uint32_t {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        if constexpr (VB == 16) {
            if constexpr (KC) {
                const uint32_t row = grp * (64 / CPR) + lane / CPR;
                const uint32_t chunk = (lane % CPR) ^ swizzle(row);
                return (min(row, last) * ld + 4 * chunk) * 4u;
            } else {
                constexpr int PER_ROW = ROWS / 4; // 16-byte chunks per row of k
                const uint32_t k = grp * (64 / PER_ROW) + lane / PER_ROW;
                const uint32_t chunk = (lane % PER_ROW) ^ (((k >> 2) & 1) * 8);
                return (k * ld + 4 * min(chunk, last >> 2)) * 4u;
            }
        } else {
            const uint32_t f = 64 * q + lane; // float of the group
            if constexpr (KC) {
                const uint32_t row = grp * (256 / BK) + f / BK, pos = f % BK;
                const uint32_t chunk = (pos >> 2) ^ swizzle(row);
                return (min(row, last) * ld + 4 * chunk + (pos & 3)) * 4u;
            } else {
                const uint32_t k = grp * (256 / ROWS) + f / ROWS;
                const uint32_t m = (f % ROWS) ^ (((k >> 2) & 1) * 32);
                return (k * ld + min(m, last)) * 4u;
            }
        }
    };
    using std::integral_constant;
    const uint32_t m_last = g.M - 1 - m0, n_last = g.N - 1 - n0;
#pragma unroll
    for (int i = 0; i < A_LOADS * SUB; ++i)
        a_off[i] = lane_offset((i / SUB) * WAVES + wave, i % SUB, g.lda, m_last, integral_constant<bool, A_K>{}, integral_constant<int, BM>{});
#pragma unroll
    for (int i = 0; i < B_LOADS * SUB; ++i)
        b_off[i] = lane_offset((i / SUB) * WAVES + wave, i % SUB, g.ldb, n_last, integral_constant<bool, B_K>{}, integral_constant<int, BN>{});
    const uint32_t lds0 =
        __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) float *)lds); // byte address of the array

    // the next slab of both operands into the stage at byte offset `stage_bytes`; the bases then point at
    // the slab after it
    auto issue = [&](uint32_t stage_bytes) {
        const uint32_t sbase = lds0 + stage_bytes + (uint32_t)wave * 1024u;
        if constexpr (VB == 16) {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) dma16(a_base, a_off[i], sbase + (uint32_t)i * (WAVES * 1024u));
#pragma unroll
            for (int i = 0; i < B_LOADS; ++i) dma16(b_base, b_off[i], sbase + A_FLOATS * 4u + (uint32_t)i * (WAVES * 1024u));
        } else {
#pragma unroll
            for (int i = 0; i < A_LOADS * SUB; ++i)
                dma4(a_base, a_off[i], sbase + (uint32_t)(i / SUB) * (WAVES * 1024u) + (uint32_t)(i % SUB) * 256u);
#pragma unroll
            for (int i = 0; i < B_LOADS * SUB; ++i)
                dma4(b_base, b_off[i], sbase + A_FLOATS * 4u + (uint32_t)(i / SUB) * (WAVES * 1024u) + (uint32_t)(i % SUB) * 256u);
        }
        a_base += a_step;
        b_base += b_step;
    };

    // ---- the last slab when K is not a multiple of 16: krem = K % 16 of its k values exist ----
    // Chunks (k-contiguous operand) or rows of k (m-contiguous) that lie wholly beyond K are fetched from
    // the last existing one instead; once a wavefront's own loads of that slab have landed it writes
    // zeros over every float of its share whose k does not exist (products with them must vanish).
    const uint32_t krem = !SK || ke * BK >= g.K ? g.K % BK : 0u; // (a range that ends inside the tile has whole slabs only)
    // k of the float that lane `lane` of load q of group grp fetches with one float per lane (VB = 4)
    auto k_of_float = [&](int grp, int q, auto kc_tag, auto rows_tag) -> uint32_t {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        const uint32_t f = 64 * q + lane;
        if constexpr (KC) {
            const uint32_t row = grp * (256 / BK) + f / BK, pos = f % BK;
            return 4 * ((pos >> 2) ^ swizzle(row)) + (pos & 3);
        } else {
            return grp * (256 / ROWS) + f / ROWS;
        }
    };
    auto tail_offset = [&](uint32_t off, int grp, int q, uint32_t ld, auto kc_tag, auto rows_tag) -> uint32_t {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        if constexpr (VB == 4) { // a float whose k does not exist: the last existing one of its row (column) instead
            const uint32_t k = k_of_float(grp, q, kc_tag, rows_tag);
            return k >= krem ? off - (k - (krem - 1)) * (KC ? 1u : ld) * 4u : off;
        } else if constexpr (KC) {
            const uint32_t row = grp * (64 / CPR) + lane / CPR;
            const uint32_t chunk = (lane % CPR) ^ swizzle(row);
            return 4 * chunk >= krem ? off - 16u * chunk : off; // chunk 0 of the row always has a float (krem >= 1)
        } else {
            constexpr int PER_ROW = ROWS / 4;
            const uint32_t k = grp * (64 / PER_ROW) + lane / PER_ROW;
            return k >= krem ? off - (k - (krem - 1)) * ld * 4u : off;
        }
    };
    auto tail_offsets = [&]() {
#pragma unroll
        for (int i = 0; i < A_LOADS * SUB; ++i)
            a_off[i] = tail_offset(a_off[i], (i / SUB) * WAVES + wave, i % SUB, g.lda, integral_constant<bool, A_K>{}, integral_constant<int, BM>{});
#pragma unroll
        for (int i = 0; i < B_LOADS * SUB; ++i)
            b_off[i] = tail_offset(b_off[i], (i / SUB) * WAVES + wave, i % SUB, g.ldb, integral_constant<bool, B_K>{}, integral_constant<int, BN>{});
    };
    auto tail_zero = [&](float *dst, int grp, int q, auto kc_tag, auto rows_tag) { // dst: this lane's bytes of the load
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        if constexpr (VB == 4) {
            if (k_of_float(grp, q, kc_tag, rows_tag) >= krem) dst[0] = 0.f;
        } else if constexpr (KC) {
            const uint32_t row = grp * (64 / CPR) + lane / CPR;
            const uint32_t chunk = (lane % CPR) ^ swizzle(row);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (4 * chunk + e >= krem) dst[e] = 0.f;
        } else {
            constexpr int PER_ROW = ROWS / 4;
            const uint32_t k = grp * (64 / PER_ROW) + lane / PER_ROW;
            if (k >= krem) *reinterpret_cast<f32x4 *>(dst) = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };
    auto tail_zeros = [&](uint32_t stage_bytes) {
        float *base = lds + stage_bytes / 4 + wave * 256 + lane * (VB / 4);
#pragma unroll
        for (int i = 0; i < A_LOADS * SUB; ++i)
            tail_zero(base + (i / SUB) * (WAVES * 256) + (i % SUB) * 64, (i / SUB) * WAVES + wave, i % SUB, integral_constant<bool, A_K>{},
                      integral_constant<int, BM>{});
#pragma unroll
        for (int i = 0; i < B_LOADS * SUB; ++i)
            tail_zero(base + A_FLOATS + (i / SUB) * (WAVES * 256) + (i % SUB) * 64, (i / SUB) * WAVES + wave, i % SUB,
                      integral_constant<bool, B_K>{}, integral_constant<int, BN>{});
    };

    // ---- LDS side: per-lane fragment addresses (floats from the start of a stage's A or B part) ----
    // k-contiguous: row * BK + 4 * (chunk ^ swz); chunk = 2 s + lhi, swz from l32 alone (row offsets are multiples of 32)
    // m-contiguous: k * ROWS + (m ^ 32 lhi); k = 8 s + 4 lhi + t; m = wave offset + 32 i + l32
    const int sw4 = 4 * (lhi ^ (int)swizzle((uint32_t)l32));
    // A_PERM (m-contiguous A, four blocks per wavefront): lane l32 of block i stands for tile row 4 l32 + i
    // instead of 32 i + l32, so that one 16-byte read (four consecutive m at one k) serves all four blocks;
    // the epilogue maps the rows back.  (16 four-byte reads per step otherwise: T,N and T,T were the slow layouts.)
    constexpr bool A_PERM = !A_K && FM == 4;
    int a_frag[FM], b_frag[FN]; // k-contiguous: one base (block i is an immediate away); m-contiguous: block i's column
#pragma unroll
    for (int i = 0; i < FM; ++i)
        a_frag[i] = A_K      ? (wm * WM + l32) * BK + sw4
                    : A_PERM ? 4 * lhi * BM + ((wm * WM + 4 * l32) ^ (32 * lhi))
                             : 4 * lhi * BM + (((wm * WM + 32 * i) ^ (32 * lhi)) + l32);
#pragma unroll
    for (int j = 0; j < FN; ++j)
        b_frag[j] = B_K ? (wn * WN + l32) * BK + sw4 : 4 * lhi * BN + (((wn * WN + 32 * j) ^ (32 * lhi)) + l32);
    if constexpr (KS > 1) { // group kg starts at step kg * SG of every slab (SG a power of two: the bits do not meet)
#pragma unroll
        for (int i = 0; i < FM; ++i) a_frag[i] = A_K ? a_frag[i] ^ (8 * SG * kg) : a_frag[i] + 8 * SG * kg * BM;
#pragma unroll
        for (int j = 0; j < FN; ++j) b_frag[j] = B_K ? b_frag[j] ^ (8 * SG * kg) : b_frag[j] + 8 * SG * kg * BN;
    }

    auto read_frags = [&](uint32_t stage_bytes, int s, f32x4 *af, f32x4 *bf) {
        const float *as = lds + stage_bytes / 4;
        const float *bs = as + A_FLOATS;
        if constexpr (A_PERM) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(as + a_frag[0] + (8 * s + t) * BM);
#pragma unroll
                for (int i = 0; i < FM; ++i) af[i][t] = v[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                if constexpr (A_K) {
                    // chunk 2 s + lhi: step s flips the bits of 2 s in the chunk number
                    af[i] = *reinterpret_cast<const f32x4 *>(as + ((a_frag[i] ^ (8 * s)) + i * 32 * BK));
                } else {
#pragma unroll
                    for (int t = 0; t < 4; ++t) af[i][t] = as[a_frag[i] + (8 * s + t) * BM];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            if constexpr (B_K) {
                bf[j] = *reinterpret_cast<const f32x4 *>(bs + ((b_frag[j] ^ (8 * s)) + j * 32 * BK));
            } else {
#pragma unroll
                for (int t = 0; t < 4; ++t) bf[j][t] = bs[b_frag[j] + (8 * s + t) * BN];
            }
        }
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    f32x4 af[2][FM], bf[2][FN];
    auto mfma_step = [&](int s) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[s & 1][i][t], bf[s & 1][j][t], acc[i][j], 0, 0, 0);
    };

    const uint32_t ktiles = SK ? ke - kb : (g.K + BK - 1) / BK;

    // The NS stages rotate (byte offsets): st[0] holds the slab being multiplied, st[1] the next one, ...,
    // st[NS - 1] is the stage the slab before left, into which slab kt + NS - 1 is requested.
    constexpr uint32_t STAGE_BYTES = STAGE * 4u;
    constexpr int LOADS = (A_LOADS + B_LOADS) * SUB; // per wavefront and slab
    static_assert(LOADS * (NS - 1) <= 63 || VB == 4, "the wait counter holds 63 loads");
    uint32_t st[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) st[n] = n * STAGE_BYTES;

    // The one-block-per-wavefront tile fetches C_old ahead of everything else (16 registers): its launches
    // are short and the latency of that read at the end of a tile is a visible share of them.  These loads
    // are older than every slab load, so the counted waits below cover them as well.
    constexpr bool PRELOAD_C = FM * FN == 1 && !SK; // (a dealt work-group does not know yet whether it will run its tile's epilogue)
    float c_old[PRELOAD_C ? 16 : 1];
    if constexpr (PRELOAD_C) {
        if (g.epi == EPI_ALPHA_BETA && (KS == 1 || kg == 0)) {
            const uint32_t colc = min(n0 + wn * WN + l32, g.N - 1);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + wm * WM + 8 * (r / 4) + 4 * lhi + (r % 4);
                c_old[r] = g.C[(size_t)min(row, g.M - 1) * g.ldc + colc];
            }
        }
    }

    // prologue: the first NS - 1 slabs on their way, slab 0 landed everywhere, first fragments read
#pragma unroll
    for (int n = 0; n < NS - 1; ++n)
        if ((uint32_t)n < ktiles) {
            if ((uint32_t)n + 1 == ktiles && krem) tail_offsets();
            issue(st[n]);
        }
    wait_vm_slabs<LOADS, NS - 2>(ktiles - 1); // all but the slabs after the first
    if (ktiles == 1 && krem) {
        tail_zeros(st[0]);
        wait_lgkm0();
    }
    __builtin_amdgcn_s_barrier();
    read_frags(st[0], 0, af[0], bf[0]);

    // One iteration on the slab in stage st[0].  ISSUE: slab kt + NS - 1 exists and is requested into the
    // stage that slab kt - 1 left (every wavefront is past the barrier of iteration kt - 1, in front of
    // which it waited for its last reads of that stage).  AHEAD >= 0: slab kt + 1 exists and AHEAD slabs
    // after it have been requested; before the last step's matrix instructions this wavefront waits for
    // its own loads of slab kt + 1 (the AHEAD later ones may stay in flight) and for its LDS reads, joins
    // the barrier and reads the first fragments of slab kt + 1.  AHEAD < 0: the last slab.  LAST_NEXT: slab
    // kt + 1 is the last one (its k values beyond K are overwritten with zeros once it has landed).
    auto iteration = [&](auto issue_tag, auto ahead_tag, auto last_next_tag) __attribute__((always_inline)) {
        constexpr bool ISSUE = decltype(issue_tag)::value;
        constexpr int AHEAD = decltype(ahead_tag)::value;
        constexpr bool LAST_NEXT = decltype(last_next_tag)::value;
        static_assert(!LAST_NEXT || AHEAD == 0, "nothing is requested beyond the last slab");
        if constexpr (ISSUE) issue(st[NS - 1]);
#pragma unroll
        for (int s = 0; s + 1 < SG; ++s) {
            read_frags(st[0], s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
            mfma_step(s);
        }
        if constexpr (AHEAD >= 0) {
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<AHEAD * LOADS>();
            if constexpr (LAST_NEXT) {
                if (krem) tail_zeros(st[1]);
            }
            wait_lgkm0();
            __builtin_amdgcn_s_barrier();
            read_frags(st[1], 0, af[0], bf[0]);
            __builtin_amdgcn_sched_barrier(0);
        }
        mfma_step(SG - 1);
        const uint32_t t = st[0];
#pragma unroll
        for (int n = 0; n + 1 < NS; ++n) st[n] = st[n + 1];
        st[NS - 1] = t;
    };
    using std::integral_constant;
    using T_ = std::true_type;
    using F_ = std::false_type;
    uint32_t kt = 0;
    for (; kt + NS < ktiles; ++kt) iteration(T_{}, integral_constant<int, NS - 2>{}, F_{}); // steady state
    if (kt + NS - 1 < ktiles) { // the iteration that requests the last slab (with two stages: and hands over to it)
        if (krem) tail_offsets();
        iteration(T_{}, integral_constant<int, NS - 2>{}, integral_constant<bool, NS == 2>{});
        ++kt;
    }
    // the pipeline drains: ktiles - 2 - kt slabs are in flight beyond the next one
    drain<NS - 3>([&](auto ahead_tag) {
        if (kt + 2 + decltype(ahead_tag)::value == ktiles) {
            iteration(F_{}, ahead_tag, integral_constant<bool, decltype(ahead_tag)::value == 0>{});
            ++kt;
        }
    });
    iteration(F_{}, integral_constant<int, -1>{}, F_{}); // the last

    // ---- epilogue: acc register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 block;
    // option semantics of src/blas/gemm.zig:500-501,591-602 (C_old is read and multiplied whenever beta
    // is given); the reads of C_old of a block are issued as one batch
    if constexpr (KS > 1) {
        // the partial tile of group 1 goes through LDS to group 0: register r of block (i, j) of wavefront
        // (wm, wn) at float ((4 wm + 2 wn ... ) below, consecutive lanes on consecutive floats
        static_assert(4 * FM * FN * 16 * 64 <= NS * STAGE, "the partial tile fits the stages");
        __builtin_amdgcn_s_barrier(); // every wavefront is done with the stages (its last reads were waited for)
        float *part = lds + ((wave & 3) * FM * FN) * 16 * 64 + lane;
        if (kg == 1) {
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) part[((i * FN + j) * 16 + r) * 64] = acc[i][j][r];
        }
        __syncthreads();
        if (kg == 1) return;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] += part[((i * FN + j) * 16 + r) * 64];
    }
    if constexpr (SK) {
        const uint32_t slabs_per_tile = (g.K + BK - 1) / BK;
        if (!(kb == 0 && ke == slabs_per_tile)) {
            // a part of the tile: to memory in accumulator-register order, 16 bytes per lane (registers 4 q .. 4 q + 3
            // of thread t at (q * 256 + t) * 16 bytes: coalesced; the thread's part of the address in a register, the rest scalar); slot 2 b' holds the part that starts inside the
            // tile, 2 b' + 1 the one that starts it.  Device-scope accesses (the sc1 cache policy, bit 4 of the
            // buffer instructions' auxiliary operand): the parts of a tile come from different XCDs.
            constexpr size_t TILE = (size_t)BM * BN;
            constexpr int SC1 = 16;
            const uint32_t U = g.sk_units, t0 = (pid - g.sk_first) * slabs_per_tile;
            const uint32_t b_first = t0 / U, b_last = (t0 + slabs_per_tile - 1) / U; // the work-groups that hold parts of it
            const uint32_t nparts = b_last - b_first + 1;
            // The part that starts the tile is the last of its work-group's range, so it is usually the last to be
            // ready: when the counter says that all the others have arrived, it stays in the accumulators and the
            // others are added to it in the order of k (no store, no read-back: 0 + p0 + p1 ... and p0 + p1 ... are
            // the same bits).  Otherwise it goes to memory like any other part.
            uint32_t first_part = 0;
            if (kb == 0) {
                if (tid == 0) {
                    const uint32_t arrived = __hip_atomic_load(&g.counters[pid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (arrived == nparts - 1) __hip_atomic_store(&g.counters[pid], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    s_last = arrived == nparts - 1 ? 1u : 0u;
                }
                __syncthreads();
                first_part = s_last;
                __syncthreads(); // (s_last is written again below)
            }
            if (first_part == 0) {
                __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(
                    g.partials + (size_t)(2 * bq + (kb == 0 ? 1u : 0u)) * TILE, 0, (int)(TILE * sizeof(float)), 0x00020000);
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const f32x4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v), mine, tid * 16, ((i * FN + j) * 4 + q) * 4096, SC1);
                        }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (tid == 0) {
                    const uint32_t before = __hip_atomic_fetch_add(&g.counters[pid], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const uint32_t last = before == nparts - 1 ? 1u : 0u;
                    if (last) __hip_atomic_store(&g.counters[pid], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    s_last = last;
                }
                __syncthreads();
                if (!s_last) return;
                // the last to arrive adds the parts up in the order of k, its own read back like the others
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
            }
            // Every round trip to memory costs a few microseconds whatever it carries, so the loads of four
            // blocks of a part (64 registers) are in flight together.
            constexpr int NB = FM * FN < 4 ? FM * FN : 4; // blocks per batch of loads
            static_assert((FM * FN) % NB == 0, "blocks divide into batches");
            for (uint32_t pp = first_part; pp < nparts; ++pp) {
                const uint32_t b2 = b_first + pp;
                __amdgpu_buffer_rsrc_t part = __builtin_amdgcn_make_buffer_rsrc(
                    g.partials + (size_t)(2 * b2 + (pp == 0 ? 1u : 0u)) * TILE, 0, (int)(TILE * sizeof(float)), 0x00020000);
#pragma unroll
                for (int batch = 0; batch < FM * FN / NB; ++batch) {
                    u32x4_t v[NB][4];
#pragma unroll
                    for (int n = 0; n < NB; ++n)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            v[n][q] = __builtin_amdgcn_raw_buffer_load_b128(part, tid * 16, ((batch * NB + n) * 4 + q) * 4096, SC1);
#pragma unroll
                    for (int n = 0; n < NB; ++n) {
                        const int blk = batch * NB + n, i = blk / FN, j = blk % FN;
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const f32x4 f = __builtin_bit_cast(f32x4, v[n][q]);
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] += f[e];
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0); // (one batch of loads at a time)
                }
            }
        }
    }
    // row of the wavefront's tile that output row `rho` of block i holds
    auto tile_row = [](int i, int rho) -> uint32_t { return A_PERM ? (uint32_t)(4 * rho + i) : (uint32_t)(32 * i + rho); };
    // Tiles that reach beyond C clamp the addresses of C_old and the bias and skip the stores there.
    const float alpha = g.alpha, beta = g.beta;
    auto epilogue = [&](auto checked_tag) {
        constexpr bool CHECKED = decltype(checked_tag)::value;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const uint32_t col = n0 + wn * WN + j * 32 + l32;
                const uint32_t colc = CHECKED ? min(col, g.N - 1) : col;
                float bias_v = 0.f;
                if constexpr (EXT) {
                    if (g.bias) bias_v = g.bias[colc];
                }
                float old[16];
                if (g.epi == EPI_ALPHA_BETA) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t row = m0 + wm * WM + tile_row(i, 8 * (r / 4) + 4 * lhi + (r % 4));
                        if constexpr (PRELOAD_C) old[r] = c_old[r];
                        else old[r] = g.C[(size_t)(CHECKED ? min(row, g.M - 1) : row) * g.ldc + colc];
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = m0 + wm * WM + tile_row(i, 8 * (r / 4) + 4 * lhi + (r % 4));
                    float v = acc[i][j][r];
                    if (g.epi == EPI_ALPHA) v = alpha * v;
                    else if (g.epi == EPI_ALPHA_BETA) v = alpha * v + beta * old[r];
                    if constexpr (EXT) { // the fused epilogue of Linear.forward, as in wk_gemm_mfma.hip
                        if (g.bias) v += bias_v;
                        v = act_forward<float>(g.act, v);
                    }
                    if (!CHECKED || (row < g.M && col < g.N)) g.C[(size_t)row * g.ldc + col] = v;
                }
            }
    };
    if (m0 + BM <= g.M && n0 + BN <= g.N) epilogue(std::false_type{});
    else epilogue(std::true_type{});
    }; // run
    if constexpr (!SK) {
        // One work-group per tile, or -- a launch of more tiles than are resident at once -- as many work-groups as
        // are resident, each taking every gridDim.x-th tile in turn: which unit a late tile lands on is then fixed
        // here (every unit's work-groups get the same share) instead of left to the order in which slots come free.
        for (uint32_t pid = blockIdx.x; pid < g.tiles_run; pid += gridDim.x) {
            next_tile(pid != blockIdx.x);
            run(pid, 0u, 0u, 0u);
        }
    } else {
        const uint32_t slabs_per_tile = (g.K + BK - 1) / BK;
        bool first = true;
        // Every tile dealt: all work-groups take a run of k-slabs.  Whole rounds run whole: the launch is `slots`
        // work-groups per unit (work-group b sits on unit b % units, slot b / units: they are placed breadth
        // first); slot 0 takes the unit's run of k-slabs first, and the unit's whole tiles -- tile c + units * j for
        // j = 0 ... rounds - 1 -- go to the slots in turn, starting with slot 1, so that every unit's slots end up
        // with the same amount of work.
        const uint32_t units = g.sk_groups;
        const uint32_t slot = g.sk_first ? blockIdx.x / units : 0u;
        if (slot == 0) {
            // work-groups b, b + 8, ... share an XCD: they take consecutive ranges, and with them neighbouring tiles
            const uint32_t bq = (blockIdx.x & 7u) * (g.sk_groups >> 3) + (blockIdx.x >> 3);
            uint32_t u = bq * g.sk_units;
            const uint32_t u_end = min(u + g.sk_units, g.sk_total);
            while (u < u_end) {
                const uint32_t t = u / slabs_per_tile, kb = u - t * slabs_per_tile;
                const uint32_t ke = min(slabs_per_tile, kb + (u_end - u));
                next_tile(!first);
                run(g.sk_first + t, kb, ke, bq);
                first = false;
                u += ke - kb;
            }
        }
        if (g.sk_first) {
            // tile c + units * j for j = slot - 1 (mod slots), slot - 1 + slots, ...: every gridDim.x-th tile
            const uint32_t slots = gridDim.x / units;
            for (uint32_t pid = blockIdx.x - slot * units + units * ((slot + slots - 1) % slots); pid < g.sk_first; pid += gridDim.x) {
                next_tile(!first);
                run(pid, 0u, (g.K + BK - 1) / BK, 0u);
                first = false;
            }
        }
    }
}

// grid: the work-groups of the launch (one per tile of g.tiles_run, or fewer: they then take the tiles in turn;
// kernels that deal k-slabs: as their plan says)
template <int BM, int BN, int BK, int NS, int OCC, bool A_K, bool B_K, bool EXT, int KS = 1, int VB = 16, bool SK = false>
int launch_one(hipStream_t st, const DArgs &g, unsigned grid) {
    constexpr size_t lds_bytes = NS * (BM * BK + BN * BK) * sizeof(float); // 3 x 24 KB / 3 x 16 KB / 3 x 32 KB
    auto kern = gemm_f32_dma_kernel<BM, BN, BK, NS, OCC, A_K, B_K, EXT, KS, VB, SK>;
    static const int attr_rc = [&] {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)lds_bytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return hip_code(e);
        }
        return (int)WK_OK;
    }();
    if (attr_rc) return attr_rc;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256 * KS), lds_bytes, st, g);
    return launch_status();
}

template <int BM, int BN, int BK, int NS, int OCC, int KS = 1, int VB = 16, bool SK = false> int launch_tile(hipStream_t st, const GemmProblem &p, uint64_t first_tiles) {
    if (first_tiles > ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN)) return WK_E_INVALID_VALUE;
    DArgs g{};
    g.A = static_cast<const float *>(p.A);
    g.B = static_cast<const float *>(p.B);
    g.C = static_cast<float *>(p.C);
    g.M = (uint32_t)p.M; g.N = (uint32_t)p.N; g.K = (uint32_t)p.K;
    g.lda = (uint32_t)p.lda; g.ldb = (uint32_t)p.ldb; g.ldc = (uint32_t)p.ldc;
    g.tiles_m = (uint32_t)((p.M + BM - 1) / BM);
    g.tiles_n = (uint32_t)((p.N + BN - 1) / BN);
    g.epi = p.epi;
    std::memcpy(&g.alpha, p.alpha, sizeof(float));
    std::memcpy(&g.beta, p.beta, sizeof(float));
    g.bias = static_cast<const float *>(p.ext_bias);
    g.act = p.ext_act;
    // XCD-local patches where the tile grid divides into them, eight patches at a time (one per XCD);
    // the k-split tail numbers its tiles in the row-group order, so a body launch keeps that order
    const bool row_walk = g_test_options.gemm_walk_rows != 0;
    if (!first_tiles && !row_walk) {
        static const unsigned shapes[][2] = {{4, 8}, {4, 4}, {2, 8}, {2, 4}};
        for (const auto &sh : shapes)
            if (g.tiles_m % sh[0] == 0 && g.tiles_n % sh[1] == 0 && ((g.tiles_m / sh[0]) * (g.tiles_n / sh[1])) % 8 == 0) {
                g.patch_m = sh[0];
                g.patch_n = sh[1];
                break;
            }
    }
    const int sel = (p.op_a ? 0 : 2) | (p.op_b ? 1 : 0); // bit 1: A k-contiguous, bit 0: B k-contiguous
    g.tiles_run = first_tiles ? (uint32_t)first_tiles : g.tiles_m * g.tiles_n;
    // Between one and two rounds of what is resident at once (units x OCC work-groups): that many work-groups, each
    // taking every grid-th tile in turn.  Left to the dispatcher, the tiles of the second round go where slots come
    // free first, and when the work-groups of a unit finish close together it puts two or three of them on one unit
    // and none on others: 64 x 64 T,N at 2048 x 2048 x 2048 (1024 tiles on 768 slots) 109 TFLOP/s against 133 this way,
    // 1536 x 2560 x 2048 107 / 126, f64 128 x 128 at 3400^3 49 / 63.  Whole rounds and longer launches are left as they
    // are (8192^3 147 against 146 this way, 64 x 64 at 3000^3 128 / 125).
    const unsigned resident = g_test_options.persistent && KS == 1 ? p.num_cus * (unsigned)OCC : 0u;
    unsigned grid = resident && g.tiles_run > resident && (g.tiles_run < 2 * resident || g_test_options.persistent == 2) ? resident : g.tiles_run;
    if constexpr (SK) {
        unsigned sk_groups = 0;
        if (first_tiles || !gemm_dma_stream_k_plan(p, BM, BN, BK, OCC, sk_groups, g.sk_units, g.sk_total, g.sk_first)) return WK_E_INVALID_VALUE;
        g.sk_groups = sk_groups;
        // whole rounds run whole: one dealt work-group per unit and up to OCC - 1 more for the whole tiles
        const unsigned rounds = g.sk_first / sk_groups;
        grid = g.sk_first ? sk_groups * std::min<unsigned>((unsigned)OCC, rounds + 1) : sk_groups;
        g.partials = static_cast<float *>(p.scratch);
        g.counters = p.counters;
        g.patch_m = g.patch_n = 0; // consecutive tile numbers are neighbours in the row-group walk
    }
    if (p.ext) { // instantiated for op N, T only (what Linear.forward runs), one group of wavefronts, aligned rows
        if constexpr (KS == 1 && VB == 16)
            return sel == 3 ? launch_one<BM, BN, BK, NS, OCC, true, true, true, 1, 16, SK>(st, g, grid) : (int)WK_E_INVALID_VALUE;
        else
            return WK_E_INVALID_VALUE;
    }
    switch (sel) {
    case 0: return launch_one<BM, BN, BK, NS, OCC, false, false, false, KS, VB, SK>(st, g, grid);
    case 1: return launch_one<BM, BN, BK, NS, OCC, false, true, false, KS, VB, SK>(st, g, grid);
    case 2: return launch_one<BM, BN, BK, NS, OCC, true, false, false, KS, VB, SK>(st, g, grid);
    default: return launch_one<BM, BN, BK, NS, OCC, true, true, false, KS, VB, SK>(st, g, grid);
    }
}

// rows of both operands start on 16-byte boundaries: 16 bytes per lane and load; otherwise 4
bool f32_rows_aligned(const GemmProblem &p) {
    return p.lda % 4 == 0 && p.ldb % 4 == 0 && ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15u) == 0;
}

} // namespace

// How the work-groups of a launch that deals its work by k-slabs share it.  With at least as many tiles as
// compute units, the whole rounds of tiles (one tile per unit and round) are run whole, one work-group each, and
// only the k-slabs of the tiles that are left are dealt, to one work-group per unit: every unit then has the same
// amount of matrix work, few tiles are split, and the dealt work-groups -- the first of the launch, so the first to
// start -- are done and their parts added up while the whole tiles are still being multiplied.  With fewer tiles
// than units (or with the test option "stream_k" at 2) all tiles are dealt, to as many work-groups as are
// resident at once (units x occ).  groups: the work-groups that take dealt k-slabs (a multiple of eight), units
// = ceil(dealt tiles x slabs per tile / groups) slabs each, first: the number of tiles run whole.  false: the
// problem does not fit (no scratch for two partial tiles per dealt work-group, more tiles than counters,
// 32-bit slab numbers).
bool wk::gemm_dma_stream_k_plan(const GemmProblem &p, int bm, int bn, int bk, int occ, unsigned &groups, uint32_t &units, uint32_t &total,
                                uint32_t &first) {
    const size_t elem = p.dtype == WK_F64 ? sizeof(double) : sizeof(float);
    const uint64_t tiles = ((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn), slabs = (p.K + bk - 1) / bk;
    const uint64_t cus = p.num_cus ? p.num_cus : 256;
    uint64_t whole = g_test_options.stream_k == 2 || tiles < cus ? 0 : tiles / cus * cus;
    if (whole == tiles) whole -= cus; // (a launch of whole rounds has no use for this: deal the last round)
    groups = (unsigned)(whole ? cus : cus * occ);
    if (groups % 8 || !p.scratch || !p.counters || tiles > p.num_counters || tiles * slabs > 0x7fffffffull) return false;
    if ((uint64_t)2 * groups * bm * bn * elem > p.scratch_bytes) return false;
    first = (uint32_t)whole;
    total = (uint32_t)((tiles - whole) * slabs);
    units = (uint32_t)(((tiles - whole) * slabs + groups - 1) / groups);
    return units >= 1;
}


// What the kernels take for granted, checked on the host: element-aligned operands (rows that start on 16-byte
// boundaries get 16-byte loads, any other 4-byte ones), every per-lane byte offset inside 32 bits, and for the
// fused epilogue the one layout and the alignment it exists for.
bool wk::gemm_f32_dma_applies(const GemmProblem &p, int bm, int bn) {
    if (p.dtype != WK_F32) return false;
    if (!((bm == 256 && bn == 128) || (bm == 128 && bn == 128) || (bm == 64 && bn == 64))) return false;
    if (p.ext && (p.op_a || !p.op_b || !f32_rows_aligned(p))) return false;
    if (!p.M || !p.N || !p.K) return false;
    if ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 3u) return false;
    if (p.M > 0x7fffffffull || p.N > 0x7fffffffull || p.K > 0x7fffffffull || p.ldc > 0x7fffffffull) return false;
    // offsets reach 255 rows (k-contiguous) or 15 rows of k (m-contiguous) past the tile's origin
    if (p.lda > (1ull << 21) || p.ldb > (1ull << 21)) return false;
    if (((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) > 0x7fffffffull) return false;
    return true;
}

// rows of A and B start on 16-byte boundaries (16-byte loads; the two-group and fused kernels exist for these only)
bool wk::gemm_dma_rows_aligned(const GemmProblem &p) { return p.dtype == WK_F64 ? gemm_f64_rows_aligned(p) : f32_rows_aligned(p); }

bool wk::gemm_f32_dma_stream_k_applies(const GemmProblem &p, int bm, int bn) {
    if (!gemm_f32_dma_applies(p, bm, bn) || !f32_rows_aligned(p) || p.ext) return false;
    unsigned groups;
    uint32_t units, total, first;
    return gemm_dma_stream_k_plan(p, bm, bn, bm == 64 ? 32 : 16, bm == 256 ? 2 : 3, groups, units, total, first);
}

int wk::gemm_f32_dma_stream_k_launch(hipStream_t st, const GemmProblem &p, int bm, int bn) {
    if (!gemm_f32_dma_stream_k_applies(p, bm, bn)) return WK_E_INVALID_VALUE;
    if (bm == 256) return launch_tile<256, 128, 16, 3, 2, 1, 16, true>(st, p, 0);
    if (bm == 64) return launch_tile<64, 64, 32, 3, 3, 1, 16, true>(st, p, 0);
    return launch_tile<128, 128, 16, 3, 3, 1, 16, true>(st, p, 0);
}

int wk::gemm_f32_dma_launch(hipStream_t st, const GemmProblem &p, int bm, int bn, uint64_t first_tiles, int k_groups) {
    if (!gemm_f32_dma_applies(p, bm, bn)) return WK_E_INVALID_VALUE;
    if (k_groups == 2 && f32_rows_aligned(p)) { // eight wavefronts per tile, k-slabs of 32 (128 x 128: one work-group per unit, 96 KB of stages)
        // (the 256 x 128 tile with two groups, 144 KB of stages, measured no better than two work-groups of the
        // 128 x 128 tile where it would apply: 2048 x 4096 x 4096 143 against 143 TFLOP/s, 4096 x 2048 x 2048 138 against 139)
        if (p.ext || first_tiles || bm == 256) return WK_E_INVALID_VALUE;
        if (bm == 128) return launch_tile<128, 128, 32, 3, 2, 2>(st, p, 0);
        // (four, six and eight stages instead of three, for a lone work-group per unit: 1024^3, 1000^3 and
        // 1024 x 1024 x 4096 all within 1 % of three, every layout)
        return launch_tile<64, 64, 32, 3, 4, 2>(st, p, 0);
    }
    if (!f32_rows_aligned(p)) { // one float per lane and load; one group of wavefronts
        if (bm == 256) return launch_tile<256, 128, 16, 3, 2, 1, 4>(st, p, first_tiles);
        if (bm == 128) return launch_tile<128, 128, 16, 3, 3, 1, 4>(st, p, first_tiles);
        return launch_tile<64, 64, 32, 3, 3, 1, 4>(st, p, first_tiles);
    }
    if (bm == 256) return launch_tile<256, 128, 16, 3, 2>(st, p, first_tiles);
    // 128 x 128 with both operands m/n-contiguous (T,N): k-slabs of 32 in two stages, two work-groups per unit
    // (half as many hand-overs; 2048 x 4096 x 4096 139 -> 143 TFLOP/s, 4096 x 2048 x 2048 135 -> 140, 2048 x 2048 x
    // 8192 129 -> 138; the other layouts measured the same or up to 2 % less that way and keep three stages of 16)
    if (bm == 128 && p.op_a && !p.op_b) return launch_tile<128, 128, 32, 2, 2>(st, p, first_tiles);
    if (bm == 128) return launch_tile<128, 128, 16, 3, 3>(st, p, first_tiles);
    // (k-slabs of 32, three work-groups per unit; with slabs of 16 and four: 1024^3 101 against 103.5 TFLOP/s,
    // 3000^3 118 against 125, 2049 x 2047 x 2050 108 against 106.5)
    // Deeper pipelines were measured for this tile and gave nothing: four stages (two work-groups per unit)
    // and five (one) 1024^3 101-104 TFLOP/s like three, 1536^3 95 against 98; six stages of 16: 90-100.
    // Two stages instead of three (three or four work-groups per unit) and k-slabs of 64 in two stages (two per
    // unit) all measured within 2 % of this on 1536^3 ... 4097 x 4095 x 4093, in both directions.
    return launch_tile<64, 64, 32, 3, 3>(st, p, first_tiles);
}
