// f64 GEMM kernels that bring their k-slabs from global memory straight into LDS: the pipeline of
// wk_gemm_dma.hip (see there for the loads, the waits, the swizzled layouts and the ragged shapes) with
// v_mfma_f64_16x16x4_f64.
#include "wk_internal.hpp"
#include "wk_lds_dma.hpp"

#include <cstdlib>
#include <cstring>

using namespace wk;
using namespace wk::lds_dma;

namespace {

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int GROUP_M = 8;

// ------------------------------------------------------------------------------------ f64 ---
// The same pipeline with v_mfma_f64_16x16x4_f64 (lane l supplies A[l % 16][l / 16] and B[l / 16][l % 16];
// result register r of lane l is C[4 r + l / 16][l % 16] of its 16 x 16 block).  A 16-byte chunk is two
// doubles.  k-slabs of 16 (two fragment steps).  Macro tiles 64 x 64 (three stages of 16 KB, three
// work-groups per unit) and 128 x 128 (two work-groups per unit: 128 accumulator and 64 fragment registers
// do not fit the 168 of three; two stages of 32 KB, the next slab requested at the top of an iteration into
// the stage the hand-over before it set free -- one iteration of 64 matrix instructions of 64 clocks, beside
// the other work-group's, is time enough for it to arrive.  With slabs of 8 in three stages the hand-over came
// twice as often: 4096^3 70.7 against 72.3 TFLOP/s, 8192^3 72.0 against 74.2).
//   k-contiguous operand: [row][16], 8 chunks per row, chunk c of row r at position c ^ ((r >> 1) & 7); a
//     fragment is one 16-byte read (row = lane % 16, k = 8 s + 2 (lane / 16) + 0..1), sixteen consecutive rows
//     at one logical chunk cover all banks once.
//   m/n-contiguous operand: [k][ROWS], element (k, m) at m ^ (16 * ((k >> 1) & 1)); fragments are 8-byte
//     reads, the four quarter-wavefronts read rows k, k + 2, k + 4, k + 6 and the swizzle puts
//     neighbouring quarters on disjoint banks.
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef double f64x4 __attribute__((ext_vector_type(4)));

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

struct DArgsD {
    const double *A, *B;
    double *C;
    uint32_t M, N, K;
    uint32_t lda, ldb, ldc;
    uint32_t tiles_m, tiles_n;
    int epi;
    double alpha, beta;
    const double *bias;
    int act;
    uint32_t patch_m, patch_n; // as in DArgs
    // kernels instantiated with SK (work dealt by k-slabs), as in DArgs
    uint32_t sk_units, sk_total, sk_first, sk_groups;
    // tiles of this launch (one work-group each, or fewer work-groups that take every gridDim.x-th tile in turn)
    uint32_t tiles_run;
    double *partials;
    uint32_t *counters;
};


// VB as in the f32 kernel: 16 bytes per lane and load for rows that start on 16-byte boundaries, 4 (half a
// double) for any other.  SK as in the f32 kernel: the whole rounds of tiles run whole, the k-slabs of the tiles
// that are left are dealt to the first work-groups of the launch, and the parts of a split tile meet in memory.
template <int BM, int BN, int BK, int NS, int OCC, bool A_K, bool B_K, bool EXT, int VB = 16, bool SK = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC)))
void gemm_f64_dma_kernel(DArgsD g) {
    static_assert(NS == 2 || NS == 3, "stages");
    static_assert(VB == 16 || VB == 4, "bytes per lane");
    constexpr int SUB = 16 / VB;
    __shared__ uint32_t s_last;
    auto run = [&](const uint32_t pid, const uint32_t kb, const uint32_t ke, const uint32_t bq) __attribute__((always_inline)) {
    constexpr int WM = BM / 2, WN = BN / 2, FM = WM / 16, FN = WN / 16;
    constexpr int S = BK / 8;     // fragment steps per slab (8 values of k each, two matrix instructions per block)
    constexpr int CPR = BK / 2;   // 16-byte chunks per row of a k-contiguous slab
    constexpr int A_DOUBLES = BM * BK, B_DOUBLES = BN * BK, STAGE = A_DOUBLES + B_DOUBLES;
    constexpr int A_LOADS = BM * BK / 512, B_LOADS = BN * BK / 512; // 1 KB = 128 doubles per wavefront and load
    static_assert(BK == 16 && BM % 32 == 0 && BN % 32 == 0 && A_LOADS >= 1 && B_LOADS >= 1, "tile shape");

    extern __shared__ __align__(16) float lds_f[];
    double *lds = reinterpret_cast<double *>(lds_f); // [NS][STAGE]: A then B

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, lq = lane >> 4;

    uint32_t tile_m, tile_n;
    if (g.patch_m) { // XCD-local patches, as in the f32 kernel
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

    // ---- global side ----
    // Ragged shapes as in the f32 kernel: rows (columns) beyond the matrix are fetched from its last one, a
    // 16-byte chunk whose first double exists is fetched whole; `last` counts from the tile's origin.
    const double *a_base = A_K ? g.A + (size_t)m0 * g.lda : g.A + m0;
    const double *b_base = B_K ? g.B + (size_t)n0 * g.ldb : g.B + n0;
    const size_t a_step = A_K ? (size_t)BK : (size_t)BK * g.lda;
    const size_t b_step = B_K ? (size_t)BK : (size_t)BK * g.ldb;
    if constexpr (SK) { // this range starts at slab kb of the tile
        a_base += kb * a_step;
        b_base += kb * b_step;
    }
    uint32_t a_off[A_LOADS * SUB], b_off[B_LOADS * SUB];
    // (k, row or column) of the double that lane `lane` of load q of group grp fetches half of with four bytes
    // per lane: the double that belongs at double 32 q + lane / 2 of the group
    auto double_of = [&](int grp, int q, uint32_t &k, uint32_t &r, auto kc_tag, auto rows_tag) {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        const uint32_t f = 32 * q + (lane >> 1);
        if constexpr (KC) {
            r = grp * (128 / BK) + f / BK;
            const uint32_t pos = f % BK;
            k = 2 * ((pos >> 1) ^ ((r >> 1) & 7)) + (pos & 1);
        } else {
            k = grp * (128 / ROWS) + f / ROWS;
            r = (f % ROWS) ^ (((k >> 1) & 1) * 16);
        }
    };
    auto lane_offset = [&](int grp, int q, uint32_t ld, uint32_t last, auto kc_tag, auto rows_tag) -> uint32_t {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        if constexpr (VB == 4) {
            uint32_t k, r;
            double_of(grp, q, k, r, kc_tag, rows_tag);
            return (KC ? min(r, last) * ld + k : k * ld + min(r, last)) * 8u + 4u * (lane & 1);
        } else if constexpr (KC) {
            constexpr int RPL = 64 / CPR; // rows per load
            const uint32_t row = grp * RPL + lane / CPR;
            const uint32_t swz = (row >> 1) & 7;
            const uint32_t chunk = (lane % CPR) ^ swz;
            return (min(row, last) * ld + 2 * chunk) * 8u;
        } else {
            constexpr int PER_ROW = ROWS / 2; // chunks per row of k
            static_assert(PER_ROW <= 64, "a row of k is at most one load");
            const uint32_t k = grp * (64 / PER_ROW) + lane / PER_ROW;
            const uint32_t chunk = (lane % PER_ROW) ^ (((k >> 1) & 1) * 8);
            return (k * ld + 2 * min(chunk, last >> 1)) * 8u;
        }
    };
    using std::integral_constant;
    const uint32_t m_last = g.M - 1 - m0, n_last = g.N - 1 - n0;
#pragma unroll
    for (int i = 0; i < A_LOADS * SUB; ++i)
        a_off[i] = lane_offset((i / SUB) * 4 + wave, i % SUB, g.lda, m_last, integral_constant<bool, A_K>{}, integral_constant<int, BM>{});
#pragma unroll
    for (int i = 0; i < B_LOADS * SUB; ++i)
        b_off[i] = lane_offset((i / SUB) * 4 + wave, i % SUB, g.ldb, n_last, integral_constant<bool, B_K>{}, integral_constant<int, BN>{});
    const uint32_t lds0 =
        __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) float *)lds_f);

    auto issue = [&](uint32_t stage_bytes) {
        const uint32_t sbase = lds0 + stage_bytes + (uint32_t)wave * 1024u;
        if constexpr (VB == 16) {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) dma16(a_base, a_off[i], sbase + (uint32_t)i * 4096u);
#pragma unroll
            for (int i = 0; i < B_LOADS; ++i) dma16(b_base, b_off[i], sbase + A_DOUBLES * 8u + (uint32_t)i * 4096u);
        } else {
#pragma unroll
            for (int i = 0; i < A_LOADS * SUB; ++i) dma4(a_base, a_off[i], sbase + (uint32_t)(i / SUB) * 4096u + (uint32_t)(i % SUB) * 256u);
#pragma unroll
            for (int i = 0; i < B_LOADS * SUB; ++i)
                dma4(b_base, b_off[i], sbase + A_DOUBLES * 8u + (uint32_t)(i / SUB) * 4096u + (uint32_t)(i % SUB) * 256u);
        }
        a_base += a_step;
        b_base += b_step;
    };

    // ---- the last slab when K is not a multiple of 16 (krem = K % 16 of its k values exist): chunks or rows
    // of k wholly beyond K are fetched from the last existing one, and the wavefront that loaded a share of
    // that slab writes zeros over its doubles whose k does not exist once the loads have landed ----
    const uint32_t krem = !SK || ke * BK >= g.K ? g.K % BK : 0u; // (a range that ends inside the tile has whole slabs only)
    auto tail_offset = [&](uint32_t off, int grp, int q, uint32_t ld, auto kc_tag, auto rows_tag) -> uint32_t {
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        if constexpr (VB == 4) { // a double whose k does not exist: the last existing one of its row (column) instead
            uint32_t k, r;
            double_of(grp, q, k, r, kc_tag, rows_tag);
            return k >= krem ? off - (k - (krem - 1)) * (KC ? 1u : ld) * 8u : off;
        } else if constexpr (KC) {
            const uint32_t row = grp * (64 / CPR) + lane / CPR;
            const uint32_t chunk = (lane % CPR) ^ ((row >> 1) & 7);
            return 2 * chunk >= krem ? off - 16u * chunk : off; // chunk 0 of the row always has a double (krem >= 1)
        } else {
            constexpr int PER_ROW = ROWS / 2;
            const uint32_t k = grp * (64 / PER_ROW) + lane / PER_ROW;
            return k >= krem ? off - (k - (krem - 1)) * ld * 8u : off;
        }
    };
    auto tail_offsets = [&]() {
#pragma unroll
        for (int i = 0; i < A_LOADS * SUB; ++i)
            a_off[i] = tail_offset(a_off[i], (i / SUB) * 4 + wave, i % SUB, g.lda, integral_constant<bool, A_K>{}, integral_constant<int, BM>{});
#pragma unroll
        for (int i = 0; i < B_LOADS * SUB; ++i)
            b_off[i] = tail_offset(b_off[i], (i / SUB) * 4 + wave, i % SUB, g.ldb, integral_constant<bool, B_K>{}, integral_constant<int, BN>{});
    };
    auto tail_zero = [&](float *dst, int grp, int q, auto kc_tag, auto rows_tag) { // dst: this lane's bytes of the load
        constexpr bool KC = decltype(kc_tag)::value;
        constexpr int ROWS = decltype(rows_tag)::value;
        if constexpr (VB == 4) {
            uint32_t k, r;
            double_of(grp, q, k, r, kc_tag, rows_tag);
            if (k >= krem) dst[0] = 0.f; // (its half of the double)
        } else if constexpr (KC) {
            const uint32_t row = grp * (64 / CPR) + lane / CPR;
            const uint32_t chunk = (lane % CPR) ^ ((row >> 1) & 7);
#pragma unroll
            for (int e = 0; e < 2; ++e)
                if (2 * chunk + e >= krem) reinterpret_cast<double *>(dst)[e] = 0.0;
        } else {
            constexpr int PER_ROW = ROWS / 2;
            const uint32_t k = grp * (64 / PER_ROW) + lane / PER_ROW;
            if (k >= krem) *reinterpret_cast<f64x2 *>(dst) = f64x2{0.0, 0.0};
        }
    };
    auto tail_zeros = [&](uint32_t stage_bytes) {
        float *base = lds_f + stage_bytes / 4 + wave * 256 + lane * (VB / 4);
#pragma unroll
        for (int i = 0; i < A_LOADS * SUB; ++i)
            tail_zero(base + (i / SUB) * 1024 + (i % SUB) * 64, (i / SUB) * 4 + wave, i % SUB, integral_constant<bool, A_K>{},
                      integral_constant<int, BM>{});
#pragma unroll
        for (int i = 0; i < B_LOADS * SUB; ++i)
            tail_zero(base + A_DOUBLES * 2 + (i / SUB) * 1024 + (i % SUB) * 64, (i / SUB) * 4 + wave, i % SUB,
                      integral_constant<bool, B_K>{}, integral_constant<int, BN>{});
    };

    // ---- LDS side: per-lane fragment addresses in doubles from the start of a stage's A or B part ----
    // k-contiguous: row * BK + 2 * ((4 s + lq) ^ swz(row)); row = wave offset + 16 i + l16, so swz depends on l16 only
    const int swz_l = (l16 >> 1) & 7;
    int a_frag[FM], b_frag[FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
        a_frag[i] = A_K ? (wm * WM + 16 * i + l16) * BK + 2 * (lq ^ swz_l) : 2 * lq * BM + (((wm * WM + 16 * i) ^ (16 * (lq & 1))) + l16);
#pragma unroll
    for (int j = 0; j < FN; ++j)
        b_frag[j] = B_K ? (wn * WN + 16 * j + l16) * BK + 2 * (lq ^ swz_l) : 2 * lq * BN + (((wn * WN + 16 * j) ^ (16 * (lq & 1))) + l16);

    auto read_frags = [&](uint32_t stage_bytes, int s, f64x2 *af, f64x2 *bf) {
        const double *as = lds + stage_bytes / 8;
        const double *bs = as + A_DOUBLES;
#pragma unroll
        for (int i = 0; i < FM; ++i) {
            if constexpr (A_K) {
                // chunk 4 s + lq: the second step's chunk has bit 2 flipped
                af[i] = *reinterpret_cast<const f64x2 *>(as + (a_frag[i] ^ (8 * s)));
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t) af[i][t] = as[a_frag[i] + (8 * s + t) * BM];
            }
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            if constexpr (B_K) {
                bf[j] = *reinterpret_cast<const f64x2 *>(bs + (b_frag[j] ^ (8 * s)));
            } else {
#pragma unroll
                for (int t = 0; t < 2; ++t) bf[j][t] = bs[b_frag[j] + (8 * s + t) * BN];
            }
        }
    };

    f64x4 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0;

    // fragment sets alternate from step to step; a slab has an even number of steps, so its first uses set 0
    f64x2 af[2][FM], bf[2][FN];
    auto mfma_step = [&](int set) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[set][i][t], bf[set][j][t], acc[i][j], 0, 0, 0);
    };

    // The stages rotate and the slabs are requested, waited for and handed over exactly as in the f32 kernel
    // (see there): st[0] holds the slab being multiplied, slab kt + NS - 1 goes into st[NS - 1].
    const uint32_t ktiles = SK ? ke - kb : (g.K + BK - 1) / BK;
    constexpr uint32_t STAGE_BYTES = STAGE * 8u;
    constexpr int LOADS = (A_LOADS + B_LOADS) * SUB;
    uint32_t st[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) st[n] = n * STAGE_BYTES;

#pragma unroll
    for (int n = 0; n < NS - 1; ++n)
        if ((uint32_t)n < ktiles) {
            if ((uint32_t)n + 1 == ktiles && krem) tail_offsets();
            issue(st[n]);
        }
    wait_vm_slabs<LOADS, NS - 2>(ktiles - 1);
    if (ktiles == 1 && krem) {
        tail_zeros(st[0]);
        wait_lgkm0();
    }
    __builtin_amdgcn_s_barrier();
    read_frags(st[0], 0, af[0], bf[0]);

    auto iteration = [&](auto issue_tag, auto ahead_tag, auto last_next_tag) __attribute__((always_inline)) {
        constexpr bool ISSUE = decltype(issue_tag)::value;
        constexpr int AHEAD = decltype(ahead_tag)::value;
        constexpr bool LAST_NEXT = decltype(last_next_tag)::value;
        static_assert(!LAST_NEXT || AHEAD == 0, "nothing is requested beyond the last slab");
        if constexpr (ISSUE) issue(st[NS - 1]);
#pragma unroll
        for (int s = 0; s + 1 < S; ++s) {
            read_frags(st[0], s + 1, af[(s + 1) & 1], bf[(s + 1) & 1]);
            mfma_step(s & 1);
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
        mfma_step((S - 1) & 1);
        const uint32_t t = st[0];
#pragma unroll
        for (int n = 0; n + 1 < NS; ++n) st[n] = st[n + 1];
        st[NS - 1] = t;
    };
    using T_ = std::true_type;
    using F_ = std::false_type;
    uint32_t kt = 0;
    for (; kt + NS < ktiles; ++kt) iteration(T_{}, integral_constant<int, NS - 2>{}, F_{}); // steady state
    if (kt + NS - 1 < ktiles) { // the iteration that requests the last slab (with two stages: and hands over to it)
        if (krem) tail_offsets();
        iteration(T_{}, integral_constant<int, NS - 2>{}, integral_constant<bool, NS == 2>{});
        ++kt;
    }
    drain<NS - 3>([&](auto ahead_tag) {
        if (kt + 2 + decltype(ahead_tag)::value == ktiles) {
            iteration(F_{}, ahead_tag, integral_constant<bool, decltype(ahead_tag)::value == 0>{});
            ++kt;
        }
    });
    iteration(F_{}, integral_constant<int, -1>{}, F_{}); // the last

    if constexpr (SK) {
        const uint32_t slabs_per_tile = (g.K + BK - 1) / BK;
        if (!(kb == 0 && ke == slabs_per_tile)) {
            // A part of the tile, exchanged as in the f32 kernel: to memory in accumulator-register order, 16 bytes
            // (two doubles) per lane and store, slot 2 b' for the part that starts inside the tile and 2 b' + 1 for
            // the one that starts it; device-scope accesses; the last to arrive adds the parts in the order of k.
            constexpr size_t TILE = (size_t)BM * BN;
            constexpr int SC1 = 16;
            const uint32_t U = g.sk_units, t0 = (pid - g.sk_first) * slabs_per_tile;
            const uint32_t b_first = t0 / U, b_last = (t0 + slabs_per_tile - 1) / U;
            const uint32_t nparts = b_last - b_first + 1;
            uint32_t first_part = 0;
            if (kb == 0) { // the part that starts the tile stays in the registers when all the others have arrived
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
                    g.partials + (size_t)(2 * bq + (kb == 0 ? 1u : 0u)) * TILE, 0, (int)(TILE * sizeof(double)), 0x00020000);
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const f64x2 v = {acc[i][j][2 * h], acc[i][j][2 * h + 1]};
                            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v), mine, tid * 16, ((i * FN + j) * 2 + h) * 4096, SC1);
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
#pragma unroll
                for (int i = 0; i < FM; ++i)
#pragma unroll
                    for (int j = 0; j < FN; ++j)
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0;
            }
            constexpr int NB = FM * FN < 8 ? FM * FN : 8; // blocks per batch of loads (two loads per block)
            static_assert((FM * FN) % NB == 0, "blocks divide into batches");
            for (uint32_t pp = first_part; pp < nparts; ++pp) {
                const uint32_t b2 = b_first + pp;
                __amdgpu_buffer_rsrc_t part = __builtin_amdgcn_make_buffer_rsrc(
                    g.partials + (size_t)(2 * b2 + (pp == 0 ? 1u : 0u)) * TILE, 0, (int)(TILE * sizeof(double)), 0x00020000);
#pragma unroll
                for (int batch = 0; batch < FM * FN / NB; ++batch) {
                    u32x4_t v[NB][2];
#pragma unroll
                    for (int n = 0; n < NB; ++n)
#pragma unroll
                        for (int h = 0; h < 2; ++h)
                            v[n][h] = __builtin_amdgcn_raw_buffer_load_b128(part, tid * 16, ((batch * NB + n) * 2 + h) * 4096, SC1);
#pragma unroll
                    for (int n = 0; n < NB; ++n) {
                        const int blk = batch * NB + n, i = blk / FN, j = blk % FN;
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const f64x2 f = __builtin_bit_cast(f64x2, v[n][h]);
                            acc[i][j][2 * h] += f[0];
                            acc[i][j][2 * h + 1] += f[1];
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0); // (one batch of loads at a time)
                }
            }
        }
    }

    // Tiles that reach beyond C clamp the addresses of C_old and the bias and skip the stores there.
    const double alpha = g.alpha, beta = g.beta;
    auto epilogue = [&](auto checked_tag) {
        constexpr bool CHECKED = decltype(checked_tag)::value;
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
                const uint32_t col = n0 + wn * WN + j * 16 + l16;
                const uint32_t colc = CHECKED ? min(col, g.N - 1) : col;
                double bias_v = 0.;
                if constexpr (EXT) {
                    if (g.bias) bias_v = g.bias[colc];
                }
                double old[4];
                if (g.epi == EPI_ALPHA_BETA) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const uint32_t row = m0 + wm * WM + i * 16 + 4 * r + lq;
                        old[r] = g.C[(size_t)(CHECKED ? min(row, g.M - 1) : row) * g.ldc + colc];
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

// grid: the work-groups of the launch (one per tile, or fewer: they then take the tiles in turn; kernels that deal
// k-slabs: as their plan says)
template <int BM, int BN, int BK, int NS, int OCC, bool A_K, bool B_K, bool EXT, int VB = 16, bool SK = false>
int launch_one_d(hipStream_t st, const DArgsD &g, unsigned grid) {
    constexpr size_t lds_bytes = NS * (BM * BK + BN * BK) * sizeof(double);
    auto kern = gemm_f64_dma_kernel<BM, BN, BK, NS, OCC, A_K, B_K, EXT, VB, SK>;
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
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds_bytes, st, g);
    return launch_status();
}

template <int BM, int BN, int BK, int NS, int OCC, int VB = 16, bool SK = false> int launch_tile_d(hipStream_t st, const GemmProblem &p) {
    DArgsD g{};
    g.A = static_cast<const double *>(p.A);
    g.B = static_cast<const double *>(p.B);
    g.C = static_cast<double *>(p.C);
    g.M = (uint32_t)p.M; g.N = (uint32_t)p.N; g.K = (uint32_t)p.K;
    g.lda = (uint32_t)p.lda; g.ldb = (uint32_t)p.ldb; g.ldc = (uint32_t)p.ldc;
    g.tiles_m = (uint32_t)((p.M + BM - 1) / BM);
    g.tiles_n = (uint32_t)((p.N + BN - 1) / BN);
    g.epi = p.epi;
    std::memcpy(&g.alpha, p.alpha, sizeof(double));
    std::memcpy(&g.beta, p.beta, sizeof(double));
    g.bias = static_cast<const double *>(p.ext_bias);
    g.act = p.ext_act;
    const bool row_walk = g_test_options.gemm_walk_rows != 0;
    if (!row_walk) {
        static const unsigned shapes[][2] = {{4, 8}, {4, 4}, {2, 8}, {2, 4}};
        for (const auto &sh : shapes)
            if (g.tiles_m % sh[0] == 0 && g.tiles_n % sh[1] == 0 && ((g.tiles_m / sh[0]) * (g.tiles_n / sh[1])) % 8 == 0) {
                g.patch_m = sh[0];
                g.patch_n = sh[1];
                break;
            }
    }
    const int sel = (p.op_a ? 0 : 2) | (p.op_b ? 1 : 0);
    g.tiles_run = g.tiles_m * g.tiles_n;
    const unsigned resident = g_test_options.persistent ? p.num_cus * (unsigned)OCC : 0u; // as in the f32 launch
    unsigned grid = resident && g.tiles_run > resident && (g.tiles_run < 2 * resident || g_test_options.persistent == 2) ? resident : g.tiles_run;
    if constexpr (SK) {
        unsigned groups = 0;
        if (p.ext || !gemm_dma_stream_k_plan(p, BM, BN, BK, OCC, groups, g.sk_units, g.sk_total, g.sk_first)) return WK_E_INVALID_VALUE;
        g.sk_groups = groups;
        const unsigned rounds = g.sk_first / groups;
        grid = g.sk_first ? groups * std::min<unsigned>((unsigned)OCC, rounds + 1) : groups;
        g.partials = static_cast<double *>(p.scratch);
        g.counters = p.counters;
        g.patch_m = g.patch_n = 0; // consecutive tile numbers are neighbours in the row-group walk
    }
    if (p.ext) {
        if constexpr (VB == 16 && !SK) return sel == 3 ? launch_one_d<BM, BN, BK, NS, OCC, true, true, true>(st, g, grid) : (int)WK_E_INVALID_VALUE;
        else return WK_E_INVALID_VALUE;
    }
    switch (sel) {
    case 0: return launch_one_d<BM, BN, BK, NS, OCC, false, false, false, VB, SK>(st, g, grid);
    case 1: return launch_one_d<BM, BN, BK, NS, OCC, false, true, false, VB, SK>(st, g, grid);
    case 2: return launch_one_d<BM, BN, BK, NS, OCC, true, false, false, VB, SK>(st, g, grid);
    default: return launch_one_d<BM, BN, BK, NS, OCC, true, true, false, VB, SK>(st, g, grid);
    }
}

bool f64_rows_aligned(const GemmProblem &p) {
    return p.lda % 2 == 0 && p.ldb % 2 == 0 && ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 15u) == 0;
}

} // namespace

bool wk::gemm_f64_rows_aligned(const GemmProblem &p) { return f64_rows_aligned(p); }

bool wk::gemm_f64_dma_applies(const GemmProblem &p, int bm, int bn) {
    if (p.dtype != WK_F64) return false;
    if (!((bm == 128 && bn == 128) || (bm == 64 && bn == 64))) return false;
    if (p.ext && (p.op_a || !p.op_b || !f64_rows_aligned(p))) return false;
    if (!p.M || !p.N || !p.K) return false;
    if ((reinterpret_cast<uintptr_t>(p.A) | reinterpret_cast<uintptr_t>(p.B)) & 7u) return false;
    if (p.M > 0x7fffffffull || p.N > 0x7fffffffull || p.K > 0x7fffffffull || p.ldc > 0x7fffffffull) return false;
    if (p.lda > (1ull << 20) || p.ldb > (1ull << 20)) return false; // 127 rows * ld * 8 bytes inside 32 bits
    if (((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) > 0x7fffffffull) return false;
    return true;
}

int wk::gemm_f64_dma_launch(hipStream_t st, const GemmProblem &p, int bm, int bn) {
    if (!gemm_f64_dma_applies(p, bm, bn)) return WK_E_INVALID_VALUE;
    if (!f64_rows_aligned(p)) // rows that start anywhere: four bytes per lane and load
        return bm == 128 ? launch_tile_d<128, 128, 16, 2, 2, 4>(st, p) : launch_tile_d<64, 64, 16, 3, 3, 4>(st, p);
    if (bm == 128) return launch_tile_d<128, 128, 16, 2, 2>(st, p);
    // (64 x 64 with k-slabs of 32 in two stages, two work-groups per unit, measured the same within the run-to-run
    // spread: 8192 x 256 x 8192 67.4-68.6 against 68.0-68.2 TFLOP/s, 2048^3 68-69 against 66-68, 3072^3 70-71 both;
    // two stages of 16 with three or four per unit: 8192 x 256 x 8192 65.6 against 68.7, 1024^3 45 against 53-56)
    return launch_tile_d<64, 64, 16, 3, 3>(st, p);
}

// work dealt by k-slabs (rows that start on 16-byte boundaries)
bool wk::gemm_f64_dma_stream_k_applies(const GemmProblem &p, int bm, int bn) {
    if (!gemm_f64_dma_applies(p, bm, bn) || !f64_rows_aligned(p) || p.ext) return false;
    unsigned groups;
    uint32_t units, total, first;
    return gemm_dma_stream_k_plan(p, bm, bn, 16, bm == 128 ? 2 : 3, groups, units, total, first);
}

int wk::gemm_f64_dma_stream_k_launch(hipStream_t st, const GemmProblem &p, int bm, int bn) {
    if (!gemm_f64_dma_stream_k_applies(p, bm, bn)) return WK_E_INVALID_VALUE;
    if (bm == 128) return launch_tile_d<128, 128, 16, 2, 2, 16, true>(st, p);
    return launch_tile_d<64, 64, 16, 3, 3, 16, true>(st, p);
}

