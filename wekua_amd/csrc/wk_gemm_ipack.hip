// 32-bit integer GEMM on the int8 matrix cores with a pack pass: the two-launch form of
// wk_gemm_imfma.hip, used when the caller brings a workspace (blas.PackedTensors does, as the
// reference's PackedTensors brings packed_a / packed_b and runs its pack kernel before every
// product: src/blas/gemm.zig:272-357, 705-720).
//
// The arithmetic is the same ring identity (a = sum_i 256^i s_i with balanced signed digits s_i, ten
// signed-digit products; see wk_gemm_imfma.hip).  What changes is where the digits are made:
//
//   pass 1  ipack_kernel      reads op(A) and op(B) once, whatever their layout, and writes their
//                             signed-digit planes in the order the matrix instruction eats them:
//                             1 KiB blocks, one per (32 rows, 32 k, digit), lane l of a wavefront
//                             owning bytes 16 l .. 16 l + 15 = row l % 32, k 16 (l / 32) .. + 15.
//                             Rows and k beyond the matrix are zero digits.
//   pass 2  gemm_i32_packed_kernel   128 x 128 tile, 8 waves, k-slab 32: 32 KiB of blocks per slab
//                             go global -> registers -> LDS as plain 16-byte copies, fragments come
//                             back with one conflict-free 16-byte LDS read each, and the loop is
//                             otherwise matrix instructions (20 per wave and slab).  No digit
//                             arithmetic, no edge cases (the planes are padded to the tile), one
//                             set of staging registers that fits beside the 128 accumulators.
//
// Workspace: 128 bytes per (padded row, 32 k) of each operand; for 2048^3 that is 2 x 16 MiB.  The pack pass costs what reading A and B once and writing as much costs.
//
// 8- and 16-bit integers take the same two passes with one or two digits per element (modulo 2^8 only
// the pair (0,0) survives, modulo 2^16 the pairs with i + j <= 1): a slab is then four or two k-blocks
// of 32, so that it is 4 KiB per 32 rows whatever the width, and the matrix work per slab is 4 x 1 or
// 2 x 3 instructions per 32 x 32 block instead of 10.  Their only other kernel is the vector-ALU one.
#include "wk_internal.hpp"
#include "wk_lds_dma.hpp"

#include <cstring>
#include <type_traits>

using namespace wk;

namespace {

typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
struct __attribute__((packed, aligned(4))) u32x4_u { u32x4 v; };

constexpr int TILE = 128, BK = 32, BLOCK_BYTES = 1024, GROUP_BYTES = 4 * BLOCK_BYTES; // one slab of 32 rows: 4 blocks
// element of D bytes = D digits; a slab holds 4 / D k-blocks of D digit blocks
template <typename E> struct Digits {
    static constexpr int D = sizeof(E), KB_PER_SLAB = 4 / D;
};
constexpr int PACK_THREADS = 256;
constexpr uint32_t MAX_KSPLIT = 16;

struct Layout {
    uint64_t Mp, Np, KB, slabs, ksplit; // KB: k-blocks of 32, padded to whole slabs; ksplit: k-ranges of the pack launch
    size_t planes_a, planes_b;          // byte offsets into the workspace
    size_t flags_a, flags_b;            // one byte per (row block, k-range of the pack launch): which digit planes hold a non-zero digit
    size_t total;
};

Layout make_layout(int digits, uint64_t M, uint64_t N, uint64_t K) {
    Layout w;
    const uint64_t per_slab = 4 / digits;
    const uint64_t m_tile = digits < 4 ? 256 : TILE; // the narrow types may run the 256-row tile
    w.Mp = (M + m_tile - 1) / m_tile * m_tile;
    const uint64_t n_tile = digits == 1 ? 256 : TILE; // 8-bit: also the 256-column tile
    w.Np = (N + n_tile - 1) / n_tile * n_tile;
    // (an even number of slabs, for the two-stage loop of the direct-to-LDS kernels; the 32-bit product kernel
    // takes stages of up to four k-blocks when the upper digit planes are empty: eight k-blocks)
    const uint64_t kb_round = digits == 4 ? 8 : 2 * per_slab;
    w.KB = ((K + BK - 1) / BK + kb_round - 1) / kb_round * kb_round;
    w.slabs = w.KB / per_slab;
    // enough work-groups in the pack launch to fill the chip: (Mp + Np) / 32 row blocks x ksplit
    uint64_t ks = 2048 / ((w.Mp + w.Np) / 32);
    ks = ks < 1 ? 1 : ks > MAX_KSPLIT ? MAX_KSPLIT : ks;
    if (ks > w.KB) ks = w.KB;
    w.ksplit = ks;
    w.planes_a = 0;
    w.planes_b = w.planes_a + (size_t)w.Mp / 32 * w.slabs * GROUP_BYTES;
    w.flags_a = w.planes_b + (size_t)w.Np / 32 * w.slabs * GROUP_BYTES;
    w.flags_b = w.flags_a + (size_t)w.Mp / 32 * MAX_KSPLIT;
    w.total = w.flags_b + (size_t)w.Np / 32 * MAX_KSPLIT;
    return w;
}

// Balanced digits: with c = 0x80 in every byte, the bytes t_i of t = a + c (carries and all, modulo 2^32) give
// a = t - c = sum_i 256^i (t_i - 128), and t_i - 128 as a signed byte is t_i ^ 0x80.  Small |a| have zero upper digits.
// 4x4 byte transpose: e[t] = element at k+t -> p[d] = digit d of k+0..k+3
__device__ __forceinline__ void digit_planes(const uint32_t e[4], uint32_t p[4]) {
    constexpr uint32_t CBIAS = 0x80808080u;
    const uint32_t a = (e[0] + CBIAS) ^ CBIAS, b = (e[1] + CBIAS) ^ CBIAS, c = (e[2] + CBIAS) ^ CBIAS, d = (e[3] + CBIAS) ^ CBIAS;
    const uint32_t ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400u), ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602u);
    const uint32_t cd_lo = __builtin_amdgcn_perm(d, c, 0x05010400u), cd_hi = __builtin_amdgcn_perm(d, c, 0x07030602u);
    p[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);
    p[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
    p[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
    p[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
}

// the same for D = 1 or 2 digits of the four (zero-extended) elements (one digit: the byte itself, read as signed)
template <int D> __device__ __forceinline__ void digit_planes_narrow(const uint32_t e[4], uint32_t p[D]) {
    constexpr uint32_t c = D == 1 ? 0u : 0x8080u;
    const uint32_t a = (e[0] + c) ^ c, b = (e[1] + c) ^ c, cc = (e[2] + c) ^ c, d = (e[3] + c) ^ c;
#pragma unroll
    for (int i = 0; i < D; ++i)
        p[i] = ((a >> (8 * i)) & 0xffu) | (((b >> (8 * i)) & 0xffu) << 8) | (((cc >> (8 * i)) & 0xffu) << 16) |
               (((d >> (8 * i)) & 0xffu) << 24);
}

struct PackOperand {
    const void *src;       // element (r, k) at src[r * ld + k] (k-contiguous) or src[k * ld + r]
    uint32_t ld, rows, row_blocks; // true rows; padded rows / 32
    unsigned char *planes;
    unsigned char *flags;  // [row block][MAX_KSPLIT]: bit d set when digit plane d of that row block and k-range is not all zero
    uint32_t k_contiguous, vector_ok; // vector_ok: 16-byte loads along the contiguous direction are aligned
};
struct PackArgs {
    PackOperand op[2];
    uint32_t K, KB, kb_per_split;
};

// blockIdx.x: row block of A, then of B; blockIdx.y: k-range.  Wave w of the work-group takes the
// k-blocks start + w, start + w + 4, ...; lane l the row l % 32 and the 16 k of half l / 32.
template <typename E>
__global__ __launch_bounds__(PACK_THREADS) void ipack_kernel(PackArgs g) {
    constexpr int D = Digits<E>::D;
    __shared__ __align__(16) unsigned char gather_tile[(PACK_THREADS / 64) * 32 * (32 * (D < 4 ? D : 1) + 4)];
    const int which = blockIdx.x >= g.op[0].row_blocks;
    const PackOperand &o = g.op[which];
    const E *__restrict__ src = static_cast<const E *>(o.src);
    unsigned char *__restrict__ planes = o.planes;
    const uint32_t rb = blockIdx.x - (which ? g.op[0].row_blocks : 0u);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5;
    const uint32_t row = rb * 32 + l32;
    const bool row_ok = row < o.rows;
    const uint32_t kb_begin = blockIdx.y * g.kb_per_split, kb_end = min(g.KB, kb_begin + g.kb_per_split);
    uint32_t nonzero[D];
#pragma unroll
    for (int d = 0; d < D; ++d) nonzero[d] = 0u;
    for (uint32_t kb = kb_begin + wave; kb < kb_end; kb += PACK_THREADS / 64) {
        const uint32_t k0 = kb * BK + 16 * half;
        uint32_t e[16];
        if (o.k_contiguous) {
            const E *p = src + (size_t)row * o.ld + k0;
            if (row_ok && o.vector_ok && k0 + 16 <= g.K) {
                u32x4 vec[D];
#pragma unroll
                for (int q = 0; q < D; ++q) vec[q] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const unsigned char *>(p) + 16 * q);
                E raw[16];
                __builtin_memcpy(raw, vec, 16 * D);
#pragma unroll
                for (int j = 0; j < 16; ++j) e[j] = raw[j];
            } else {
#pragma unroll
                for (int j = 0; j < 16; ++j) e[j] = row_ok && k0 + j < g.K ? (uint32_t)p[j] : 0u;
            }
        } else if (D < 4 && o.vector_ok && rb * 32 + 32 <= o.rows && kb * BK + BK <= g.K) {
            // Row-contiguous storage of a narrow type, block inside the operand: a lane gathering its
            // 16 k from 16 rows would load one element at a time (32 * D bytes per row and wave
            // instruction).  Instead the wave copies the 32 k-rows x 32 * D bytes of the block with
            // 16-byte loads (2 D lanes per row), parks them in its own LDS tile and every lane picks
            // its column out of that.  The tile is private to the wave: LDS executes a wave's
            // instructions in order, the fences only pin the compiler.
            constexpr int LANES_PER_ROW = 2 * D, ROWS_PER_LOAD = 64 / LANES_PER_ROW, PITCH = 32 * D + 4;
            unsigned char *tile = gather_tile + wave * (32 * PITCH);
            const int seg = lane % LANES_PER_ROW;
            const unsigned char *base = reinterpret_cast<const unsigned char *>(src) + (size_t)rb * 32 * D + seg * 16;
#pragma unroll
            for (int q = 0; q < D; ++q) {
                const int k = q * ROWS_PER_LOAD + lane / LANES_PER_ROW;
                const u32x4 v = *reinterpret_cast<const u32x4 *>(base + (size_t)(kb * BK + k) * o.ld * D);
                uint32_t *dst = reinterpret_cast<uint32_t *>(tile + k * PITCH + seg * 16);
                dst[0] = v[0]; dst[1] = v[1]; dst[2] = v[2]; dst[3] = v[3];
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int j = 0; j < 16; ++j) e[j] = *reinterpret_cast<const E *>(tile + (16 * half + j) * PITCH + l32 * D);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier(); // the tile is overwritten by the next block
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j) e[j] = row_ok && k0 + j < g.K ? (uint32_t)src[(size_t)(k0 + j) * o.ld + row] : 0u;
        }
        u32x4 out[D];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t pd[D];
            if constexpr (D == 4) digit_planes(e + 4 * q, pd);
            else digit_planes_narrow<D>(e + 4 * q, pd);
#pragma unroll
            for (int d = 0; d < D; ++d) out[d][q] = pd[d];
        }
        // block (rb, kb, d) is the (kb * D + d)-th of its row block
        unsigned char *dst = planes + ((size_t)rb * g.KB * D + (size_t)kb * D) * BLOCK_BYTES + lane * 16;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            *reinterpret_cast<u32x4 *>(dst + d * BLOCK_BYTES) = out[d];
            nonzero[d] |= out[d][0] | out[d][1] | out[d][2] | out[d][3];
        }
    }
    // Which digit planes of this row block and k-range hold anything: elements of small magnitude have zero
    // upper digits, and a product kernel that knows it multiplies only the digit pairs that can be non-zero.
    // One byte per work-group, written by plain stores (every byte has exactly one writer, so nothing needs
    // clearing beforehand).
    __shared__ uint32_t wave_mask[PACK_THREADS / 64];
    uint32_t mask = 0;
#pragma unroll
    for (int d = 0; d < D; ++d) mask |= __builtin_amdgcn_ballot_w64(nonzero[d] != 0u) ? 1u << d : 0u;
    if (lane == 0) wave_mask[wave] = mask;
    __syncthreads();
    if (tid == 0) {
        mask = 0;
#pragma unroll
        for (int w2 = 0; w2 < PACK_THREADS / 64; ++w2) mask |= wave_mask[w2];
        o.flags[(size_t)rb * MAX_KSPLIT + blockIdx.y] = (unsigned char)mask;
    }
}

struct PArgs {
    const unsigned char *planes_a, *planes_b;
    const unsigned char *flags_a, *flags_b; // the pack pass's digit-plane masks, [row block][MAX_KSPLIT]
    void *C;
    uint32_t M, N, K, slabs, Mp, Np, ldc, tiles_m, tiles_n; // slabs: what a row block's planes hold (their stride)
    uint32_t kblocks, ksplit;  // k-blocks of 32 that hold any of k; k-ranges of the pack launch (valid flag bytes per row block)
    int epi;
    uint32_t alpha, beta;
    uint32_t patch_m, patch_n; // the direct-to-LDS kernel's tile walk (0: groups of tile rows)
};

// BM x 128 tile, BM / 32 x 2 waves.  BM = 128 (one 8-wave work-group per CU) is what is launched.
// BM = 64 -- two independent 4-wave work-groups per CU, so that the two waves of a SIMD are not held
// in the same phase by one barrier -- was measured and is slower (8192^3: 207 against 222 TOP/s): it
// copies half as much again per matrix instruction.
// WMF: 32-row blocks of A per wavefront.  With WMF = 1 a wavefront's tile is 32 x 64 and it reads
// three 4 KiB groups from LDS per eight (8-bit: per slab) matrix instructions, which for one and two
// digits is as long as the matrix work itself; WMF = 2 (64 x 64) reads four groups per sixteen.  The
// 32-bit type, with ten digit products per group pair, is not short of LDS bandwidth and its four
// accumulator sets leave no room for the larger tile.
// BN: columns of the tile (two wavefronts across, BN / 64 blocks of 32 columns each).
template <int BM, int WMF = 1, int BN = TILE> struct PackedTile {
    static constexpr int WAVES_M = BM / (32 * WMF);
    static constexpr int NT = WAVES_M * 2 * 64;             // threads
    static constexpr int GROUPS = BM / 32 + BN / 32;        // 4 KiB groups per slab: A row blocks, then B column blocks
    static constexpr int STAGE_BYTES = GROUPS * GROUP_BYTES;
    static constexpr int GROUPS_PER_PASS = NT * 16 / GROUP_BYTES; // 1 or 2
    static constexpr int PASSES = GROUPS / GROUPS_PER_PASS;
    static constexpr size_t LDS_BYTES = 2 * STAGE_BYTES;
};

template <typename E, int BM, bool EDGE, int WMF = 1, int BN = TILE>
__global__ __launch_bounds__(BM / (32 * WMF) * 128) __attribute__((amdgpu_waves_per_eu(2)))
void gemm_int_packed_kernel(PArgs g) {
    using TL = PackedTile<BM, WMF, BN>;
    constexpr int WNF = BN / 64;        // 32-column blocks of B per wavefront
    static_assert(TL::GROUPS % TL::GROUPS_PER_PASS == 0, "tile shape");
    constexpr int D = Digits<E>::D, KB_PER_SLAB = Digits<E>::KB_PER_SLAB;
    constexpr int STAGE_BYTES = TL::STAGE_BYTES, PASSES = TL::PASSES, A_GROUPS = BM / 32;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    unsigned char *stages = lds_raw;                                              // [2][STAGE_BYTES]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
    uint32_t tile_m, tile_n;
    {
        const uint32_t pid = blockIdx.x, group_size = 8 * g.tiles_n, group = pid / group_size, first_m = group * 8;
        const uint32_t gsz = min(g.tiles_m - first_m, 8u), in_group = pid - group * group_size;
        tile_m = first_m + in_group % gsz;
        tile_n = in_group / gsz;
    }
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    i32x16 acc[D][WMF][WNF]; // one set per shift i + j
#pragma unroll
    for (int s = 0; s < D; ++s)
#pragma unroll
        for (int am = 0; am < WMF; ++am)
#pragma unroll
            for (int b = 0; b < WNF; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[s][am][b][r] = 0;

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
        const unsigned char *p = gi < A_GROUPS ? g.planes_a + (size_t)(tile_m * A_GROUPS + gi) * g.slabs * GROUP_BYTES
                                               : g.planes_b + (size_t)(tile_n * (BN / 32) + gi - A_GROUPS) * g.slabs * GROUP_BYTES;
        src[i] = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char *>(p), 0, (int)(g.slabs * GROUP_BYTES), 0x00020000);
    }
    // Two register sets: the slab loaded in step kb is stored to LDS at the end of step kb + 1 and
    // used in step kb + 2, so a load has two slabs of matrix work to arrive.
    // (past the end the last slab is loaded again and dropped: no branch, so the loads stay where
    // they are written, ahead of the matrix work)
    u32x4 staged[2][PASSES];
    auto gload = [&](u32x4 *dst, uint32_t kb) {
        const int off = (int)(min(kb, g.slabs - 1) * GROUP_BYTES);
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
        const unsigned char *sa = stages + buf * STAGE_BYTES + wm * WMF * GROUP_BYTES + lane * 16;
        const unsigned char *sb = stages + buf * STAGE_BYTES + (A_GROUPS + wn * WNF) * GROUP_BYTES + lane * 16;
        // the four blocks of a group: k-block f / D of the slab, digit f % D
        i32x4 a[WMF][4], b[WNF][4];
#pragma unroll
        for (int f = 0; f < 4; ++f) {
#pragma unroll
            for (int am = 0; am < WMF; ++am) a[am][f] = *reinterpret_cast<const i32x4 *>(sa + am * GROUP_BYTES + f * BLOCK_BYTES);
#pragma unroll
            for (int blk = 0; blk < WNF; ++blk) b[blk][f] = *reinterpret_cast<const i32x4 *>(sb + blk * GROUP_BYTES + f * BLOCK_BYTES);
        }
#pragma unroll
        for (int kbl = 0; kbl < KB_PER_SLAB; ++kbl)
#pragma unroll
            for (int s = 0; s < D; ++s)
#pragma unroll
                for (int i = 0; i <= s; ++i)
#pragma unroll
                    for (int am = 0; am < WMF; ++am)
#pragma unroll
                        for (int blk = 0; blk < WNF; ++blk)
                            acc[s][am][blk] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[am][kbl * D + i], b[blk][kbl * D + s - i],
                                                                                   acc[s][am][blk], 0, 0, 0);
    };
    // one step: slab kb is in LDS stage `cur`, slab kb + 1 in flight in staged[other]
    auto step = [&](uint32_t kb, auto cur_tag) {
        constexpr int cur = decltype(cur_tag)::value;
        gload(staged[cur], kb + 2);
        compute(cur);
        if (kb + 1 < g.slabs) {
            sstore(staged[cur ^ 1], cur ^ 1);
            __syncthreads();
        }
    };

    gload(staged[0], 0);
    gload(staged[1], 1);
    sstore(staged[0], 0);
    __syncthreads();
    for (uint32_t kb = 0; kb < g.slabs; kb += 2) {
        step(kb, std::integral_constant<int, 0>{});
        if (kb + 1 < g.slabs) step(kb + 1, std::integral_constant<int, 1>{});
    }

    // epilogue: register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 block
    // (all of it modulo 2^32; the store keeps the low 8 * D bits, which is the product modulo 2^(8 D))
    E *C = static_cast<E *>(g.C);
#pragma unroll
    for (int am = 0; am < WMF; ++am)
#pragma unroll
    for (int blk = 0; blk < WNF; ++blk) {
        const uint32_t col = n0 + wn * (BN / 2) + blk * 32 + l32;
        uint32_t old[16];
        if (g.epi == EPI_ALPHA_BETA) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + (wm * WMF + am) * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                const uint32_t rowc = EDGE ? min(row, g.M - 1) : row, colc = EDGE ? min(col, g.N - 1) : col;
                old[r] = C[(size_t)rowc * g.ldc + colc];
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = m0 + (wm * WMF + am) * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
            uint32_t v = 0;
#pragma unroll
            for (int s = 0; s < D; ++s) v += (uint32_t)acc[s][am][blk][r] << (8 * s);
            if (g.epi == EPI_ALPHA) v = g.alpha * v;
            else if (g.epi == EPI_ALPHA_BETA) v = g.alpha * v + g.beta * old[r];
            if (!EDGE || ((row < g.M) & (col < g.N))) C[(size_t)row * g.ldc + col] = (E)v;
        }
    }
}

template <typename E, int BM, bool EDGE, int WMF = 1, int BN = TILE> int launch_packed(hipStream_t st, PArgs g) {
    constexpr size_t lds = PackedTile<BM, WMF, BN>::LDS_BYTES;
    auto kern = gemm_int_packed_kernel<E, BM, EDGE, WMF, BN>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) { (void)hipGetLastError(); return hip_code(attr); }
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(PackedTile<BM, WMF, BN>::NT), lds, st, g);
    return launch_status();
}

// ---- 32-bit product kernel with the slabs brought straight into LDS ------------------------------
// The packed planes are already in the order the matrix instruction eats them (1 KiB per block, lane l
// owning bytes 16 l .. 16 l + 15), which is also the order in which a direct global -> LDS load lays a
// wavefront's 64 x 16 bytes down.  So a slab of the 128 x 128 tile (four row groups of A, four column
// groups of B, 32 KiB) is 32 such loads, eight per wavefront, NS stages deep, with no staging registers
// and no LDS stores.  The registers go to the tile instead: four wavefronts of 64 x 64 (one per SIMD,
// 256 accumulator registers: 2 x 2 blocks x four shift sets) with two sets of the slab's sixteen
// fragments, so that a wavefront reads 16 KiB from LDS per 40 matrix instructions (the 8-wavefront
// kernel above: 12 KiB per 20) and the fragments of slab kt + 1 are on their way while slab kt is
// multiplied.  Per iteration: request slab kt + NS - 1, half of the matrix instructions, wait for the
// own loads of slab kt + 1, barrier, read its fragments into the other set, the other half.
struct PackedDmaTile {
    static constexpr int BM = TILE, BN = TILE, GROUPS = 8, STAGE_BYTES = GROUPS * GROUP_BYTES;
    static constexpr size_t lds_bytes(int ns) { return (size_t)ns * STAGE_BYTES; }
};

template <bool EDGE, int NS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_i32_packed_dma_kernel(PArgs g) {
    using namespace wk::lds_dma;
    using TL = PackedDmaTile;
    constexpr int BM = TL::BM, BN = TL::BN, STAGE_BYTES = TL::STAGE_BYTES;
    extern __shared__ __align__(16) unsigned char lds_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
    uint32_t tile_m, tile_n;
    if (g.patch_m) { // XCD-local patches: work-group b runs on XCD b % 8 (see wk_gemm_dma.hip)
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

    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds_raw);

    // How many digit planes of this tile's operands hold anything (the pack pass's masks: one byte per row
    // block and k-range, 4 x MAX_KSPLIT = 64 bytes per operand and tile, one per lane).  Planes that are all
    // zero contribute nothing to any digit product, so leaving their products out changes no bit of the
    // result.  ND = 1: only digit 0 anywhere (entries in [-128, 127]); 2: digits 0 and 1; else all four.
    uint32_t nd;
    {
        static_assert(MAX_KSPLIT == 16, "one flag byte per lane: four row blocks x sixteen k-ranges");
        const uint32_t blk = lane >> 4, range = lane & 15;
        uint32_t m = 0;
        if (range < g.ksplit)
            m = (uint32_t)g.flags_a[(size_t)(tile_m * 4 + blk) * MAX_KSPLIT + range] |
                (uint32_t)g.flags_b[(size_t)(tile_n * 4 + blk) * MAX_KSPLIT + range];
        const bool upper = __builtin_amdgcn_ballot_w64((m & 0xCu) != 0u) != 0, second = __builtin_amdgcn_ballot_w64((m & 0x2u) != 0u) != 0;
        nd = upper ? 4u : second ? 2u : 1u;
    }

    // The main loop for ND digit planes per operand.  A stage of the pipeline is always 32 KiB: for each of
    // the tile's eight groups (A's four row groups, then B's four column groups) four 1 KiB blocks, which are
    // the ND digit blocks of 4 / ND consecutive k-blocks (block slot s = k-block s / ND of the stage, digit
    // s % ND).  ND = 4 is the whole product: ten digit pairs on one k-block, 40 matrix instructions per
    // stage and wavefront; ND = 2 multiplies the four pairs of digits 0 and 1 on two k-blocks (32); ND = 1
    // the pair (0, 0) on four k-blocks (16).  Wavefront w brings groups 2 w and 2 w + 1 of every stage.
    //
    // Fragment reads and matrix instructions are written as inline assembly, in the order they are to be
    // issued.  (1) The accumulators: the compiler keeps all sixteen in the 256 accumulation registers,
    // needs a few of those for itself and then spills accumulators inside the loop; here shifts 0..2
    // (twelve accumulators) are pinned to accumulation registers and shift 3 (four) to vector registers
    // beside the fragments.  (2) The order: a wavefront is alone on its SIMD, so whatever holds up its
    // instruction stream idles the matrix pipe.  Sixteen 16-byte LDS reads in a row do (four wavefronts'
    // reads of a slab keep the LDS busy for 512 clocks and the read queue is short), so the reads follow
    // the matrix instructions one by one, and the slab requests are spread over the first half in the same way.
    // What the compiler cannot see in inline assembly are the latencies: LDS reads are waited for by hand
    // (lgkmcnt at the top of the iteration that uses them), two matrix instructions on one accumulator
    // are at least four instructions apart, and in front of the epilogue, which reads the accumulators
    // with vector instructions, the wait is written out.
    auto main_loop = [&](auto nd_tag) __attribute__((always_inline)) {
        constexpr int ND = decltype(nd_tag)::value;
        constexpr int KBS = 4 / ND;                                  // k-blocks per stage
        constexpr int PAIRS = ND == 4 ? 10 : ND == 2 ? 4 : 1;        // digit pairs (i, j), i, j < ND, i + j <= 3
        constexpr int NM = KBS * PAIRS * 4, HALF = NM / 2;           // matrix instructions per stage and wavefront
        constexpr int SHIFTS = ND == 4 ? 4 : 2 * ND - 1;             // accumulator sets: one per shift i + j
        constexpr int LOADS = 8;
        i32x16 acc[SHIFTS][2][2]; // [shift i + j][row block][column block]
#pragma unroll
        for (int s = 0; s < SHIFTS; ++s)
#pragma unroll
            for (int am = 0; am < 2; ++am)
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[s][am][b][r] = 0;
        // C_old (beta given) of all four blocks as one batch of loads.  With fewer than four accumulator sets
        // the registers are there to request it ahead of the loop, so that a launch of one round does not
        // pay that latency between its last matrix instruction and its stores; the whole product reads it
        // after the loop (the fragment registers are free by then).
        uint32_t *C = static_cast<uint32_t *>(g.C);
        uint32_t old[2][2][16];
        auto read_c_old = [&]() {
            if (g.epi != EPI_ALPHA_BETA) return;
#pragma unroll
            for (int am = 0; am < 2; ++am)
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    const uint32_t col = n0 + wn * 64 + blk * 32 + l32, colc = EDGE ? min(col, g.N - 1) : col;
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const uint32_t row = m0 + (wm * 2 + am) * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                        old[am][blk][r] = C[(size_t)(EDGE ? min(row, g.M - 1) : row) * g.ldc + colc];
                    }
                }
        };
        if constexpr (ND < 4) read_c_old();
        const unsigned char *src_g[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int gi = 2 * wave + h;
            src_g[h] = gi < 4 ? g.planes_a + (size_t)(tile_m * 4 + gi) * g.slabs * GROUP_BYTES
                              : g.planes_b + (size_t)(tile_n * 4 + gi - 4) * g.slabs * GROUP_BYTES;
        }
        uint32_t voff[4]; // block slot s of a stage, relative to the stage's first k-block of the group
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) voff[sl] = lane * 16 + (sl / ND) * GROUP_BYTES + (sl % ND) * BLOCK_BYTES;
        // one of the eight requests of this wavefront per stage (group h = R / 4 of its two, block slot R % 4)
        auto issue_one = [&](uint32_t stage_bytes, auto r_tag) __attribute__((always_inline)) {
            constexpr int R = decltype(r_tag)::value, H = R / 4, SL = R & 3;
            dma16(src_g[H], voff[SL], lds0 + stage_bytes + (uint32_t)(2 * wave + H) * GROUP_BYTES + SL * BLOCK_BYTES);
            if constexpr (SL == 3) src_g[H] += KBS * GROUP_BYTES;
        };
        auto issue = [&](uint32_t stage_bytes) {
            static_for<LOADS>([&](auto r_tag) { issue_one(stage_bytes, r_tag); });
        };

        i32x4 fa[2][2][4], fb[2][2][4]; // [set][block][block slot]
        const uint32_t frag_a = lds0 + lane * 16 + (wm * 2) * GROUP_BYTES, frag_b = lds0 + lane * 16 + (4 + wn * 2) * GROUP_BYTES;
        // fragment number f of a stage: 0..7 A (block f / 4, slot f % 4), 8..15 B
        auto read_frag = [&](uint32_t stage_bytes, auto set_tag, auto f_tag) __attribute__((always_inline)) {
            constexpr int SET = decltype(set_tag)::value, F = decltype(f_tag)::value;
            constexpr int BLK = (F & 7) / 4, SL = F & 3, IMM = BLK * GROUP_BYTES + SL * BLOCK_BYTES;
            // (operands of inline assembly do not capture by themselves inside a generic lambda)
            i32x4 &dst = F < 8 ? fa[SET][BLK][SL] : fb[SET][BLK][SL];
            const uint32_t addr = (F < 8 ? frag_a : frag_b) + stage_bytes;
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(IMM));
        };
        // matrix instruction number n of a stage: k-block n / (4 PAIRS), digit pair (n / 4) % PAIRS in the order
        // (0,0) (0,1) (1,0) (0,2) (1,1) (2,0) (0,3) (1,2) (2,1) (3,0) -- for ND = 2: (0,0) (0,1) (1,0) (1,1) --
        // row block (n / 2) % 2, column block n % 2
        auto mfma_n = [&](auto set_tag, auto n_tag) __attribute__((always_inline)) {
            constexpr int SET = decltype(set_tag)::value, N = decltype(n_tag)::value;
            constexpr int Q = N / (4 * PAIRS), PAIR = (N / 4) % PAIRS, AM = (N / 2) & 1, B = N & 1;
            constexpr int SH = ND == 2 ? (PAIR + 1) / 2 : PAIR < 1 ? 0 : PAIR < 3 ? 1 : PAIR < 6 ? 2 : 3;
            constexpr int I = ND == 2 ? PAIR / 2 : PAIR - (SH == 0 ? 0 : SH == 1 ? 1 : SH == 2 ? 3 : 6);
            static_assert(I < ND && SH - I < ND && SH - I >= 0, "digit pair");
            i32x16 &c = acc[SH][AM][B];
            const i32x4 &a = fa[SET][AM][Q * ND + I], &b = fb[SET][B][Q * ND + SH - I];
            if constexpr (SH == 3) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
            else asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
        };

        // stages that hold any of k, rounded up to an even number (the planes are padded with zero digits
        // to eight k-blocks)
        const uint32_t ktiles = (g.kblocks + 2 * KBS - 1) / (2 * KBS) * 2;
        uint32_t st[NS];
#pragma unroll
        for (int n = 0; n < NS; ++n) st[n] = n * STAGE_BYTES;

        using std::integral_constant;
#pragma unroll
        for (int n = 0; n < NS - 1; ++n)
            if ((uint32_t)n < ktiles) issue(st[n]);
        wait_vm_slabs<LOADS, NS - 2>(ktiles - 1);
        __builtin_amdgcn_s_barrier();
        static_for<16>([&](auto f_tag) { read_frag(st[0], integral_constant<int, 0>{}, f_tag); });

        // P: the fragment set that holds stage kt.  ISSUE / AHEAD as in the f32 kernel of wk_gemm_dma.hip.
        // The eight requests go behind the first matrix instructions of the first half (every other one when
        // there are at least sixteen), the sixteen fragment reads behind those of the second half.
        auto iteration = [&](auto parity_tag, auto issue_tag, auto ahead_tag) __attribute__((always_inline)) {
            constexpr int P = decltype(parity_tag)::value;
            constexpr bool ISSUE = decltype(issue_tag)::value;
            constexpr int AHEAD = decltype(ahead_tag)::value;
            constexpr int ISTEP = HALF >= 16 ? 2 : 1, RPER = (16 + HALF - 1) / HALF; // reads per matrix instruction
            wait_lgkm0(); // the fragments of this stage
            static_for<HALF>([&](auto n_tag) {
                constexpr int N = decltype(n_tag)::value;
                mfma_n(integral_constant<int, P>{}, n_tag);
                if constexpr (ISSUE && N % ISTEP == 0 && N / ISTEP < LOADS) issue_one(st[NS - 1], integral_constant<int, N / ISTEP>{});
            });
            if constexpr (AHEAD >= 0) {
                wait_vm<AHEAD * LOADS>();
                __builtin_amdgcn_s_barrier();
            }
            static_for<HALF>([&](auto n_tag) {
                constexpr int N = decltype(n_tag)::value;
                mfma_n(integral_constant<int, P>{}, integral_constant<int, HALF + N>{});
                if constexpr (AHEAD >= 0)
                    static_for<RPER>([&](auto r_tag) {
                        constexpr int F = N * RPER + decltype(r_tag)::value;
                        if constexpr (F < 16) read_frag(st[1], integral_constant<int, P ^ 1>{}, integral_constant<int, F>{});
                    });
            });
            const uint32_t t = st[0];
#pragma unroll
            for (int n = 0; n + 1 < NS; ++n) st[n] = st[n + 1];
            st[NS - 1] = t;
        };
        using T_ = std::true_type;
        using F_ = std::false_type;
        using P0 = integral_constant<int, 0>;
        using P1 = integral_constant<int, 1>;
        using STEADY = integral_constant<int, NS - 2>;
        static_assert(NS == 3 || NS == 4, "the drain below is written out for these depths");
        // The fragment sets swap with the stages, so the loop runs two stages per trip; the stage count is
        // even (above), which keeps the drain below to one fixed sequence per pipeline depth.
        uint32_t kt = 0;
        for (; kt + NS < ktiles; kt += 2) {
            iteration(P0{}, T_{}, STEADY{});
            iteration(P1{}, T_{}, STEADY{});
        }
        if constexpr (NS == 4) {
            if (kt + 4 == ktiles) { // four left: the last stage is still to be requested
                iteration(P0{}, T_{}, integral_constant<int, 2>{});
                iteration(P1{}, F_{}, integral_constant<int, 1>{});
            }
        }
        iteration(P0{}, F_{}, integral_constant<int, 0>{}); // two left
        iteration(P1{}, F_{}, integral_constant<int, -1>{});

        // the last matrix instructions' results are not back yet (eight passes of four clocks and change)
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");

        // epilogue: register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32x32 block, all of it
        // modulo 2^32
        if constexpr (ND == 4) read_c_old();
#pragma unroll
        for (int am = 0; am < 2; ++am)
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                const uint32_t col = n0 + wn * 64 + blk * 32 + l32;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = m0 + (wm * 2 + am) * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                    uint32_t v = 0;
#pragma unroll
                    for (int sh = 0; sh < SHIFTS; ++sh) v += (uint32_t)acc[sh][am][blk][r] << (8 * sh);
                    if (g.epi == EPI_ALPHA) v = g.alpha * v;
                    else if (g.epi == EPI_ALPHA_BETA) v = g.alpha * v + g.beta * old[am][blk][r];
                    if (!EDGE || ((row < g.M) & (col < g.N))) C[(size_t)row * g.ldc + col] = v;
                }
            }
    };
    if (nd == 1u) main_loop(std::integral_constant<int, 1>{});
    else if (nd == 2u) main_loop(std::integral_constant<int, 2>{});
    else main_loop(std::integral_constant<int, 4>{});
}

template <bool EDGE, int NS> int launch_packed_dma(hipStream_t st, PArgs g) {
    constexpr size_t lds = PackedDmaTile::lds_bytes(NS);
    auto kern = gemm_i32_packed_dma_kernel<EDGE, NS>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) { (void)hipGetLastError(); return hip_code(attr); }
    g.tiles_m = (g.M + TILE - 1) / TILE;
    g.tiles_n = (g.N + TILE - 1) / TILE;
    g.patch_m = g.patch_n = 0;
    static const unsigned shapes[][2] = {{4, 8}, {4, 4}, {2, 8}, {2, 4}};
    for (const auto &sh : shapes)
        if (g.tiles_m % sh[0] == 0 && g.tiles_n % sh[1] == 0 && ((g.tiles_m / sh[0]) * (g.tiles_n / sh[1])) % 8 == 0) {
            g.patch_m = sh[0];
            g.patch_n = sh[1];
            break;
        }
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(256), lds, st, g);
    return launch_status();
}

// ---- 8-bit product kernel with the slabs brought straight into LDS -------------------------------
// One digit per element: the 256 x 256 tile (256 operations per byte fetched) with four wavefronts of 128 x 128
// (one per SIMD: 4 x 4 blocks = 256 accumulator registers, twelve blocks pinned to accumulation registers and
// four to vector registers as in the 32-bit kernel).  The unit of the pipeline is half a slab, two k-blocks
// of 32: eight row groups of A and eight column groups of B at 2 KiB each = 32 KiB per stage, four stages;
// a wavefront requests eight KiB of it, multiplies 2 x 16 blocks and reads sixteen fragments per stage.
// (Five stages, all of the 160 KiB, measured the same as four at 4096^3 ... 16384^3.)
struct ByteDmaTile {
    static constexpr int BM = 256, BN = 256, GROUPS = 16, HALF = GROUP_BYTES / 2, STAGE_BYTES = GROUPS * HALF;
    static constexpr size_t lds_bytes(int ns) { return (size_t)ns * STAGE_BYTES; }
};

template <bool EDGE, int NS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_i8_packed_dma_kernel(PArgs g) {
    using namespace wk::lds_dma;
    using TL = ByteDmaTile;
    constexpr int BM = TL::BM, BN = TL::BN, STAGE_BYTES = TL::STAGE_BYTES, HALF = TL::HALF;
    static_assert(NS == 4, "the drain below is written out for four stages");
    extern __shared__ __align__(16) unsigned char lds_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
    uint32_t tile_m, tile_n;
    if (g.patch_m) { // XCD-local patches: work-group b runs on XCD b % 8 (see wk_gemm_dma.hip)
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

    // wavefront w brings groups 4 w .. 4 w + 3 of every stage: A's row groups 0..7, then B's column groups
    const unsigned char *src_g[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
        const int gi = 4 * wave + h;
        src_g[h] = gi < 8 ? g.planes_a + (size_t)(tile_m * 8 + gi) * g.slabs * GROUP_BYTES
                          : g.planes_b + (size_t)(tile_n * 8 + gi - 8) * g.slabs * GROUP_BYTES;
    }
    uint32_t voff[2];
#pragma unroll
    for (int d = 0; d < 2; ++d) voff[d] = lane * 16 + d * BLOCK_BYTES;
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds_raw);
    auto issue = [&](uint32_t stage_bytes) {
#pragma unroll
        for (int h = 0; h < 4; ++h) {
#pragma unroll
            for (int d = 0; d < 2; ++d)
                dma16(src_g[h], voff[d], lds0 + stage_bytes + (uint32_t)(4 * wave + h) * HALF + d * BLOCK_BYTES);
            src_g[h] += HALF;
        }
    };
    constexpr int LOADS = 8;

    i32x16 acc[4][4]; // [row block][column block]
#pragma unroll
    for (int am = 0; am < 4; ++am)
#pragma unroll
        for (int b = 0; b < 4; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[am][b][r] = 0;

    i32x4 fa[2][4][2], fb[2][4][2]; // [set][block][k-block of the stage]
    const uint32_t frag_a = lds0 + lane * 16 + (wm * 4) * HALF, frag_b = lds0 + lane * 16 + (8 + wn * 4) * HALF;
    // fragment number f of a stage: 0..7 A (block f / 2, k-block f % 2), 8..15 B
    auto read_frag = [&](uint32_t stage_bytes, auto set_tag, auto f_tag) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_tag)::value, F = decltype(f_tag)::value;
        constexpr int BLK = (F & 7) / 2, Q = F & 1, IMM = BLK * HALF + Q * BLOCK_BYTES;
        i32x4 &dst = F < 8 ? fa[SET][BLK][Q] : fb[SET][BLK][Q];
        const uint32_t addr = (F < 8 ? frag_a : frag_b) + stage_bytes;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(IMM));
    };
    // matrix instruction number n of a stage (0..31): k-block n / 16, row block (n / 4) % 4, column block n % 4;
    // two on one accumulator are sixteen instructions apart
    auto mfma_n = [&](auto set_tag, auto n_tag) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_tag)::value, N = decltype(n_tag)::value;
        constexpr int Q = N / 16, AM = (N / 4) & 3, B = N & 3;
        i32x16 &c = acc[AM][B];
        const i32x4 &a = fa[SET][AM][Q], &b = fb[SET][B][Q];
        if constexpr (AM == 3) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
        else asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    };
    auto issue_one = [&](uint32_t stage_bytes, auto r_tag) __attribute__((always_inline)) {
        constexpr int R = decltype(r_tag)::value, H = R / 2, Q = R & 1;
        dma16(src_g[H], voff[Q], lds0 + stage_bytes + (uint32_t)(4 * wave + H) * HALF + Q * BLOCK_BYTES);
        if constexpr (Q == 1) src_g[H] += HALF;
    };

    const uint32_t ktiles = g.slabs * 2; // stages of two k-blocks; a multiple of four (the pack pass pads the planes)
    uint32_t st[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) st[n] = n * STAGE_BYTES;

    using std::integral_constant;
#pragma unroll
    for (int n = 0; n < NS - 1; ++n)
        if ((uint32_t)n < ktiles) issue(st[n]);
    wait_vm_slabs<LOADS, NS - 2>(ktiles - 1);
    __builtin_amdgcn_s_barrier();
    static_for<16>([&](auto f_tag) { read_frag(st[0], integral_constant<int, 0>{}, f_tag); });

    auto iteration = [&](auto parity_tag, auto issue_tag, auto ahead_tag) __attribute__((always_inline)) {
        constexpr int P = decltype(parity_tag)::value;
        constexpr bool ISSUE = decltype(issue_tag)::value;
        constexpr int AHEAD = decltype(ahead_tag)::value;
        wait_lgkm0(); // the fragments of this stage
        static_for<16>([&](auto n_tag) {
            constexpr int N = decltype(n_tag)::value;
            mfma_n(integral_constant<int, P>{}, n_tag);
            if constexpr (ISSUE && N % 2 == 0) issue_one(st[NS - 1], integral_constant<int, N / 2>{});
        });
        if constexpr (AHEAD >= 0) {
            wait_vm<AHEAD * LOADS>();
            __builtin_amdgcn_s_barrier();
        }
        static_for<16>([&](auto n_tag) {
            mfma_n(integral_constant<int, P>{}, integral_constant<int, 16 + decltype(n_tag)::value>{});
            if constexpr (AHEAD >= 0) read_frag(st[1], integral_constant<int, P ^ 1>{}, n_tag);
        });
        const uint32_t t = st[0];
#pragma unroll
        for (int n = 0; n + 1 < NS; ++n) st[n] = st[n + 1];
        st[NS - 1] = t;
    };
    using T_ = std::true_type;
    using F_ = std::false_type;
    using P0 = integral_constant<int, 0>;
    using P1 = integral_constant<int, 1>;
    using STEADY = integral_constant<int, NS - 2>;
    uint32_t kt = 0;
    for (; kt + NS < ktiles; kt += 2) { // the fragment sets swap with the stages: two per trip
        iteration(P0{}, T_{}, STEADY{});
        iteration(P1{}, T_{}, STEADY{});
    }
    if (kt + 4 == ktiles) { // four left: the last stage is still to be requested
        iteration(P0{}, T_{}, integral_constant<int, 2>{});
        iteration(P1{}, F_{}, integral_constant<int, 1>{});
    }
    iteration(P0{}, F_{}, integral_constant<int, 0>{}); // two left
    iteration(P1{}, F_{}, integral_constant<int, -1>{});

    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory"); // the last matrix instructions' results

    // epilogue as in the kernels above, modulo 2^8 (the store keeps the low byte)
    unsigned char *C = static_cast<unsigned char *>(g.C);
#pragma unroll
    for (int am = 0; am < 4; ++am) {
        uint32_t old[4][16];
        if (g.epi == EPI_ALPHA_BETA) {
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                const uint32_t col = n0 + wn * 128 + blk * 32 + l32, colc = EDGE ? min(col, g.N - 1) : col;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = m0 + (wm * 4 + am) * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                    old[blk][r] = C[(size_t)(EDGE ? min(row, g.M - 1) : row) * g.ldc + colc];
                }
            }
        }
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            const uint32_t col = n0 + wn * 128 + blk * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + (wm * 4 + am) * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                uint32_t v = (uint32_t)acc[am][blk][r];
                if (g.epi == EPI_ALPHA) v = g.alpha * v;
                else if (g.epi == EPI_ALPHA_BETA) v = g.alpha * v + g.beta * old[blk][r];
                if (!EDGE || ((row < g.M) & (col < g.N))) C[(size_t)row * g.ldc + col] = (unsigned char)v;
            }
        }
    }
}

template <bool EDGE, int NS> int launch_i8_dma(hipStream_t st, PArgs g) {
    constexpr size_t lds = ByteDmaTile::lds_bytes(NS);
    auto kern = gemm_i8_packed_dma_kernel<EDGE, NS>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) { (void)hipGetLastError(); return hip_code(attr); }
    g.tiles_m = (g.M + ByteDmaTile::BM - 1) / ByteDmaTile::BM;
    g.tiles_n = (g.N + ByteDmaTile::BN - 1) / ByteDmaTile::BN;
    g.patch_m = g.patch_n = 0;
    static const unsigned shapes[][2] = {{4, 8}, {4, 4}, {2, 8}, {2, 4}};
    for (const auto &sh : shapes)
        if (g.tiles_m % sh[0] == 0 && g.tiles_n % sh[1] == 0 && ((g.tiles_m / sh[0]) * (g.tiles_n / sh[1])) % 8 == 0) {
            g.patch_m = sh[0];
            g.patch_n = sh[1];
            break;
        }
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(256), lds, st, g);
    return launch_status();
}

// ---- 16-bit product kernel with the slabs brought straight into LDS ------------------------------
// Two digits per element: the 256 x 128 tile with four wavefronts of 128 x 64 (one per SIMD: 4 x 2 blocks x two
// shift sets = 256 accumulator registers, pinned as above).  The unit of the pipeline is one k-block of 32 with
// its two digit blocks: eight row groups of A and four column groups of B at 2 KiB = 24 KiB per stage, four
// stages; per stage a wavefront requests six KiB, runs the three digit products (0,0), (0,1), (1,0) on its
// eight blocks and reads twelve fragments.
struct WordDmaTile {
    static constexpr int BM = 256, BN = TILE, GROUPS = 12, HALF = GROUP_BYTES / 2, STAGE_BYTES = GROUPS * HALF;
    static constexpr size_t lds_bytes(int ns) { return (size_t)ns * STAGE_BYTES; }
};

template <bool EDGE, int NS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_i16_packed_dma_kernel(PArgs g) {
    using namespace wk::lds_dma;
    using TL = WordDmaTile;
    constexpr int BM = TL::BM, BN = TL::BN, STAGE_BYTES = TL::STAGE_BYTES, HALF = TL::HALF;
    static_assert(NS == 4, "the drain below is written out for four stages");
    extern __shared__ __align__(16) unsigned char lds_raw[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lhi = lane >> 5;
    uint32_t tile_m, tile_n;
    if (g.patch_m) { // XCD-local patches: work-group b runs on XCD b % 8 (see wk_gemm_dma.hip)
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

    // wavefront w brings groups 3 w .. 3 w + 2 of every stage: A's row groups 0..7, then B's column groups
    const unsigned char *src_g[3];
#pragma unroll
    for (int h = 0; h < 3; ++h) {
        const int gi = 3 * wave + h;
        src_g[h] = gi < 8 ? g.planes_a + (size_t)(tile_m * 8 + gi) * g.slabs * GROUP_BYTES
                          : g.planes_b + (size_t)(tile_n * 4 + gi - 8) * g.slabs * GROUP_BYTES;
    }
    uint32_t voff[2];
#pragma unroll
    for (int d = 0; d < 2; ++d) voff[d] = lane * 16 + d * BLOCK_BYTES;
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds_raw);
    auto issue = [&](uint32_t stage_bytes) {
#pragma unroll
        for (int h = 0; h < 3; ++h) {
#pragma unroll
            for (int d = 0; d < 2; ++d)
                dma16(src_g[h], voff[d], lds0 + stage_bytes + (uint32_t)(3 * wave + h) * HALF + d * BLOCK_BYTES);
            src_g[h] += HALF;
        }
    };
    constexpr int LOADS = 6;

    i32x16 acc[2][4][2]; // [shift i + j][row block][column block]
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int am = 0; am < 4; ++am)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[s][am][b][r] = 0;

    i32x4 fa[2][4][2], fb[2][2][2]; // [set][block][digit]
    const uint32_t frag_a = lds0 + lane * 16 + (wm * 4) * HALF, frag_b = lds0 + lane * 16 + (8 + wn * 2) * HALF;
    // fragment number f of a stage: 0..7 A (block f / 2, digit f % 2), 8..11 B
    auto read_frag = [&](uint32_t stage_bytes, auto set_tag, auto f_tag) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_tag)::value, F = decltype(f_tag)::value;
        constexpr int BLK = (F & 7) / 2, DIG = F & 1, IMM = BLK * HALF + DIG * BLOCK_BYTES;
        i32x4 &dst = F < 8 ? fa[SET][BLK][DIG] : fb[SET][BLK][DIG];
        const uint32_t addr = (F < 8 ? frag_a : frag_b) + stage_bytes;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(IMM));
    };
    // matrix instruction number n of a stage (0..23): digit pair n / 8 in the order (0,0) (0,1) (1,0), row block
    // (n / 2) % 4, column block n % 2; two on one accumulator are eight instructions apart
    auto mfma_n = [&](auto set_tag, auto n_tag) __attribute__((always_inline)) {
        constexpr int SET = decltype(set_tag)::value, N = decltype(n_tag)::value;
        constexpr int PAIR = N / 8, AM = (N / 2) & 3, B = N & 1;
        constexpr int SH = PAIR == 0 ? 0 : 1, I = PAIR == 2 ? 1 : 0;
        i32x16 &c = acc[SH][AM][B];
        const i32x4 &a = fa[SET][AM][I], &b = fb[SET][B][SH - I];
        if constexpr (SH == 1 && AM >= 2) asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
        else asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    };
    auto issue_one = [&](uint32_t stage_bytes, auto r_tag) __attribute__((always_inline)) {
        constexpr int R = decltype(r_tag)::value, H = R / 2, DIG = R & 1;
        dma16(src_g[H], voff[DIG], lds0 + stage_bytes + (uint32_t)(3 * wave + H) * HALF + DIG * BLOCK_BYTES);
        if constexpr (DIG == 1) src_g[H] += HALF;
    };

    const uint32_t ktiles = g.slabs * 2; // stages of one k-block; a multiple of four (the pack pass pads the planes)
    uint32_t st[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) st[n] = n * STAGE_BYTES;

    using std::integral_constant;
#pragma unroll
    for (int n = 0; n < NS - 1; ++n)
        if ((uint32_t)n < ktiles) issue(st[n]);
    wait_vm_slabs<LOADS, NS - 2>(ktiles - 1);
    __builtin_amdgcn_s_barrier();
    static_for<12>([&](auto f_tag) { read_frag(st[0], integral_constant<int, 0>{}, f_tag); });

    auto iteration = [&](auto parity_tag, auto issue_tag, auto ahead_tag) __attribute__((always_inline)) {
        constexpr int P = decltype(parity_tag)::value;
        constexpr bool ISSUE = decltype(issue_tag)::value;
        constexpr int AHEAD = decltype(ahead_tag)::value;
        wait_lgkm0(); // the fragments of this stage
        static_for<12>([&](auto n_tag) {
            constexpr int N = decltype(n_tag)::value;
            mfma_n(integral_constant<int, P>{}, n_tag);
            if constexpr (ISSUE && N % 2 == 0) issue_one(st[NS - 1], integral_constant<int, N / 2>{});
        });
        if constexpr (AHEAD >= 0) {
            wait_vm<AHEAD * LOADS>();
            __builtin_amdgcn_s_barrier();
        }
        static_for<12>([&](auto n_tag) {
            mfma_n(integral_constant<int, P>{}, integral_constant<int, 12 + decltype(n_tag)::value>{});
            if constexpr (AHEAD >= 0) read_frag(st[1], integral_constant<int, P ^ 1>{}, n_tag);
        });
        const uint32_t t = st[0];
#pragma unroll
        for (int n = 0; n + 1 < NS; ++n) st[n] = st[n + 1];
        st[NS - 1] = t;
    };
    using T_ = std::true_type;
    using F_ = std::false_type;
    using P0 = integral_constant<int, 0>;
    using P1 = integral_constant<int, 1>;
    using STEADY = integral_constant<int, NS - 2>;
    uint32_t kt = 0;
    for (; kt + NS < ktiles; kt += 2) { // the fragment sets swap with the stages: two per trip
        iteration(P0{}, T_{}, STEADY{});
        iteration(P1{}, T_{}, STEADY{});
    }
    if (kt + 4 == ktiles) { // four left: the last stage is still to be requested
        iteration(P0{}, T_{}, integral_constant<int, 2>{});
        iteration(P1{}, F_{}, integral_constant<int, 1>{});
    }
    iteration(P0{}, F_{}, integral_constant<int, 0>{}); // two left
    iteration(P1{}, F_{}, integral_constant<int, -1>{});

    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory"); // the last matrix instructions' results

    // epilogue as in the kernels above, modulo 2^16 (the store keeps the low half)
    unsigned short *C = static_cast<unsigned short *>(g.C);
#pragma unroll
    for (int am = 0; am < 4; ++am) {
        uint32_t old[2][16];
        if (g.epi == EPI_ALPHA_BETA) {
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                const uint32_t col = n0 + wn * 64 + blk * 32 + l32, colc = EDGE ? min(col, g.N - 1) : col;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t row = m0 + (wm * 4 + am) * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                    old[blk][r] = C[(size_t)(EDGE ? min(row, g.M - 1) : row) * g.ldc + colc];
                }
            }
        }
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            const uint32_t col = n0 + wn * 64 + blk * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + (wm * 4 + am) * 32 + 8 * (r / 4) + 4 * lhi + (r % 4);
                uint32_t v = (uint32_t)acc[0][am][blk][r] + ((uint32_t)acc[1][am][blk][r] << 8);
                if (g.epi == EPI_ALPHA) v = g.alpha * v;
                else if (g.epi == EPI_ALPHA_BETA) v = g.alpha * v + g.beta * old[blk][r];
                if (!EDGE || ((row < g.M) & (col < g.N))) C[(size_t)row * g.ldc + col] = (unsigned short)v;
            }
        }
    }
}

template <bool EDGE, int NS> int launch_i16_dma(hipStream_t st, PArgs g) {
    constexpr size_t lds = WordDmaTile::lds_bytes(NS);
    auto kern = gemm_i16_packed_dma_kernel<EDGE, NS>;
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (attr != hipSuccess) { (void)hipGetLastError(); return hip_code(attr); }
    g.tiles_m = (g.M + WordDmaTile::BM - 1) / WordDmaTile::BM;
    g.tiles_n = (g.N + WordDmaTile::BN - 1) / WordDmaTile::BN;
    g.patch_m = g.patch_n = 0;
    static const unsigned shapes[][2] = {{4, 8}, {4, 4}, {2, 8}, {2, 4}};
    for (const auto &sh : shapes)
        if (g.tiles_m % sh[0] == 0 && g.tiles_n % sh[1] == 0 && ((g.tiles_m / sh[0]) * (g.tiles_n / sh[1])) % 8 == 0) {
            g.patch_m = sh[0];
            g.patch_n = sh[1];
            break;
        }
    hipLaunchKernelGGL(kern, dim3(g.tiles_m * g.tiles_n), dim3(256), lds, st, g);
    return launch_status();
}

int digits_of(int dtype) {
    switch (dtype) {
    case WK_I8: case WK_U8: return 1;
    case WK_I16: case WK_U16: return 2;
    case WK_I32: case WK_U32: return 4;
    default: return 0;
    }
}

template <typename E> int launch_typed(hipStream_t st, const GemmProblem &p, unsigned char *ws, const Layout &w) {
    constexpr int D = Digits<E>::D;
    PackArgs pa;
    auto operand = [&](PackOperand &o, const void *src, uint64_t ld, uint64_t rows, uint64_t rows_p, bool kc, size_t planes) {
        o.src = src;
        o.ld = (uint32_t)ld;
        o.rows = (uint32_t)rows;
        o.row_blocks = (uint32_t)(rows_p / 32);
        o.planes = ws + planes;
        o.k_contiguous = kc;
        // 16-byte loads along the contiguous direction (k, or for the narrow types also the rows) are aligned
        o.vector_ok = (kc || D < 4) && (ld * D) % 16 == 0 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0;
    };
    operand(pa.op[0], p.A, p.lda, p.M, w.Mp, !p.op_a, w.planes_a); // A is k-contiguous for op N
    operand(pa.op[1], p.B, p.ldb, p.N, w.Np, p.op_b != 0, w.planes_b); // B for op T
    pa.op[0].flags = ws + w.flags_a;
    pa.op[1].flags = ws + w.flags_b;
    pa.K = (uint32_t)p.K;
    pa.KB = (uint32_t)w.KB;
    pa.kb_per_split = (uint32_t)((w.KB + w.ksplit - 1) / w.ksplit);
    // A's row blocks come first in the grid: with B's planes kept from the previous call only those are launched
    const uint64_t row_blocks = (p.reuse_b ? w.Mp : w.Mp + w.Np) / 32;
    hipLaunchKernelGGL(ipack_kernel<E>, dim3((unsigned)row_blocks, (unsigned)w.ksplit), dim3(PACK_THREADS), 0, st, pa);
    int rc = launch_status();
    if (rc) return rc;

    PArgs g;
    g.planes_a = ws + w.planes_a;
    g.planes_b = ws + w.planes_b;
    g.flags_a = ws + w.flags_a;
    g.flags_b = ws + w.flags_b;
    g.kblocks = (uint32_t)((p.K + BK - 1) / BK);
    g.ksplit = (uint32_t)w.ksplit;
    g.C = p.C;
    g.M = (uint32_t)p.M; g.N = (uint32_t)p.N; g.K = (uint32_t)p.K;
    g.slabs = (uint32_t)w.slabs; g.Mp = (uint32_t)w.Mp; g.Np = (uint32_t)w.Np;
    g.ldc = (uint32_t)p.ldc;
    g.tiles_m = (uint32_t)(w.Mp / TILE);
    g.tiles_n = (uint32_t)(w.Np / TILE);
    g.epi = p.epi;
    g.alpha = g.beta = 0;
    std::memcpy(&g.alpha, p.alpha, D); // little-endian: zero-extended element
    std::memcpy(&g.beta, p.beta, D);
    if constexpr (D < 4) {
        // One and two digits: the 256 x 128 tile with 64 x 64 per wavefront once it fills the chip
        // (measured against the 128 x 128 tile on MI355X: u16 4096^3 569 -> 661 TOP/s, 8192^3 607 -> 728;
        // i8 8192^3 1535 -> 1690; below one tile per CU the smaller tile wins: i8 2048^3 663 against 511).
        // These products move one byte per 170 operations even so and are bound by what the L2 delivers.
        const uint64_t tiles256 = ((p.M + 255) / 256) * ((p.N + TILE - 1) / TILE);
        if constexpr (D == 1) {
            // one digit: from one 256 x 256 tile per CU up that tile, slabs straight into LDS (256 operations per
            // byte fetched).  Against the 256 x 128 tile of the eight-wavefront kernel: i8 4096^3 1461 -> 1631-1814
            // TOP/s by the layout, 8192^3 1736 -> 2170-2260, 16384^3 1795 -> 2470-2490 (the eight-wavefront kernel
            // on the same 256 x 256 tile, which this one replaced: 1572-1743, 1911-2002, 2083-2106)
            const uint64_t tiles256x256 = ((p.M + 255) / 256) * ((p.N + 255) / 256);
            if (tiles256x256 >= (p.num_cus ? p.num_cus : 256u)) {
                const bool edge = p.M % 256 != 0 || p.N % 256 != 0;
                return edge ? launch_i8_dma<true, 4>(st, g) : launch_i8_dma<false, 4>(st, g);
            }
        }
        if (tiles256 >= (p.num_cus ? p.num_cus : 256u)) {
            const bool edge = p.M % 256 != 0 || p.N % TILE != 0;
            // two digits: that tile with the slabs straight into LDS (four wavefronts of 128 x 64): u16 4096^3 727-737 ->
            // 817-836 TOP/s, 8192^3 799-820 -> 969-975 (entries over the whole type 688 -> 793), ci16 4096^3 645 -> 709
            if constexpr (D == 2) return edge ? launch_i16_dma<true, 4>(st, g) : launch_i16_dma<false, 4>(st, g);
            return edge ? launch_packed<E, 256, true, 2>(st, g) : launch_packed<E, 256, false, 2>(st, g);
        }
    }
    const bool edge = p.M % TILE != 0 || p.N % TILE != 0;
    if constexpr (D == 4) {
        // 32 bits: the direct-to-LDS kernel, four stages (three measured 1-2 % slower; the 8-wavefront kernel
        // above: 8192^3 222-226 against 274-280 TOP/s, 4096^3 212-226 against 249-257, 2048^3 187-190 against 218-225)
        return edge ? launch_packed_dma<true, 4>(st, g) : launch_packed_dma<false, 4>(st, g);
    } else {
        return edge ? launch_packed<E, 128, true>(st, g) : launch_packed<E, 128, false>(st, g);
    }
}

} // namespace

// 0: this problem cannot take the packed path (not an 8/16/32-bit integer type; a group stream of
// slabs * 4 KiB must fit the 31-bit extent of a buffer resource, the dimensions 31 bits)
size_t wk::gemm_int_packed_workspace_bytes(int dtype, uint64_t M, uint64_t N, uint64_t K) {
    if (dtype == WK_I64 || dtype == WK_U64) return gemm_i64_packed_workspace_bytes(M, N, K);
    const int digits = digits_of(dtype);
    if (!digits || !M || !N || !K || M > 0x7fffffffull || N > 0x7fffffffull) return 0;
    if (K > (0x7fffffffull / GROUP_BYTES - 1) * BK * (4 / digits)) return 0;
    return make_layout(digits, M, N, K).total;
}

int wk::gemm_int_packed_launch(hipStream_t st, const GemmProblem &p, void *workspace, size_t workspace_bytes) {
    if (p.dtype == WK_I64 || p.dtype == WK_U64) return gemm_i64_packed_launch(st, p, workspace, workspace_bytes);
    const size_t need = gemm_int_packed_workspace_bytes(p.dtype, p.M, p.N, p.K);
    if (!need || !workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 15u)) return WK_E_INVALID_VALUE;
    // 32-bit extents and leading dimensions inside the pack pass and the product kernel
    if (p.M > 0x7fffffffull || p.N > 0x7fffffffull || p.K > 0x7fffffffull || p.lda > 0x7fffffffull ||
        p.ldb > 0x7fffffffull || p.ldc > 0x7fffffffull)
        return WK_E_INVALID_VALUE;
    const Layout w = make_layout(digits_of(p.dtype), p.M, p.N, p.K);
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    switch (digits_of(p.dtype)) {
    case 1: return launch_typed<uint8_t>(st, p, ws, w);
    case 2: return launch_typed<uint16_t>(st, p, ws, w);
    default: return launch_typed<uint32_t>(st, p, ws, w);
    }
}
