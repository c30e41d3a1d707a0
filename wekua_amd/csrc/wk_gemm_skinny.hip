// f32 / f64 products whose C has at most 32 (one layout of the large operand: 64) rows or columns and whose other operand is large: a
// batch of a few rows through a weight matrix (Linear.forward and its sensitivities at small batch sizes are
// blas.gemm calls of this shape).  A 64 x 64 tile kernel pads the short side to 64 and spends two to eight
// times the matrix work the product needs, which makes a product that should wait for memory wait for the
// matrix pipes instead.  Here the large operand is read once, straight into registers along its storage order,
// and multiplied with v_mfma_*_16x16x4 (one, two or four blocks of sixteen on the short side), so that the launch is
// bound by the memory that operand streams from.
//
//   out(s, b) = sum_k S(s, k) * Big(k, b),   s < R <= 64 (the short index), b < L
//
// Rows short (M <= 64): s = row of C, b = column; S = op(A), Big = op(B).  Columns short (N <= 64): s = column of
// C, b = row; S(s, k) = op(B)(k, s), Big(k, b) = op(A)(b, k).
//
// A work-group of four wavefronts owns CW values of b (128 floats of a b-contiguous Big, 64 values otherwise) and one
// share of k; // its wavefronts split the share's k range in four.  The matrix instruction sums over the four k values its
// four groups of sixteen lanes supply, and it does not matter which four those are as long as S and Big agree,
// so lane (c, q) (c = lane % 16, q = lane / 16) takes the KQ consecutive k values q of every group of 4 KQ:
//   Big b-contiguous (Big[k * ld + b]): 16 bytes = EPL values of b per lane and load, rows k = kg + 4 q + i; value
//     e of the load belongs to column EPL c + e of its group of 16 EPL columns, so matrix instruction (j, e)
//     multiplies the columns {16 EPL j + EPL c + e} -- the columns of an instruction are a choice, too;
//   Big k-contiguous (Big[b * ld + k]): 32 bytes of k per lane and column (two loads), columns 16 g + c.
// Both ways a wavefront's loads cover whole 128-byte lines.  S comes from the caches (all work-groups read the
// same R rows): 16-byte loads along k where its rows allow it, single elements otherwise.  Loads are issued
// one group of k ahead of the matrix instructions that use them.
//
// The four wavefronts' sums meet in LDS (added in the order of the wavefronts); with k split over work-groups
// as well (grid y; enough work-groups to fill every unit), the shares' sums meet in the stream's scratch and
// the work-group that arrives last adds them in the order of the shares, as in the tile kernels
// (wk_gemm_mfma.hip): the same bits on every run.  Option semantics as everywhere:
// src/blas/gemm.zig:500-501,591-602; the fused bias + activation epilogue as in the tile kernels.
#include "wk_internal.hpp"

#include <cstring>
#include <type_traits>

using namespace wk;

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Vec;
template <> struct Vec<float> {
    using load_t = f32x4; // 16 bytes
    using acc_t = f32x4;
};
template <> struct Vec<double> {
    using load_t = f64x2;
    using acc_t = f64x4;
};

__device__ __forceinline__ f32x4 mfma16(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
__device__ __forceinline__ f64x4 mfma16(double a, double b, f64x4 c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }

template <typename T> struct SkinnyArgs {
    const T *S;
    uint64_t s_rs, s_ks; // S(s, k) = S[s * s_rs + k * s_ks]
    const T *Big;
    uint64_t ld;         // Big(k, b) = Big[k * ld + b] or Big[b * ld + k]
    T *C;
    uint64_t sc_s, sc_b; // C(s, b) = C[s * sc_s + b * sc_b]
    uint32_t R, L, K;
    uint32_t klen;       // k values per share: a multiple of 4 wavefronts x one group of k
    int epi;
    T alpha, beta;
    const T *bias;       // fused epilogue: bias by column of C, or null
    int ext;             // fused epilogue: + bias, activation
    int act;             // WK_ACT_*
    int bias_by_b;       // the column of C is b (rows short) rather than s
    int rotate;          // tiles of b start their walk along k at different places (k-contiguous Big)
    T *partials;         // [share][tile][16-byte piece][thread]
    uint32_t *counters;  // one per tile of b
};

template <typename T, bool BIG_K, int RB> struct Geometry {
    static constexpr int EPL = 16 / (int)sizeof(T);          // elements per 16-byte load
    // blocks of b: sixteen columns each (k-contiguous) or 16 EPL; half as many under four blocks of rows, which
    // keeps the accumulators at 64 registers
    static constexpr int NB = (BIG_K ? 4 : 2) / (RB == 4 ? 2 : 1);
    static constexpr int CW = NB * (BIG_K ? 16 : 16 * EPL);  // values of b per work-group
    static constexpr int KQ = BIG_K ? 2 * EPL : 4;           // consecutive k values per lane and group
    static constexpr int KG = 4 * KQ;                        // k values per group
    static constexpr int BIG_LOADS = BIG_K ? NB * 2 : NB * 4; // 16-byte loads of Big per lane and group
    static constexpr int ACCS = BIG_K ? NB : NB * EPL;       // matrix instructions per k value and block of rows
};

template <typename T, int RB, bool BIG_K, bool S_VEC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(RB >= 2 ? 2 : 4))) void gemm_skinny_kernel(SkinnyArgs<T> g) {
    static_assert(RB == 1 || RB == 2 || RB == 4, "one, two or four blocks of sixteen rows");
    using G = Geometry<T, BIG_K, RB>;
    using load_t = typename Vec<T>::load_t;
    using acc_t = typename Vec<T>::acc_t;
    constexpr int EPL = G::EPL, CW = G::CW, KQ = G::KQ, KG = G::KG, NB = G::NB;
    constexpr int NACC = G::ACCS * RB; // accumulators per lane, four values each
    constexpr int SV = KQ / EPL;       // 16-byte loads of S per lane, block of rows and group (S_VEC)
    __shared__ T red[4 * (NACC / 2) * 4 * 64]; // half of every wavefront's accumulators at a time
    __shared__ uint32_t s_last;

    // (the wavefront's number through readfirstlane: everything derived from it -- the k range, the loop -- is then
    // scalar, and the loop has branches the wait-count pass can follow)
    const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64, c = lane % 16, q = lane / 16;
    const uint32_t b0 = blockIdx.x * CW;
    const uint32_t kb = blockIdx.y * g.klen, ke = min(g.K, kb + g.klen);
    // this wavefront's quarter of the share, in whole groups
    const uint32_t quarter = g.klen / 4;
    const uint32_t k_lo = min(ke, kb + wave * quarter), k_hi = min(ke, k_lo + quarter);

    // ---- addresses: a scalar base that moves along k, and per-lane byte offsets of 32 bits that do not ----
    // Big: the base is the work-group's first column (row of storage) at k = 0
    const char *big_base = reinterpret_cast<const char *>(BIG_K ? g.Big + (uint64_t)b0 * g.ld : g.Big + b0);
    uint32_t big_off[NB]; // first piece of the lane: the others lie EPL values (k-contiguous) or rows of k further
    if constexpr (BIG_K) {
#pragma unroll
        for (int gb = 0; gb < NB; ++gb) big_off[gb] = ((min(b0 + 16 * gb + c, g.L - 1) - b0) * (uint32_t)g.ld + KQ * q) * (uint32_t)sizeof(T);
    } else {
        // a 16-byte piece whose first value exists is read as it is (bases and leading dimensions are multiples
        // of 16 bytes: it cannot leave that value's page); pieces wholly beyond L are read from the last one
        const uint32_t last_piece = (g.L - 1) / EPL * EPL;
#pragma unroll
        for (int j = 0; j < NB; ++j)
            big_off[j] = (min(b0 + j * 16 * EPL + EPL * c, last_piece) - b0 + 4 * q * (uint32_t)g.ld) * (uint32_t)sizeof(T);
    }
    const uint32_t ld_bytes = (uint32_t)g.ld * (uint32_t)sizeof(T);
    const uint64_t big_step = (BIG_K ? (uint64_t)1 : g.ld) * sizeof(T); // bytes per value of k
    const char *s_base = reinterpret_cast<const char *>(g.S);
    const uint64_t s_step = g.s_ks * sizeof(T);
    const uint32_t s_ks_bytes = (uint32_t)s_step;
    uint32_t s_off[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
        s_off[rb] = (min(c + 16 * rb, g.R - 1) * (uint32_t)g.s_rs + KQ * q * (uint32_t)g.s_ks) * (uint32_t)sizeof(T);

    // the byte offset of every load of a group from the group's base
    uint32_t big_lane[G::BIG_LOADS];
#pragma unroll
    for (int n = 0; n < G::BIG_LOADS; ++n) big_lane[n] = BIG_K ? big_off[n / 2] + 16u * (n % 2) : big_off[n / 4] + (n % 4) * ld_bytes;
    // single elements of S (used when its rows do not allow 16-byte loads along k): their offsets in registers,
    // except under four blocks of rows, where the registers are not there and the offsets are added up per load
    auto s_lane_of = [&](int rb, int i) -> uint32_t { return s_off[rb] + i * s_ks_bytes; };
    uint32_t s_lane[RB == 4 ? 1 : RB][RB == 4 ? 1 : KQ];
    if constexpr (RB != 4) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < KQ; ++i) s_lane[rb][i] = s_lane_of(rb, i);
    }

    struct Frag {
        load_t big[G::BIG_LOADS];
        T s[RB][KQ];
    };

    // The loads of a group that lies wholly inside K; bigp, sp: the bases at the group's first k.  Buffer loads:
    // the base travels in scalar registers and the lane's offset is one 32-bit register that never changes
    // (with flat addresses the loop would carry a 64-bit address per load and lane).
    auto load = [&](Frag &f, const char *bigp, const char *sp) {
        const __amdgpu_buffer_rsrc_t big_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(bigp), 0, 0x7fffffff, 0x00020000);
        const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(sp), 0, 0x7fffffff, 0x00020000);
#pragma unroll
        for (int n = 0; n < G::BIG_LOADS; ++n)
            f.big[n] = __builtin_bit_cast(load_t, __builtin_amdgcn_raw_buffer_load_b128(big_rsrc, big_lane[n], 0, 0));
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            if constexpr (S_VEC) {
#pragma unroll
                for (int h = 0; h < SV; ++h) {
                    const load_t v = __builtin_bit_cast(load_t, __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, s_off[rb] + 16u * h, 0, 0));
#pragma unroll
                    for (int e = 0; e < EPL; ++e) f.s[rb][EPL * h + e] = v[e];
                }
            } else {
#pragma unroll
                for (int i = 0; i < KQ; ++i) {
                    if constexpr (sizeof(T) == 4) f.s[rb][i] = __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(s_rsrc, RB == 4 ? s_lane_of(rb, i) : s_lane[RB == 4 ? 0 : rb][RB == 4 ? 0 : i], 0, 0));
                    else f.s[rb][i] = __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b64(s_rsrc, RB == 4 ? s_lane_of(rb, i) : s_lane[RB == 4 ? 0 : rb][RB == 4 ? 0 : i], 0, 0));
                }
            }
        }
    };
    // the last group of the whole product when K is no multiple of a group: what lies beyond K must multiply as
    // zero on both sides, and every address stays inside the operands (a value that does not exist is read
    // from k = K - 1, or from the start of the row of a k-contiguous operand, and replaced)
    auto load_checked = [&](Frag &f, uint32_t k) {
        if constexpr (BIG_K) {
#pragma unroll
            for (int gb = 0; gb < NB; ++gb)
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t kk = k + KQ * q + EPL * h; // first k of this piece
                    const char *at = big_base + big_off[gb] + (kk < g.K ? ((uint64_t)k + EPL * h) * sizeof(T) : (uint64_t)0 - KQ * q * sizeof(T));
                    load_t v = *reinterpret_cast<const load_t *>(at);
#pragma unroll
                    for (int e = 0; e < EPL; ++e)
                        if (kk + e >= g.K) v[e] = T(0);
                    f.big[gb * 2 + h] = v;
                }
        } else {
#pragma unroll
            for (int j = 0; j < NB; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t kk = k + 4 * q + i;
                    const int64_t row = kk < g.K ? (int64_t)(k + i) : (int64_t)g.K - 1 - 4 * (int64_t)q; // (big_off holds row 4 q)
                    load_t v = *reinterpret_cast<const load_t *>(big_base + big_off[j] + row * (int64_t)big_step);
                    if (kk >= g.K) v = load_t{};
                    f.big[j * 4 + i] = v;
                }
        }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int i = 0; i < KQ; ++i) {
                const uint32_t kk = k + KQ * q + i;
                f.s[rb][i] = kk < g.K ? *reinterpret_cast<const T *>(s_base + s_off[rb] + (uint64_t)(k + i) * s_step) : T(0);
            }
    };

    acc_t acc[NACC / RB][RB];
#pragma unroll
    for (int a = 0; a < NACC / RB; ++a)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) acc[a][rb] = acc_t{};

    auto multiply = [&](const Frag &f) {
#pragma unroll
        for (int i = 0; i < KQ; ++i) {
            if constexpr (BIG_K) {
#pragma unroll
                for (int gb = 0; gb < NB; ++gb)
#pragma unroll
                    for (int rb = 0; rb < RB; ++rb) acc[gb][rb] = mfma16(f.s[rb][i], f.big[gb * 2 + i / EPL][i % EPL], acc[gb][rb]);
            } else {
#pragma unroll
                for (int j = 0; j < NB; ++j)
#pragma unroll
                    for (int e = 0; e < EPL; ++e)
#pragma unroll
                        for (int rb = 0; rb < RB; ++rb)
                            acc[j * EPL + e][rb] = mfma16(f.s[rb][i], f.big[j * 4 + i][e], acc[j * EPL + e][rb]);
            }
        }
    };

    // ---- main loop: the loads of a group are in flight while the one before it is multiplied.  No branch lies
    // between the loads of a group and the matrix instructions of the one before: at a branch the wait-count pass
    // would wait for everything that may be in flight, the loads just issued included ----
    const uint32_t groups = (k_hi - k_lo) / KG; // whole groups inside [k_lo, k_hi)
    // The work-groups of a share all walk the same k at the same time, each along its own rows of a k-contiguous
    // Big: with a leading dimension that is a multiple of the memory channels' period those rows' pieces sit in
    // the same channels.  Each tile of b therefore starts its groups at another place and wraps around (a fixed
    // place per tile: the sums are still the same bits on every run).
    const uint32_t rot = BIG_K && g.rotate ? (uint32_t)((uint64_t)(blockIdx.x % 16u) * groups / 16u) : 0u;
    auto big_of = [&](uint32_t i) { // bases of the i-th group in walking order
        const uint32_t at = i + rot < groups ? i + rot : i + rot - groups;
        return big_base + ((uint64_t)k_lo + (uint64_t)at * KG) * big_step;
    };
    auto s_of = [&](uint32_t i) {
        const uint32_t at = i + rot < groups ? i + rot : i + rot - groups;
        return s_base + ((uint64_t)k_lo + (uint64_t)at * KG) * s_step;
    };
    Frag f0, f1;
    if (groups) {
        load(f0, big_of(0), s_of(0));
        uint32_t i = 1; // f0 holds group i - 1
        // (the scheduler is kept from moving a group's loads down among the matrix instructions that come after
        // them in the source, which is where it puts them to save registers: next to their use)
        for (; i + 1 < groups; i += 2) {
            load(f1, big_of(i), s_of(i));
            __builtin_amdgcn_sched_barrier(0);
            multiply(f0);
            __builtin_amdgcn_sched_barrier(0);
            load(f0, big_of(i + 1), s_of(i + 1));
            __builtin_amdgcn_sched_barrier(0);
            multiply(f1);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (i < groups) {
            load(f1, big_of(i), s_of(i));
            __builtin_amdgcn_sched_barrier(0);
            multiply(f0);
            multiply(f1);
        } else {
            multiply(f0);
        }
    }
    if (k_lo + groups * KG < k_hi) { // the last, partial group of the whole product (k_hi = K there)
        load_checked(f0, k_lo + groups * KG);
        multiply(f0);
    }

    // ---- the four wavefronts' sums, half of the accumulators at a time: value v of lane l of wavefront w at
    // red[(w * 2 NACC + v) * 64 + l]; wavefront w goes on with accumulators [w * MINE, (w + 1) * MINE), added in
    // the order of the wavefronts ----
    constexpr int MINE = NACC / 4, HALF = NACC / 2;
    T sum[MINE][4];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        if (h) __syncthreads();
#pragma unroll
        for (int an = 0; an < HALF; ++an)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[((wave * HALF + an) * 4 + r) * 64 + lane] = acc[(h * HALF + an) / RB][(h * HALF + an) % RB][r];
        __syncthreads();
        if (wave / 2 == (uint32_t)h) {
#pragma unroll
            for (int m = 0; m < MINE; ++m)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const uint32_t at = (((wave % 2) * MINE + m) * 4 + r) * 64 + lane;
                    T v = red[at];
#pragma unroll
                    for (int w = 1; w < 4; ++w) v += red[at + w * HALF * 4 * 64];
                    sum[m][r] = v;
                }
        }
    }

    // ---- the shares' sums.  Device-scope accesses without fences, as in wk_gemm_mfma.hip: 16 bytes per lane with
    // the sc1 cache policy (bit 4 of the buffer instructions' auxiliary operand), piece p of thread t at
    // (p * 256 + t) * 16 bytes of the (share, tile)'s part.  A round trip to memory costs a microsecond or two
    // whatever it carries, so the work-group that adds the parts up has the loads of several shares in flight
    // at a time (sixteen pieces per lane) ----
    if (gridDim.y > 1) {
        constexpr int SC1 = 16;
        constexpr int PP = MINE * 4 / EPL; // 16-byte pieces per thread
        constexpr int ZB = 16 / PP;        // shares per batch of loads
        constexpr uint32_t TILE_BYTES = MINE * 4 * 256 * sizeof(T);
        const char *parts = reinterpret_cast<const char *>(g.partials);
        auto part_of = [&](uint32_t z) {
            return __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(parts) + ((size_t)z * gridDim.x + blockIdx.x) * TILE_BYTES, 0,
                                                     (int)TILE_BYTES, 0x00020000);
        };
        {
            __amdgpu_buffer_rsrc_t mine = part_of(blockIdx.y);
#pragma unroll
            for (int pc = 0; pc < PP; ++pc) {
                load_t v;
#pragma unroll
                for (int e = 0; e < EPL; ++e) v[e] = sum[(pc * EPL + e) / 4][(pc * EPL + e) % 4];
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), mine, tid * 16, pc * 4096, SC1);
            }
        }
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
        for (int m = 0; m < MINE; ++m)
#pragma unroll
            for (int r = 0; r < 4; ++r) sum[m][r] = T(0);
        for (uint32_t z0 = 0; z0 < gridDim.y; z0 += ZB) {
            u32x4 v[ZB][PP];
#pragma unroll
            for (int zz = 0; zz < ZB; ++zz) {
                __amdgpu_buffer_rsrc_t part = part_of(min(z0 + zz, gridDim.y - 1)); // (beyond the last share: read, not added)
#pragma unroll
                for (int pc = 0; pc < PP; ++pc) v[zz][pc] = __builtin_amdgcn_raw_buffer_load_b128(part, tid * 16, pc * 4096, SC1);
            }
#pragma unroll
            for (int zz = 0; zz < ZB; ++zz) {
                if (z0 + zz < gridDim.y) {
#pragma unroll
                    for (int pc = 0; pc < PP; ++pc) {
                        const load_t f = __builtin_bit_cast(load_t, v[zz][pc]);
#pragma unroll
                        for (int e = 0; e < EPL; ++e) sum[(pc * EPL + e) / 4][(pc * EPL + e) % 4] += f[e];
                    }
                }
            }
        }
    }

    // ---- epilogue: value r of accumulator (a, rb) of lane (c, q) is out(16 rb + row of (q, r), column of (a, c)) ----
#pragma unroll
    for (int m = 0; m < MINE; ++m) {
        const int an = wave * MINE + m; // = a * RB + rb
        const uint32_t a = an / RB, rb = an % RB;
        const uint32_t b = BIG_K ? b0 + 16 * a + c : b0 + (a / EPL) * 16 * EPL + EPL * c + (a % EPL);
        if (b >= g.L) continue;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            // (the two instructions lay their results out differently: f32 rows 4 q + r, f64 rows 4 r + q)
            const uint32_t s = 16 * rb + (sizeof(T) == 4 ? 4 * q + r : 4 * r + q);
            if (s >= g.R) continue;
            T *at = g.C + (uint64_t)s * g.sc_s + (uint64_t)b * g.sc_b;
            T v = sum[m][r];
            if (g.epi == EPI_ALPHA) v = g.alpha * v;
            else if (g.epi == EPI_ALPHA_BETA) v = g.alpha * v + g.beta * *at;
            if (g.ext) {
                if (g.bias) v += g.bias[g.bias_by_b ? b : s];
                v = act_forward<T>(g.act, v);
            }
            *at = v;
        }
    }
}

struct Shape {
    bool rows_short;
    uint64_t R, L;
    bool big_k, s_kc;
};

Shape shape_of(const GemmProblem &p) {
    Shape sh;
    sh.rows_short = p.M <= 64 && p.M <= p.N;
    if (sh.rows_short) {
        sh.R = p.M;
        sh.L = p.N;
        sh.big_k = p.op_b != 0; // op(B)(k, n) = B[n * ldb + k] for op T
        sh.s_kc = p.op_a == 0;  // op(A)(m, k) = A[m * lda + k] for op N
    } else {
        sh.R = p.N;
        sh.L = p.M;
        sh.big_k = p.op_a == 0; // op(A)(m, k) = A[m * lda + k] for op N
        sh.s_kc = p.op_b != 0;  // op(B)(k, n) = B[n * ldb + k] for op T
    }
    return sh;
}

// blocks of sixteen rows the short side is padded to: 1, 2 or 4
uint32_t row_blocks(const Shape &sh) { return sh.R <= 16 ? 1 : sh.R <= 32 ? 2 : 4; }
uint32_t tile_width(const GemmProblem &p, const Shape &sh) { return (sh.big_k || p.dtype == WK_F64 ? 64u : 128u) / (row_blocks(sh) == 4 ? 2u : 1u); }

// k shares.  Two (two blocks of rows) or four work-groups are resident per unit; a launch takes
// ceil(work-groups / resident) turns, each as long as a share of k plus what a work-group costs whatever its
// share (start, the sums: about 128 values of k), and every share adds a part per tile to write and read back.
// The number of shares with the smallest such time, every wavefront with at least four groups of k; klen a
// multiple of 4 wavefronts x one group.  (32 x 8200 x 8200: 129 tiles; three shares leave a quarter of the
// slots empty, seven fill two turns.)
void plan_shares(const GemmProblem &p, const Shape &sh, uint32_t &tiles, uint32_t &shares, uint32_t &klen) {
    const bool f64 = p.dtype == WK_F64;
    const uint32_t rb = row_blocks(sh);
    const uint32_t cw = tile_width(p, sh);
    const uint32_t step = 4 * (sh.big_k && !f64 ? 32 : 16);
    tiles = (uint32_t)((sh.L + cw - 1) / cw);
    const uint64_t per_unit = g_test_options.skinny >= 2 && g_test_options.skinny != 7 ? (uint64_t)g_test_options.skinny : rb >= 2 ? 2 : 4;
    const uint64_t resident = per_unit * (p.num_cus ? p.num_cus : 256);
    const uint64_t most = p.K / (4 * step) ? p.K / (4 * step) : 1; // shares of at least four groups per wavefront
    double best = 0.0;
    uint64_t best_len = 0;
    for (uint64_t want = 1; want <= most && want <= 64; ++want) {
        uint64_t len = (p.K + want - 1) / want;
        len = (len + step - 1) / step * step;
        const uint64_t n = (p.K + len - 1) / len; // shares this length gives
        const double turns = (double)((tiles * n + resident - 1) / resident);
        const double parts = n > 1 ? 1.0 + (double)n * 2.0 * 16.0 * rb / (double)p.K : 1.0;
        const double t = turns * ((double)len + 128.0) * parts;
        if (!best_len || t < best) {
            best = t;
            best_len = len;
        }
    }
    klen = (uint32_t)best_len;
    shares = (uint32_t)((p.K + best_len - 1) / best_len);
}

template <typename T, int RB, bool BIG_K> int launch_s(hipStream_t st, const SkinnyArgs<T> &g, dim3 grid, bool s_vec) {
    if (s_vec) hipLaunchKernelGGL((gemm_skinny_kernel<T, RB, BIG_K, true>), grid, dim3(256), 0, st, g);
    else hipLaunchKernelGGL((gemm_skinny_kernel<T, RB, BIG_K, false>), grid, dim3(256), 0, st, g);
    return launch_status();
}

template <typename T> int launch_t(hipStream_t st, const GemmProblem &p) {
    const Shape sh = shape_of(p);
    SkinnyArgs<T> g{};
    const T *A = static_cast<const T *>(p.A), *B = static_cast<const T *>(p.B);
    if (sh.rows_short) {
        g.S = A; g.s_rs = p.op_a ? 1 : p.lda; g.s_ks = p.op_a ? p.lda : 1;
        g.Big = B; g.ld = p.ldb;
        g.sc_s = p.ldc; g.sc_b = 1;
    } else {
        g.S = B; g.s_rs = p.op_b ? p.ldb : 1; g.s_ks = p.op_b ? 1 : p.ldb;
        g.Big = A; g.ld = p.lda;
        g.sc_s = 1; g.sc_b = p.ldc;
    }
    g.C = static_cast<T *>(p.C);
    g.R = (uint32_t)sh.R; g.L = (uint32_t)sh.L; g.K = (uint32_t)p.K;
    g.epi = p.epi;
    std::memcpy(&g.alpha, p.alpha, sizeof(T));
    std::memcpy(&g.beta, p.beta, sizeof(T));
    g.ext = p.ext ? 1 : 0;
    g.act = p.ext_act;
    g.bias = p.ext ? static_cast<const T *>(p.ext_bias) : nullptr;
    g.bias_by_b = sh.rows_short ? 1 : 0;
    g.rotate = g_test_options.skinny == 7 ? 0 : 1;
    uint32_t tiles, shares;
    plan_shares(p, sh, tiles, shares, g.klen);
    if (shares > 1) {
        const size_t need = (size_t)shares * tiles * 16 * row_blocks(sh) * tile_width(p, sh) * sizeof(T);
        if (!p.scratch || !p.counters || need > p.scratch_bytes || tiles > p.num_counters) return WK_E_SCRATCH_TOO_SMALL;
        g.partials = static_cast<T *>(p.scratch);
        g.counters = p.counters;
    }
    constexpr uint64_t EPL = 16 / sizeof(T);
    const bool s_vec = sh.s_kc && g.s_rs % EPL == 0 && (reinterpret_cast<uintptr_t>(g.S) & 15u) == 0;
    const dim3 grid(tiles, shares);
    if (sh.R > 32) return sh.big_k ? launch_s<T, 4, true>(st, g, grid, s_vec) : launch_s<T, 4, false>(st, g, grid, s_vec);
    if (sh.R > 16) return sh.big_k ? launch_s<T, 2, true>(st, g, grid, s_vec) : launch_s<T, 2, false>(st, g, grid, s_vec);
    return sh.big_k ? launch_s<T, 1, true>(st, g, grid, s_vec) : launch_s<T, 1, false>(st, g, grid, s_vec);
}

} // namespace

// At most 32 rows or columns of C, the large operand with rows on 16-byte boundaries and large enough for the
// launch to be about reading it (below that the tile kernels' split over k does as well), scratch and counters
// for the shares.  (A single row or column is the thin-product kernel's: wk_gemm.hip, narrow_kind.)
bool wk::gemm_skinny_applies(const GemmProblem &p) {
    if ((p.dtype != WK_F32 && p.dtype != WK_F64) || !g_test_options.skinny) return false;
    if (!p.M || !p.N || !p.K) return false;
    if (p.M > 64 && p.N > 64) return false;
    const Shape sh = shape_of(p);
    if (sh.L < 256 || sh.L > 0x7fffffffull || p.K < 256 || p.K > 0x7fffffffull) return false;
    if (sh.L * p.K < (1ull << 22)) return false;
    const uint64_t epl = 16 / wk_dtype_size(p.dtype);
    // (f32 with two blocks of rows and a short k: the 64 x 64 tiles pad it to twice the work only, and start faster;
    // 32 x 4096 x 1024: 9 us there, 13 here)
    if (p.dtype == WK_F32 && sh.R > 16 && p.K < 2048) return false;
    // 33 to 64 rows or columns (four blocks, tiles of half the width): where the large operand is b-contiguous; a
    // k-contiguous one is then read 128 bytes at a time from 32 rows per wavefront and loses to the 64 x 64 tiles
    // (f32 64 x 8192 x 8192 N,N 80 -> 71 us, 48 rows 85 -> 69, N,T 79 -> 93; f64 48 rows N,N 165 -> 141, N,T 163 -> 165)
    if (sh.R > 32 && sh.big_k) return false;
    if (p.dtype == WK_F32 && sh.R > 32) {
        // (four blocks of rows, a b-contiguous large operand and single-element loads of the short one do not fit
        // the registers of a wavefront in f32: the short operand must allow 16-byte loads along k)
        const void *sp = sh.rows_short ? p.A : p.B;
        const uint64_t s_rs = sh.rows_short ? p.lda : p.ldb;
        if (!sh.s_kc || s_rs % epl || (reinterpret_cast<uintptr_t>(sp) & 15u)) return false;
    }
    const void *big = sh.rows_short ? p.B : p.A;
    const uint64_t ld = sh.rows_short ? p.ldb : p.lda;
    if (ld % epl || (reinterpret_cast<uintptr_t>(big) & 15u)) return false;
    if (p.lda > (1ull << 21) || p.ldb > (1ull << 21)) return false; // (the lanes' offsets from the moving base are 32 bits)
    uint32_t tiles, shares, klen;
    plan_shares(p, sh, tiles, shares, klen);
    if (shares > 65535) return false;
    if (shares > 1) {
        const size_t need = (size_t)shares * tiles * 16 * row_blocks(sh) * tile_width(p, sh) * wk_dtype_size(p.dtype);
        if (!p.scratch || !p.counters || need > p.scratch_bytes || tiles > p.num_counters) return false;
    }
    return true;
}

int wk::gemm_skinny_launch(hipStream_t st, const GemmProblem &p) {
    if (!gemm_skinny_applies(p)) return WK_E_INVALID_VALUE;
    return p.dtype == WK_F32 ? launch_t<float>(st, p) : launch_t<double>(st, p);
}
