// blas.gemm entry point: argument validation, option semantics of alpha/beta, and the choice
// of kernel variant (what src/blas/gemm.zig:361-440,487-617 does with JIT flags and
// per-tensor work-item tables).
#include "wk_internal.hpp"

#include <array>
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <string>

using namespace wk;

namespace {

// -3: the packed integer path whenever a workspace comes along; -2: automatic; -1: generic tile kernel;
// >= 0: index into the MFMA variant table
std::atomic<int> g_forced{-2};

const char *k_generic_name = "tile64";
// indexed by dtype (WK_I8 .. WK_U64)
const char *k_packed_names[8] = {"mfma_i8_packed", "mfma_u8_packed", "mfma_i16_packed", "mfma_u16_packed",
                                 "mfma_i32_packed", "mfma_u32_packed", "mfma_i64_packed", "mfma_u64_packed"};
// indexed by dtype - WK_COMPLEX
const char *k_complex_packed_names[10] = {"mfma_ci8_packed",  "mfma_cu8_packed",  "mfma_ci16_packed", "mfma_cu16_packed",
                                          "mfma_ci32_packed", "mfma_cu32_packed", "mfma_ci64_packed", "mfma_cu64_packed",
                                          "mfma_cf32_packed", "mfma_cf64_packed"};
bool is_complex_float(int dtype) { return dtype == WK_CF32 || dtype == WK_CF64; }
bool is_complex_small_int(int dtype) { return dtype >= WK_COMPLEX + WK_I8 && dtype <= WK_COMPLEX + WK_U64; }
bool has_complex_packed_path(int dtype) { return is_complex_float(dtype) || is_complex_small_int(dtype); }
const char *complex_packed_name(int dtype) { return k_complex_packed_names[dtype - WK_COMPLEX]; }
// Two to four extra launches over the operands.  Measured against the generic kernel on MI355X: 512^3
// 4x faster (cf32 0.137 -> 0.034 ms), 1024^3 3.7x, 4096^3 1.8x; the launches alone cost ~15 us.
bool complex_packed_pays(const GemmProblem &p) {
    // Complex integers have only the generic kernel beside this path, and it is slow for them
    // (ci32 128^3: 37 us against 26; 512^3: 136 against 45; ci8 / ci16 256^3: 66 against 20-22).
    if (is_complex_small_int(p.dtype))
        return p.M >= 64 && p.N >= 64 && p.K >= 64 && (double)p.M * (double)p.N * (double)p.K >= 2.0e6;
    return p.M >= 64 && p.N >= 64 && p.K >= 64 && (double)p.M * (double)p.N * (double)p.K >= 1.6e7;
}
int transpose_for_gemm(void *ctx, int dtype, uint64_t rows, uint64_t cols, const void *src, uint64_t ld, void *dst) {
    const uint64_t shape[2] = {rows, cols}, src_pitches[2] = {ld, 1}, dst_pitches[2] = {rows, 1};
    return wk_transpose(static_cast<wk_stream *>(ctx), dtype, 2, shape, src_pitches, dst_pitches, 0, 1, src, dst);
}

bool is_int32(int dtype) { return dtype == WK_I32 || dtype == WK_U32; }
bool is_int64(int dtype) { return dtype == WK_I64 || dtype == WK_U64; }
bool has_packed_path(int dtype) { return dtype >= WK_I8 && dtype <= WK_U64; }
// The pack pass reads A and B once more and writes as much.  32-bit, measured against the fused
// matrix-core kernels on MI355X (N,N / T,N, microseconds, fused best of its two tiles -> packed): 1024^3
// 34 / 43 -> 39, 1536^3 61 / 63 -> 48, 2048^3 86 -> 77, 1024 x 1024 x 4096 117 / 154 -> 96, 2048 x 2048 x 512
// 28 -> 33; 4096^3 +15 %, 8192^3 +25 %.  8- and 16-bit integers have only the vector-ALU kernel (36-45 TOP/s)
// beside it: the two launches of the packed path take 16-20 us up to 1024^3, which that kernel beats below ~700^3.
bool packed_pays(const GemmProblem &p) {
    const double work = (double)p.M * (double)p.N * (double)p.K;
    if (is_int32(p.dtype)) return p.M >= 1024 && p.N >= 1024 && work >= 3.0e9;
    // 64 bits: the vector-ALU kernel (14-17 TOP/s) is the only other one (128^3: 36 us against 14, 512^3: 126 against 33)
    if (is_int64(p.dtype)) return p.M >= 32 && p.N >= 32 && p.K >= 32 && work >= 262144.0;
    return p.M >= 256 && p.N >= 256 && work >= 4.0e8;
}

int build_problem(GemmProblem &p, int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
                  const void *host_alpha, const void *A, uint64_t lda, const void *B, uint64_t ldb,
                  const void *host_beta, void *C, uint64_t ldc) {
    const size_t es = wk_dtype_size(dtype);
    if (es == 0) return WK_E_TYPE_NOT_SUPPORTED;
    if ((op_a != WK_OP_NO_TRANSPOSE && op_a != WK_OP_TRANSPOSE) || (op_b != WK_OP_NO_TRANSPOSE && op_b != WK_OP_TRANSPOSE))
        return WK_E_INVALID_VALUE;
    if (!M || !N || !K || !A || !B || !C) return WK_E_INVALID_VALUE;
    // stored shapes: A is M x K (N) or K x M (T); B is K x N (N) or N x K (T)
    const uint64_t a_cols = op_a ? M : K, b_cols = op_b ? K : N;
    if (lda < a_cols || ldb < b_cols || ldc < N) return WK_E_INVALID_VALUE;

    p.dtype = dtype; p.op_a = op_a; p.op_b = op_b;
    p.M = M; p.N = N; p.K = K; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    p.A = A; p.B = B; p.C = C;
    p.num_cus = 0;
    std::memset(p.alpha, 0, sizeof p.alpha);
    std::memset(p.beta, 0, sizeof p.beta);
    // has_alpha = alpha or beta given; alpha defaults to one (src/blas/gemm.zig:500-501,592-596)
    if (!host_alpha && !host_beta) {
        p.epi = EPI_STORE;
    } else {
        p.epi = host_beta ? EPI_ALPHA_BETA : EPI_ALPHA;
        if (host_alpha) {
            std::memcpy(p.alpha, host_alpha, es);
        } else {
            const int r = dtype % 10;
            if (r == WK_F32) { const float one = 1.f; std::memcpy(p.alpha, &one, 4); }
            else if (r == WK_F64) { const double one = 1.; std::memcpy(p.alpha, &one, 8); }
            else p.alpha[0] = 1; // little-endian integer one; the imaginary part stays zero
        }
        if (host_beta) std::memcpy(p.beta, host_beta, es);
    }
    return WK_OK;
}

// A matrix that is a few rows or columns more than whole large tiles (4097 x 4095: one row beyond 16 tiles of
// 256) makes every large tile pay for a started round and sends the whole product to the small tile.  Such
// a product is launched in parts instead: the body of whole tiles, and the thin strip(s) beyond it as
// products of their own (same K, disjoint parts of C, the same arithmetic per entry), each with the kernel the
// cost model picks for it.  A strip of one row still reads the whole other operand, so this wants a body
// that is large beside it and a k long enough for a launch more not to matter.  Measured (N,N, TFLOP/s):
// f32 4097 x 4095 x 4093 125-129 -> 137-139, 4097^3 120 -> 130, 8191 x 8193 x 8190 136-141 -> 142-143,
// 6145 x 6144 x 6144 136 -> 141, 3073 x 3072 x 3072 121 -> 127;
// f64 4097 x 4095 x 4093 61-64 -> 69.6, 4100^3 60-63 -> 67.  Wider remainders
// are split off only where the cost model says so (second half of plan_strips).
struct StripPlan {
    int parts = 0;
    GemmProblem part[3]; // body, rows beyond it (over all of N), columns beyond it (over the body's rows)
};
// the product in parts: rows [0, Mb) x columns [0, Nb), then the rows beyond Mb over all of N, then the
// columns beyond Nb over the body's rows (Mb = M / Nb = N: no such strip)
void make_parts(const GemmProblem &p, uint64_t Mb, uint64_t Nb, StripPlan &out) {
    const size_t es = wk_dtype_size(p.dtype);
    out.parts = 0;
    GemmProblem &body = out.part[out.parts++];
    body = p;
    body.M = Mb;
    body.N = Nb;
    if (Mb < p.M) {
        GemmProblem &q = out.part[out.parts++];
        q = p;
        q.M = p.M - Mb;
        q.A = static_cast<const unsigned char *>(p.A) + (p.op_a ? Mb : Mb * p.lda) * es;
        q.C = static_cast<unsigned char *>(p.C) + Mb * p.ldc * es;
    }
    if (Nb < p.N) {
        GemmProblem &q = out.part[out.parts++];
        q = p;
        q.M = Mb;
        q.N = p.N - Nb;
        q.B = static_cast<const unsigned char *>(p.B) + (p.op_b ? Nb * p.ldb : Nb) * es;
        q.C = static_cast<unsigned char *>(p.C) + Nb * es;
    }
}

// Products with a handful of rows or columns of C have kernels of their own, which read the long operand once:
// a single row or column (a matrix-vector product) goes to the thin kernel, whose lanes walk k without matrix
// instructions; two to 32 (64 in one layout) to the skinny kernel where it applies (4 x 8192 x 8192 f32: 45 us there against 72-114
// in the thin kernel), else up to four to the thin one.  0: neither, 1: thin, 2: skinny.
int narrow_kind(const GemmProblem &p) {
    const bool vector = p.M == 1 || p.N == 1;
    if (vector && gemm_thin_applies(p)) return 1;
    if (gemm_skinny_applies(p)) return 2;
    return gemm_thin_applies(p) ? 1 : 0;
}

int narrow_launch(hipStream_t st, const GemmProblem &p, int kind) { return kind == 1 ? gemm_thin_launch(st, p) : gemm_skinny_launch(st, p); }

bool plan_strips(const GemmProblem &p, StripPlan &out) {
    if ((p.dtype != WK_F32 && p.dtype != WK_F64) || p.ext || p.K < 512 || !g_test_options.strips) return false;
    if (!(p.dtype == WK_F32 ? gemm_f32_dma_applies(p, 128, 128) : gemm_f64_dma_applies(p, 128, 128))) return false;
    const uint64_t bn = 128, big = p.dtype == WK_F32 ? 256 : 128;
    // (1) thin strips -- at most a quarter of the tile's rows (256 or 128 of them: the large tiles) or of its 128
    // columns: when the body is large enough to carry the extra launches and the model agrees
    {
        uint64_t bm = big;
        if (bm == 256 && (p.M % 256 == 0 || p.M % 256 > 64)) bm = 128;
        const uint64_t m_rem = p.M % bm, n_rem = p.N % bn;
        const bool thin_m = m_rem && m_rem <= bm / 4 && p.M > bm, thin_n = n_rem && n_rem <= bn / 4 && p.N > bn;
        const uint64_t Mb = thin_m ? p.M - m_rem : p.M, Nb = thin_n ? p.N - n_rem : p.N;
        if ((thin_m || thin_n) && Mb * Nb >= (1ull << 22)) { // (2048 x 2047 and below: N,N gains 7 %, T,N loses as much)
            make_parts(p, Mb, Nb, out);
            if (g_test_options.strips == 2) return true;
            // Strips of at most four rows or columns go to the thin-product kernels, which read the long operand once
            // (16-46 us): split off as ever (4096 x 4100 x 1024: 128 TFLOP/s against 107 whole, 2050 x 4097 x 1536 125
            // against 120, f64 2049 x 2050 x 1024 58 against 54), unless the whole product would have its work dealt
            // by k-slabs -- such a launch does not pay for a started round -- and the model puts it below the parts.
            // Wider strips are launches of tile kernels, 20 us and more each: the model decides (2200^3: 123 TFLOP/s
            // whole against 106 in parts, 4000^3 138 against 130, 2312 x 2304 x 2304 127 against 120).
            bool all_thin = true;
            for (int i = 1; i < out.parts; ++i)
                all_thin = all_thin && (out.part[i].M <= 4 || out.part[i].N <= 4) && narrow_kind(out.part[i]) != 0;
            double whole = 0.0;
            const int wv = gemm_mfma_pick(p, &whole);
            if (wv < 0) return true;
            const char *wname = gemm_mfma_variant_name(wv);
            const bool whole_dealt = wname && wname[0] && wname[std::strlen(wname) - 1] == 'k';
            if (all_thin && !whole_dealt) return true;
            const double launch = 4.0 * (p.dtype == WK_F32 ? 3.05e5 : 1.525e5) / (double)p.K;
            double sum = 0.0;
            for (int i = 0; i < out.parts; ++i) {
                double c = 0.0;
                // (a thin or skinny product reads the long operand once; beyond 32 rows or columns the tile kernels'
                // figure stands for it)
                if (narrow_kind(out.part[i]) && (out.part[i].M <= 32 || out.part[i].N <= 32)) c = 5.0 * launch;
                else if (gemm_mfma_pick(out.part[i], &c) < 0) return true;
                sum += c + (i ? launch : 0.0);
            }
            return sum < whole;
        }
    }
    // (2) any remainder beyond whole large tiles, where the cost model puts the parts, with a launch each, well
    // below the whole (4296 x 4096 x 4096: 127 -> 142 TFLOP/s, 4096 x 4160 x 4096 123 -> 143, 8292 x 8192 x 4096
    // 141 -> 146, 4200^3 126 -> 135; 3000^3, 2500^3, 6000^3: the whole stays cheaper, by the model and measured)
    double whole = 0.0;
    if (gemm_mfma_pick(p, &whole) < 0) return false;
    // a launch more: about 4 us in the model's unit (cost x k / 3.05e5 = microseconds in f32, half that rate in f64)
    const double launch = 4.0 * (p.dtype == WK_F32 ? 3.05e5 : 1.525e5) / (double)p.K;
    const uint64_t m_rem = p.M > big ? p.M % big : 0, n_rem = p.N > bn ? p.N % bn : 0;
    // (a whole whose work is dealt by k-slabs was already chosen with a margin of its own; measured either side of
    // the model by 2-3 %: 4296 x 4096 x 4096 142 TFLOP/s in parts against 139 dealt, 4096 x 4160 x 4096 143 / 139, but
    // 4700^3 137 / 141 and 4300^3 136 / 138)
    const int whole_v = gemm_mfma_pick(p, nullptr);
    const char *whole_name = whole_v >= 0 ? gemm_mfma_variant_name(whole_v) : "";
    const bool whole_dealt = whole_name[0] && whole_name[std::strlen(whole_name) - 1] == 'k';
    double best = (whole_dealt ? 1.0 : 0.95) * whole;
    bool found = false;
    for (int cand = 1; cand < 4; ++cand) {
        const bool sm = cand & 1, sn = cand & 2;
        if ((sm && !m_rem) || (sn && !n_rem)) continue;
        const uint64_t Mb = sm ? p.M - m_rem : p.M, Nb = sn ? p.N - n_rem : p.N;
        if (Mb * Nb < (1ull << 21)) continue;
        StripPlan trial;
        make_parts(p, Mb, Nb, trial);
        double sum = 0.0;
        bool ok = true;
        for (int i = 0; i < trial.parts && ok; ++i) {
            double c = 0.0;
            ok = gemm_mfma_pick(trial.part[i], &c) >= 0;
            sum += c + (i ? launch : 0.0);
        }
        if (ok && sum < best) {
            best = sum;
            out = trial;
            found = true;
        }
    }
    return found;
}

int choose(const GemmProblem &p) {
    const int forced = g_forced.load(std::memory_order_relaxed);
    if (forced == -1) return -1;
    if (forced == -3) return gemm_mfma_pick(p);
    if (forced >= 0) return gemm_mfma_variant_dtype(forced) == p.dtype ? forced : gemm_mfma_pick(p);
    return gemm_mfma_pick(p);
}

} // namespace

extern "C" {

size_t wk_gemm_workspace_bytes(int dtype, int, int, uint64_t M, uint64_t N, uint64_t K) {
    if (!M || !N || !K) return 0;
    if (has_complex_packed_path(dtype)) return gemm_complex_packed_workspace_bytes(dtype, M, N, K);
    if (!has_packed_path(dtype)) return 0;
    return gemm_int_packed_workspace_bytes(dtype, M, N, K);
}

static int gemm_entry(wk_stream *s, int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K, const void *host_alpha,
                      const void *A, uint64_t lda, const void *B, uint64_t ldb, const void *host_beta, void *C, uint64_t ldc,
                      void *workspace, size_t workspace_bytes, bool reuse_b) {
    int rc = bind(s);
    if (rc) return rc;
    GemmProblem p;
    rc = build_problem(p, dtype, op_a, op_b, M, N, K, host_alpha, A, lda, B, ldb, host_beta, C, ldc);
    if (rc) return rc;
    p.num_cus = (uint32_t)s->dev->props.multiProcessorCount;
    p.reuse_b = reuse_b;
    p.scratch = s->scratch;
    p.scratch_bytes = s->scratch_bytes;
    p.counters = s->gemm_counters;
    p.num_counters = WK_GEMM_COUNTERS;
    if (has_packed_path(dtype)) {
        const int forced = g_forced.load(std::memory_order_relaxed);
        const size_t need = gemm_int_packed_workspace_bytes(dtype, M, N, K);
        const bool fits = need && workspace && workspace_bytes >= need && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0;
        if (forced == -3 && !fits) return WK_E_INVALID_VALUE;
        if (fits && (forced == -3 || (forced == -2 && packed_pays(p))))
            return gemm_int_packed_launch(s->stream, p, workspace, workspace_bytes);
    }
    if (has_complex_packed_path(dtype)) {
        const int forced = g_forced.load(std::memory_order_relaxed);
        const size_t need = gemm_complex_packed_workspace_bytes(dtype, M, N, K);
        const bool fits = need && workspace && workspace_bytes >= need && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0;
        if (forced == -3 && !fits) return WK_E_INVALID_VALUE;
        if (fits && (forced == -3 || (forced == -2 && complex_packed_pays(p)))) {
            GemmProblem real;
            void *rest = nullptr;
            size_t rest_bytes = 0;
            rc = gemm_complex_packed_prepare(s->stream, p, workspace, workspace_bytes, &transpose_for_gemm, s, real, &rest,
                                             &rest_bytes);
            if (rc) return rc;
            // the real product: 8 / 16 bits have no other matrix-core path than the packed one; 32 bits take
            // it where it pays against the fused kernel (ci32 1024^3: 78 us fused, 88 packed; 1536^3: 249 / 242)
            if (is_complex_small_int(dtype) && (forced == -3 || !is_int32(real.dtype) || packed_pays(real)))
                return gemm_int_packed_launch(s->stream, real, rest, rest_bytes);
            const int rv = gemm_mfma_pick(real);
            return rv >= 0 ? gemm_mfma_launch(s->stream, real, rv) : gemm_generic_launch(s->stream, real);
        }
    }
    if (g_forced.load(std::memory_order_relaxed) == -2) {
        const int narrow = narrow_kind(p);
        if (narrow) return narrow_launch(s->stream, p, narrow);
        StripPlan sp;
        if (plan_strips(p, sp)) {
            for (int i = 0; i < sp.parts; ++i) {
                const GemmProblem &q = sp.part[i];
                const int nq = narrow_kind(q);
                if (nq) {
                    rc = narrow_launch(s->stream, q, nq);
                } else {
                    const int pv = gemm_mfma_pick(q);
                    rc = pv >= 0 ? gemm_mfma_launch(s->stream, q, pv) : gemm_generic_launch(s->stream, q);
                }
                if (rc) return rc;
            }
            return WK_OK;
        }
    }
    const int v = choose(p);
    if (v >= 0) return gemm_mfma_launch(s->stream, p, v);
    return gemm_generic_launch(s->stream, p);
}

// a HIP error out of a launch may have cut a counting kernel short
static int after_launch(wk_stream *s, int rc) {
    if (rc >= WK_E_HIP_BASE) reset_gemm_counters(s);
    return rc;
}

int wk_gemm(wk_stream *s, int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K, const void *host_alpha,
            const void *A, uint64_t lda, const void *B, uint64_t ldb, const void *host_beta, void *C, uint64_t ldc,
            void *workspace, size_t workspace_bytes) {
    return after_launch(s, gemm_entry(s, dtype, op_a, op_b, M, N, K, host_alpha, A, lda, B, ldb, host_beta, C, ldc, workspace,
                                      workspace_bytes, false));
}

int wk_gemm_packed_b_kept(wk_stream *s, int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
                          const void *host_alpha, const void *A, uint64_t lda, const void *B, uint64_t ldb, const void *host_beta,
                          void *C, uint64_t ldc, void *workspace, size_t workspace_bytes) {
    return after_launch(s, gemm_entry(s, dtype, op_a, op_b, M, N, K, host_alpha, A, lda, B, ldb, host_beta, C, ldc, workspace,
                                      workspace_bytes, true));
}

int wk_gemm_bias_activation(wk_stream *s, int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K, const void *A,
                            uint64_t lda, const void *B, uint64_t ldb, void *C, uint64_t ldc, const void *bias, int kind) {
    int rc = bind(s);
    if (rc) return rc;
    if (kind != WK_ACT_NONE && kind != WK_ACT_SIGMOID && kind != WK_ACT_TANH) return WK_E_INVALID_VALUE;
    if (dtype != WK_F32 && dtype != WK_F64) return WK_E_TYPE_NOT_SUPPORTED;
    GemmProblem p;
    rc = build_problem(p, dtype, op_a, op_b, M, N, K, nullptr, A, lda, B, ldb, nullptr, C, ldc);
    if (rc) return rc;
    p.num_cus = (uint32_t)s->dev->props.multiProcessorCount;
    p.scratch = s->scratch;
    p.scratch_bytes = s->scratch_bytes;
    p.counters = s->gemm_counters;
    p.num_counters = WK_GEMM_COUNTERS;
    if (g_forced.load(std::memory_order_relaxed) == -2 && gemm_skinny_applies(p)) {
        p.ext = bias || kind != WK_ACT_NONE; // (every layout: the kernel's epilogue is one for all)
        p.ext_bias = bias;
        p.ext_act = kind;
        return gemm_skinny_launch(s->stream, p);
    }
    const int v = choose(p);
    if (v >= 0 && gemm_mfma_fuses(p, v) && (bias || kind != WK_ACT_NONE)) {
        p.ext = true;
        p.ext_bias = bias;
        p.ext_act = kind;
        return gemm_mfma_launch(s->stream, p, v);
    }
    // no fused kernel for this layout or variant: the product, then the element-wise pass
    rc = v >= 0 ? gemm_mfma_launch(s->stream, p, v) : gemm_generic_launch(s->stream, p);
    if (rc || (!bias && kind == WK_ACT_NONE)) return rc;
    return wk_bias_activation(s, dtype, kind, M, N, C, ldc, bias);
}

const char *wk_gemm_variant(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K, uint64_t lda, uint64_t ldb,
                            uint64_t ldc, const void *A, const void *B, const void *C) {
    GemmProblem p;
    // non-null stand-ins keep the alignment test meaningful when the caller passes no pointers
    alignas(16) static unsigned char dummy[16];
    if (build_problem(p, dtype, op_a, op_b, M, N, K, nullptr, A ? A : dummy, lda, B ? B : dummy, ldb, nullptr,
                      C ? const_cast<void *>(C) : dummy, ldc))
        return "invalid";
    // what a stream brings along (scratch for partial tiles, arrival counters), so that the answer is
    // the kernel a wk_gemm call on a stream would launch
    alignas(4) static uint32_t dummy_counter;
    p.scratch = dummy;
    p.scratch_bytes = WK_STREAM_SCRATCH_BYTES;
    p.counters = &dummy_counter;
    p.num_counters = WK_GEMM_COUNTERS;
    if (g_forced.load(std::memory_order_relaxed) == -2) {
        if (const int narrow = narrow_kind(p)) return narrow == 1 ? "thin" : "skinny";
        StripPlan sp;
        if (plan_strips(p, sp)) { // the body's kernel, marked: the strips beyond it are launches of their own
            const int bv = gemm_mfma_pick(sp.part[0]);
            static const std::array<std::string, 64> marked = [] {
                std::array<std::string, 64> names;
                for (int i = 0; i < 64 && gemm_mfma_variant_name(i); ++i) names[i] = std::string(gemm_mfma_variant_name(i)) + "+strips";
                return names;
            }();
            if (bv >= 0 && bv < 64) return marked[bv].c_str();
        }
    }
    const int v = choose(p);
    return v >= 0 ? gemm_mfma_variant_name(v) : k_generic_name;
}

const char *wk_gemm_variant_with_workspace(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K, uint64_t lda,
                                           uint64_t ldb, uint64_t ldc, const void *A, const void *B, const void *C,
                                           size_t workspace_bytes) {
    const char *plain = wk_gemm_variant(dtype, op_a, op_b, M, N, K, lda, ldb, ldc, A, B, C);
    if (!std::strcmp(plain, "invalid")) return plain;
    if (has_complex_packed_path(dtype)) {
        const int forced = g_forced.load(std::memory_order_relaxed);
        const size_t need = gemm_complex_packed_workspace_bytes(dtype, M, N, K);
        const bool fits = need && workspace_bytes >= need;
        GemmProblem q;
        q.dtype = dtype; q.M = M; q.N = N; q.K = K;
        if (forced == -3) return fits ? complex_packed_name(dtype) : "invalid";
        return fits && forced == -2 && complex_packed_pays(q) ? complex_packed_name(dtype) : plain;
    }
    if (!has_packed_path(dtype)) return plain;
    const int forced = g_forced.load(std::memory_order_relaxed);
    const size_t need = gemm_int_packed_workspace_bytes(dtype, M, N, K);
    const bool fits = need && workspace_bytes >= need;
    GemmProblem p;
    p.dtype = dtype; p.M = M; p.N = N; p.K = K;
    if (forced == -3) return fits ? k_packed_names[dtype] : "invalid";
    return fits && forced == -2 && packed_pays(p) ? k_packed_names[dtype] : plain;
}

int wk_gemm_split_plan(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K, const char *variant, uint32_t *shares,
                       uint32_t *klen, uint64_t *first_tile, uint64_t *tiles, size_t *scratch_bytes) {
    if (!shares || !klen || !first_tile || !tiles || !scratch_bytes) return WK_E_INVALID_VALUE;
    *shares = 1;
    *klen = 0;
    *first_tile = 0;
    *tiles = 0;
    *scratch_bytes = 0;
    GemmProblem p;
    alignas(16) static unsigned char dummy[16];
    alignas(4) static uint32_t dummy_counter;
    const uint64_t lda = op_a ? M : K, ldb = op_b ? K : N;
    int rc = build_problem(p, dtype, op_a, op_b, M, N, K, nullptr, dummy, lda, dummy, ldb, nullptr, dummy, N);
    if (rc) return rc;
    p.scratch = dummy;
    p.scratch_bytes = WK_STREAM_SCRATCH_BYTES;
    p.counters = &dummy_counter;
    p.num_counters = WK_GEMM_COUNTERS;
    int v = -1;
    if (variant) {
        for (int i = 0; gemm_mfma_variant_name(i); ++i)
            if (!std::strcmp(variant, gemm_mfma_variant_name(i))) v = i;
        if (v < 0 || gemm_mfma_variant_dtype(v) != dtype) return WK_E_INVALID_VALUE;
    } else {
        v = gemm_mfma_pick(p);
    }
    GemmSplitPlan plan;
    if (v >= 0 && gemm_mfma_split_plan(p, v, variant != nullptr, plan)) {
        *shares = plan.shares;
        *klen = plan.klen;
        *first_tile = plan.first_tile;
        *tiles = plan.tiles;
        *scratch_bytes = plan.bytes;
    }
    return WK_OK;
}

int wk_gemm_force_variant(const char *name) {
    if (!name || !std::strcmp(name, "auto")) { g_forced.store(-2); return WK_OK; }
    if (!std::strcmp(name, k_generic_name)) { g_forced.store(-1); return WK_OK; }
    for (const char *packed : k_packed_names)
        if (!std::strcmp(name, packed)) { g_forced.store(-3); return WK_OK; }
    for (const char *packed : k_complex_packed_names)
        if (!std::strcmp(name, packed)) { g_forced.store(-3); return WK_OK; }
    for (int v = 0; gemm_mfma_variant_name(v); ++v)
        if (!std::strcmp(name, gemm_mfma_variant_name(v))) { g_forced.store(v); return WK_OK; }
    return WK_E_INVALID_VALUE;
}

} // extern "C"
