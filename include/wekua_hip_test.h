/*
 * wekua_hip_test.h -- entry points of libwekua_hip that exist for tests, benchmarks and profiles
 * only.  The library exports them, but they are not part of the surface that replaces the
 * reference's OpenCL calls (wekua_hip.h) and product code must not depend on them: they expose or
 * override what wk_gemm chooses by itself, and several of them change process-wide state.  None has
 * a counterpart in the reference.
 */
#ifndef WEKUA_HIP_TEST_H
#define WEKUA_HIP_TEST_H

#include "wekua_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Name of the kernel variant wk_gemm() would launch for these arguments ("mfma_f32_256x128",
 * "tile64", "thin" for a product of one row or column (up to four where the next does not apply), "skinny" for one of
 * two to 32 (in one layout of the large operand: 64) rows or columns against a large other operand, ...).  A name that ends in "+strips" is the kernel of the body of whole tiles of a product
 * that wk_gemm launches in parts: the rows or columns beyond the body follow as products of their own.
 */
const char *wk_gemm_variant(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
                            uint64_t lda, uint64_t ldb, uint64_t ldc, const void *A, const void *B, const void *C);
/* The same for a call that brings workspace_bytes bytes of workspace ("mfma_i32_packed", ...). */
const char *wk_gemm_variant_with_workspace(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
                                           uint64_t lda, uint64_t ldb, uint64_t ldc, const void *A, const void *B,
                                           const void *C, size_t workspace_bytes);

/* Host arithmetic only, for tests and benchmarks: how a wk_gemm call on a stream lays out a product
 * whose k is split over work-groups.  Two cases: few tiles of C and a long k (every tile is split:
 * first_tile = 0), and a launch whose tiles do not fill whole rounds of the compute units (the whole
 * rounds, tiles 0 .. first_tile - 1, run as they are; the `tiles` left-over ones follow as a second
 * launch with k split).  A split tile goes to `shares` work-groups that each sum `klen` values of k
 * -- the last one what is left -- into partial tiles of `scratch_bytes` bytes in the stream's own
 * scratch memory; the last work-group to arrive at a tile adds them in the order of the shares, so
 * results are the same bits on every run.  variant NULL: the automatic choice (shares = 1 when it
 * does not split); a splitting variant's name ("mfma_f32_64x64z", "mfma_f64_64x64z",
 * "mfma_f32_256x128t", "mfma_f32_128x128t"): the plan that variant runs when forced.  No counterpart
 * in the reference. */
int wk_gemm_split_plan(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K, const char *variant,
                       uint32_t *shares, uint32_t *klen, uint64_t *first_tile, uint64_t *tiles, size_t *scratch_bytes);

/* Test and benchmark knob only, not for product code: force a gemm variant by name ("auto" restores
 * selection).  Process-wide, read by every wk_gemm call on every stream; changing it while a
 * PackedTensors keeps B invalidates what that handle remembers.  A forced variant whose kernel
 * cannot take the problem (a dimension or leading dimension of 2^31 or more) makes wk_gemm return
 * WK_E_INVALID_VALUE.  Returns WK_E_INVALID_VALUE for an unknown name. */
int wk_gemm_force_variant(const char *name);

/* Process-wide switches for A/B measurements; the library reads nothing from the environment.
 * Returns WK_E_INVALID_VALUE for an unknown name.
 *   "gemm_walk_rows" 1: the direct-to-LDS GEMM kernels number their tiles in groups of tile rows
 *                       instead of the XCD-local patches (default 0);
 *   "tail_strict"    1: a forced k-split tail variant ("...t") plans like the automatic choice (at
 *                       least one whole round in the body) instead of splitting every left-over tile,
 *                       which is what lets tests reach the tail path on small shapes (default 0);
 *                       wk_gemm_split_plan reports the plan of the mode in force;
 *   "alloc_colours"  0: wk_malloc returns blocks as the device allocator hands them out (default 1:
 *                       blocks of 1 MiB and more start 0 / 3 / 6 / 9 KiB into their allocation in turn);
 *   "stream_k"       0: the automatic choice never takes the kernels that deal their work by k-slabs
 *                       ("...k") (default 1); 2: those kernels deal every tile's k-slabs instead of running the
 *                       whole rounds of tiles whole; 3: they run the whole rounds whole also where the default would not;
 *   "persistent"     0: a launch of the direct-to-LDS GEMM kernels with between one and two rounds of the work-groups
 *                       that are resident at once is one work-group per tile, placed by the dispatcher as slots come
 *                       free (default 1: as many work-groups as are resident, each taking every n-th tile; 2: the same for
 *                       every launch of more tiles than are resident, which measures 0.5-2 % slower on long launches);
 *   "skinny"         0: products of at most 32 rows or columns of C never take the kernel that streams the large
 *                       operand into registers (default 1); n >= 2: that kernel splits k over n work-groups per
 *                       compute unit instead of what its registers allow to be resident (7: the default number, and
 *                       every tile walks k from the start of its share instead of from a place of its own);
 *   "strips"         0: a product is never multiplied in parts (body of whole tiles + strips); 2: thin strips are
 *                       split off whatever the cost model says (default 1: where the model puts the parts below
 *                       the whole). */
int wk_test_option(const char *name, int value);

/* Launch-cost probes for profiles: a kernel with the grid, work-group size (a multiple of 64) and dynamic LDS
 * claim of a GEMM launch that does nothing (kind 0), or only stores 16 floats per thread into dst (kind 1:
 * what the C write-back of a tile costs; dst_bytes >= work_groups * threads * 64). */
int wk_probe_launch(wk_stream *s, int kind, unsigned work_groups, unsigned threads, size_t lds_bytes, void *dst,
                    size_t dst_bytes);

/* Memory-rate probes in the shape of the AXPY stream kernel (one wavefront per work-group, one 16-byte
 * vector per lane, non-temporal loads, streaming stores): kind 0 copies src to dst, kind 1 only reads src,
 * kind 2 reads src and dst.  The reading kinds write a vector to dst only where all four of its words (of
 * src, or of src xor dst) equal `sentinel`: pass a value the data cannot hold.  They give the benchmark the
 * rates this memory system reaches with fewer streams than AXPY's two reads and one write.  bytes % 16 == 0. */
int wk_stream_probe(wk_stream *s, int kind, void *dst, const void *src, size_t bytes, unsigned sentinel);

/* A plain device-to-device streaming copy kernel of known size, used only to calibrate
 * profiler byte counters against a known amount of traffic. */
int wk_copy_kernel(wk_stream *s, void *dst, const void *src, size_t bytes);

#ifdef __cplusplus
}
#endif

#endif /* WEKUA_HIP_TEST_H */
