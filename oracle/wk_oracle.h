/*
 * wk_oracle.h -- CPU restatement of wekua's BLAS hot path (gemm / axpy).
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker for the HIP
 * implementation and the timed "port" CPU baseline of the benchmark.  Nothing
 * in the shipped GPU path may link, load or call it.
 *
 * It follows the reference's OpenCL CPU-device algorithm file by file:
 *   src/blas/kernels/axpy.cl:3-72            element update y += alpha*x
 *   src/blas/axpy.zig:66-111                 alpha classification (null / -1 / other)
 *   src/blas/kernels/gemm_2x2.cl:65-277      2x2 work-item kernel
 *   src/blas/kernels/gemm_nxn.cl:107-423     BSxBS work-item kernel, 2x2 / 4x4 micro-kernel
 *   src/blas/kernels/gemm_pack.cl:50-96      tile packing pass
 *   src/blas/kernels/gemm_nxn_pack.cl:66-393 packed-tile kernel (same arithmetic as gemm_nxn.cl)
 *   src/core/wekua_cl_lib.cl:591-609         sum() lane tree, :648-653 3-multiply complex product
 *   src/tensor/main.zig:142-199              padded tensor layout the kernels rely on
 *   src/tensor/work_configuration.zig:110-193 default block size per tensor (CPU: .global branch)
 *   src/blas/gemm.zig:42-58,487-617,695-832  block choice, k padding, option semantics of alpha/beta
 *
 * Parity status of each function (what pins it) is listed in wk_oracle.c.
 */
#ifndef WK_ORACLE_H
#define WK_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* dtype ids = src/core/types.zig:60-86 getTypeIndex (0..9 real, 10..19 complex of the same order) */
enum {
    WKO_I8 = 0, WKO_U8, WKO_I16, WKO_U16, WKO_I32, WKO_U32, WKO_I64, WKO_U64, WKO_F32, WKO_F64,
    WKO_COMPLEX = 10 /* WKO_COMPLEX + real id */
};

typedef struct wko_layout {
    uint64_t depth;                  /* product of all dims before the last two        */
    uint64_t rows;                   /* penultimate dim (1 for 1-D tensors)            */
    uint64_t cols;                   /* last dim                                        */
    uint64_t padded_rows;            /* rows + rows % 2                                 */
    uint64_t row_pitch;              /* elements                                        */
    uint64_t row_pitch_for_vectors;  /* row_pitch / vector_width                        */
    uint64_t slice_pitch;            /* row_pitch * padded_rows                         */
    uint64_t number_of_elements;     /* slice_pitch * depth                             */
    uint64_t number_of_elements_without_padding;
    uint64_t number_of_vectors;
} wko_layout;

size_t wko_dtype_size(int dtype);

/* src/tensor/main.zig:142-199.  vector_width is the device's native width for the
 * dtype (1 disables vectors, as does a complex dtype or vectors_enabled == 0). */
int wko_tensor_layout(const uint64_t *shape, int ndim, int dtype, uint64_t vector_width,
                      int vectors_enabled, wko_layout *out);

/* src/tensor/work_configuration.zig:110-193, `.global` (CPU) branch: the largest block
 * in {2,..,64} dividing both padded dims whose BS x BS*vw tile fits 16 KiB. */
int wko_default_block_cpu(uint64_t padded_rows, uint64_t row_pitch, uint64_t vector_width, size_t elem_size);

/* src/blas/gemm.zig:42-58: largest block <= default_block dividing k_size. */
int wko_get_algorithm(int default_block, uint64_t k_size);

/* y = alpha*x + y over a logical {depth, rows, cols} region with pitches in elements
 * (scalar build of axpy.cl).  alpha == NULL: y += x.  alpha == -1 (floats: within
 * machine eps): y -= x.  contract != 0: float multiply-add is fused (fma). */
int wko_axpy(int dtype, const uint64_t shape3[3],
             const void *x, uint64_t x_row_pitch, uint64_t x_slice_pitch,
             void *y, uint64_t y_row_pitch, uint64_t y_slice_pitch,
             const void *alpha, int contract);
/* The same with the elements spread over `threads` host threads (<= 0: all), the way an OpenCL CPU
 * device spreads its work-items over the cores; every element is computed as by wko_axpy. */
int wko_axpy_threads(int dtype, const uint64_t shape3[3],
                     const void *x, uint64_t x_row_pitch, uint64_t x_slice_pitch,
                     void *y, uint64_t y_row_pitch, uint64_t y_slice_pitch,
                     const void *alpha, int contract, int threads);

/* C = alpha*op(A)*op(B) + beta*C exactly as the reference's CPU device computes it.
 *  - A, B, C are dense row-major host arrays with leading dimensions lda/ldb/ldc
 *    (elements); stored shapes follow the op flags as in gemm.zig:471-480.
 *  - alpha/beta: NULL = absent (gemm.zig:500-501,591-602): both NULL overwrites C;
 *    beta given reads C_old and multiplies it even when beta == 0.
 *  - vector_width: the emulated device's native width (1 = scalar build).  As in
 *    gemm.zig:503-508 the unpacked path only uses vectors for op_a=N, op_b=T.
 *  - packed != 0: take the PackedTensors path (two pack passes, then the packed kernel).
 *  - block: 0 = choose like the reference, else force (must divide the padded dims).
 *  - contract: fuse the float multiply-adds.   threads: OpenMP threads (<=0: all).
 * Operands are copied into the reference's padded layout first, so every read the
 * kernels make beyond the logical region sees zeros, as after Tensor.alloc. */
int wko_gemm(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
             const void *alpha, const void *A, uint64_t lda, const void *B, uint64_t ldb,
             const void *beta, void *C, uint64_t ldc,
             uint64_t vector_width, int packed, int block, int contract, int threads);

/* The block size wko_gemm would pick for these arguments (for reporting). */
int wko_gemm_block(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
                   uint64_t vector_width, int packed);

/* One pack pass (gemm_pack.cl:50-96) on a dense rows x cols source into a dense
 * [tiles][ktiles][BS][BS*vw] destination that must be zero-initialised by the caller.
 * transpose as in gemm.zig:285-289.  Returns number of elements of dst written region. */
int wko_pack(int dtype, const void *src, uint64_t src_rows, uint64_t src_cols, uint64_t src_pitch,
             void *dst, uint64_t tiles, uint64_t ktiles, int block, uint64_t vector_width, int transpose);

#ifdef __cplusplus
}
#endif
#endif
