/*
 * wekua_hip.h -- C ABI of libwekua_hip: wekua's BLAS hot path (gemm, axpy) and the
 * device/tensor plumbing it needs, on one AMD Instinct MI355X (gfx950) through HIP.
 *
 * The reference (kython28/wekua) has no FFI boundary of its own for this path: its Zig
 * modules call OpenCL through the zig-opencl binding.  Each entry point below names
 * the reference interface it replaces, so that a wekua maintainer can swap
 * `cl.buffer.*` / `cl.kernel.enqueueNdRange` call sites for one `extern fn` each.
 *
 * Conventions
 *   - every function returns 0 (WK_OK) or a WK_E_* code; nothing throws or aborts;
 *   - pointers are DEVICE pointers unless the name starts with host_;
 *   - pitches / leading dimensions are in ELEMENTS of `dtype`;
 *   - host_alpha / host_beta point at ONE element of `dtype` in host memory and are
 *     read before the call returns; NULL means "absent" (Zig `null`), which selects
 *     the reference's option semantics, not the value 0 or 1;
 *   - all work is enqueued on the wk_stream (in order, like the reference's in-order
 *     cl_command_queue, src/core/command_queue.zig:130) and is complete after
 *     wk_stream_sync();
 *   - dtype = src/core/types.zig:60-86 getTypeIndex: 0 i8, 1 u8, 2 i16, 3 u16, 4 i32,
 *     5 u32, 6 i64, 7 u64, 8 f32, 9 f64, 10..19 the complex {real, imag} struct of each.
 *   - one thread per wk_stream at a time (the reference's queues have no locking either).
 */
#ifndef WEKUA_HIP_H
#define WEKUA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define WK_ABI_VERSION 1

/* ---- error codes: src/tensor/main.zig:25-33 `Errors`, plus allocator / device errors --- */
enum {
    WK_OK = 0,
    WK_E_INVALID_VALUE = 1,            /* Errors.InvalidValue            */
    WK_E_INVALID_COORDINATES = 2,      /* Errors.InvalidCoordinates      */
    WK_E_INVALID_BUFFER = 3,           /* Errors.InvalidBuffer           */
    WK_E_UNQUAL_TENSORS_ATTRIBUTE = 4, /* Errors.UnqualTensorsAttribute  */
    WK_E_UNQUAL_TENSORS_SHAPE = 5,     /* Errors.UnqualTensorsShape      */
    WK_E_UNQUAL_TENSORS_DIMENSION = 6, /* Errors.UnqualTensorsDimension  */
    WK_E_UNQUAL_TENSORS_CONTEXT = 7,   /* Errors.UnqualTensorsContext    */
    WK_E_OUT_OF_MEMORY = 8,            /* std.mem.Allocator.Error.OutOfMemory / hipErrorOutOfMemory */
    WK_E_TYPE_NOT_SUPPORTED = 9,       /* core.KernelsSet.Errors.TypeNotSupported (src/core/kernel.zig:151) */
    WK_E_NO_DEVICE = 10,               /* Context.init: DevicesArrayEmpty (src/core/context.zig:18) */
    WK_E_SCRATCH_TOO_SMALL = 11,       /* an operand beyond the fixed scratch array of a *_static entry point */
    WK_E_HIP_BASE = 1000               /* WK_E_HIP_BASE + hipError_t: replaces cl.errors.OpenCLError */
};

enum {
    WK_I8 = 0, WK_U8, WK_I16, WK_U16, WK_I32, WK_U32, WK_I64, WK_U64, WK_F32, WK_F64,
    WK_COMPLEX = 10, /* WK_COMPLEX + real id */
    WK_DTYPE_COUNT = 20
};

/* src/blas/gemm.zig:25-29 `Operation` */
enum { WK_OP_NO_TRANSPOSE = 0, WK_OP_TRANSPOSE = 1 };

typedef struct wk_device wk_device;
typedef struct wk_stream wk_stream;

/* What src/core/command_queue.zig:10-229 caches per queue from clGetDeviceInfo. */
typedef struct wk_props {
    char     name[64];
    char     arch[32];               /* "gfx950..." */
    int      ordinal;
    int      compute_units;          /* CommandQueue.compute_units */
    int      wavefront_size;
    int      max_work_group_size;    /* CommandQueue.max_work_group_size */
    uint64_t local_mem_bytes;        /* CommandQueue.local_mem_size (LDS per work-group) */
    uint64_t global_mem_bytes;
    int      cache_line_size;        /* CommandQueue.cache_line_size */
    int      clock_mhz;
} wk_props;

const char *wk_strerror(int code);
int         wk_abi_version(void);
size_t      wk_dtype_size(int dtype);

/* ---- device / stream: src/core/context.zig:13-196, command_queue.zig:100-160 ---------- */
int  wk_device_count(int *out_count);                     /* cl.platform/device enumeration   */
int  wk_device_open(int ordinal, wk_device **out);        /* Context.init / initFromBestDevice */
void wk_device_close(wk_device *dev);                     /* Context.deinit                    */
int  wk_device_props(wk_device *dev, wk_props *out);      /* CommandQueue.init device queries  */
int  wk_stream_create(wk_device *dev, wk_stream **out);   /* cl.command_queue.create           */
void wk_stream_destroy(wk_stream *s);                     /* cl.command_queue.release          */
int  wk_stream_sync(wk_stream *s);                        /* Pipeline.waitAndCleanup, src/core/pipeline.zig:47-61 */
void *wk_stream_native(wk_stream *s);                     /* the hipStream_t, for event timing by the caller */

/* ---- events: cl.event.* as used by src/core/pipeline.zig:35-61 (ordering itself comes from the
 * in-order stream; events are for waiting on a point of the stream and for timing, which the
 * reference's queue cannot do: it is created without CL_QUEUE_PROFILING_ENABLE) ------------ */
typedef struct wk_event wk_event;
int  wk_event_create(wk_device *dev, wk_event **out);
void wk_event_destroy(wk_event *e);                       /* cl.event.release */
int  wk_event_record(wk_event *e, wk_stream *s);          /* the event a cl enqueue call returns */
int  wk_event_sync(wk_event *e);                          /* cl.event.wait */
int  wk_event_elapsed_ms(wk_event *start, wk_event *stop, float *out_ms);

/* ---- memory: cl.buffer.create/release (src/tensor/main.zig:229-234,253-263) -----------
 * Pointers from wk_malloc are at least 1 KiB aligned and must go back through wk_free (blocks of
 * 1 MiB and more start 0 / 3 / 6 / 9 KiB into their device allocation in turn, which spreads
 * streams that are walked in step over the memory channels). */
int  wk_malloc(wk_device *dev, size_t bytes, void **out_dptr);
int  wk_free(wk_device *dev, void *dptr);
int  wk_mem_info(wk_device *dev, size_t *free_bytes, size_t *total_bytes);
/* cl.buffer.fill of the whole buffer: fill.zeroes, src/tensor/fill.zig:70-95 */
int  wk_memset_async(wk_stream *s, void *dptr, int byte, size_t bytes);
/* cl.buffer.writeRect: memory.readFromBuffer (HOST -> DEVICE), src/tensor/memory/read_from_buffer.zig:13-63.
 * Copies `slices` x `rows` runs of width_bytes; pitches in BYTES.  The host buffer must
 * stay valid until wk_stream_sync(). */
int  wk_copy_h2d_rect_async(wk_stream *s, void *dst, size_t dst_row_pitch_bytes, size_t dst_slice_pitch_bytes,
                            const void *host_src, size_t src_row_pitch_bytes, size_t src_slice_pitch_bytes,
                            size_t width_bytes, size_t rows, size_t slices);
/* cl.buffer.readRect: memory.writeToBuffer (DEVICE -> HOST), src/tensor/memory/write_to_buffer.zig:13-63 */
int  wk_copy_d2h_rect_async(wk_stream *s, void *host_dst, size_t dst_row_pitch_bytes, size_t dst_slice_pitch_bytes,
                            const void *src, size_t src_row_pitch_bytes, size_t src_slice_pitch_bytes,
                            size_t width_bytes, size_t rows, size_t slices);
/* cl.buffer.copyRect: memory.copy, src/tensor/memory/copy.zig */
int  wk_copy_d2d_rect_async(wk_stream *s, void *dst, size_t dst_row_pitch_bytes, size_t dst_slice_pitch_bytes,
                            const void *src, size_t src_row_pitch_bytes, size_t src_slice_pitch_bytes,
                            size_t width_bytes, size_t rows, size_t slices);

/* ---- support kernels used by the reference's gemm/axpy tests -------------------------- */
/* fill.constant / fill.one: `fill` kernel over the logical {depth, rows, cols} region,
 * src/tensor/fill.zig:16-57, kernels/fill.cl */
int  wk_fill(wk_stream *s, int dtype, void *dptr, const uint64_t shape3[3],
             uint64_t row_pitch, uint64_t slice_pitch, const void *host_scalar);
/* identity: ones at index i*sum(pitches) for i < size, src/tensor/identity.zig:16-70,
 * kernels/identity.cl.  The caller zeroes the buffer first (as identity.zig:27 does). */
int  wk_identity(wk_stream *s, int dtype, void *dptr, uint64_t size, uint64_t pitch_sum);

/* ---- the hot path ----------------------------------------------------------------------- */
/* blas.axpy: y = alpha*x + y over the logical {depth, rows, cols} region
 * (src/blas/axpy.zig:93-169, kernels/axpy.cl:3-72).
 *   host_alpha == NULL      -> y += x
 *   alpha == -1 (floats: |alpha+1| < eps; signed ints exactly; axpy.zig:66-91) -> y -= x
 *   otherwise               -> y[i] = fma(alpha, x[i], y[i]) for floats, wrapping for ints,
 *                              the 3-multiply product of wekua_cl_lib.cl:648-653 for complex.
 * x and y must not overlap.  A region whose rows are contiguous in both operands
 * (row_pitch == cols, slice_pitch == rows*cols) runs the vectorised streaming kernel. */
int  wk_axpy(wk_stream *s, int dtype, const uint64_t shape3[3],
             const void *x, uint64_t x_row_pitch, uint64_t x_slice_pitch,
             void *y, uint64_t y_row_pitch, uint64_t y_slice_pitch,
             const void *host_alpha);

/* blas.gemm: C = alpha*op(A)*op(B) + beta*C  (src/blas/gemm.zig:834-874; kernels
 * gemm_nxn_gpu.cl, gemm_nxn.cl, gemm_2x2.cl and their packed twins).
 *   op(A) is M x K, op(B) is K x N, C is M x N, all row-major; A is stored M x K
 *   (op_a = N) or K x M (op_a = T) with leading dimension lda, likewise B.
 *   Option semantics (gemm.zig:500-501,591-602):
 *     alpha NULL, beta NULL -> C = op(A)op(B)                 (C is not read)
 *     alpha set,  beta NULL -> C = alpha*op(A)op(B)           (C is not read)
 *     beta set              -> C = (alpha or 1)*op(A)op(B) + beta*C_old; C_old is read and
 *                              multiplied even when beta == 0 (NaN/Inf propagate).
 *   Integers wrap modulo 2^width; f32/f64 accumulate in their own precision.
 *   The reference's PackedTensors pass (gemm.zig:60-359, 705-720: pack A and B into two scratch
 *   tensors before every product) survives for the 8-, 16- and 32-bit integers: with `workspace` of
 *   at least wk_gemm_workspace_bytes() bytes of device memory (16-byte aligned; what
 *   blas.PackedTensors holds) products that are large enough first pack both operands into
 *   signed-digit planes there and then run a lean int8 matrix-core kernel (for 8 and 16 bits the
 *   only matrix-core path); the result is the same bits either way.  cf32 / cf64 and the complex
 *   8/16/32-bit integers use a workspace too: B is rebuilt there as its real 2K x 2N form
 *   (transposed operands are turned first) and the product runs on the real matrix-core kernels
 *   (floats: to the float tolerance; integers: the same bits).  Every other type stages
 *   its tiles through LDS straight from the row-major operands, asks for 0 bytes and ignores the
 *   workspace, which may always be NULL.  The workspace is overwritten by every call that uses it:
 *   calls sharing one must be ordered on one stream. */
int    wk_gemm(wk_stream *s, int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
               const void *host_alpha, const void *A, uint64_t lda, const void *B, uint64_t ldb,
               const void *host_beta, void *C, uint64_t ldc, void *workspace, size_t workspace_bytes);
size_t wk_gemm_workspace_bytes(int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K);

/* wk_gemm for a caller whose op(B) has not changed since the previous call: the workspace still
 * holds B's packed form (digit planes of an integer B; the real 2K x 2N form of a
 * complex B, which has alpha folded in), so only A is packed again.  The reference packs both
 * operands before every product (gemm.zig:713-719) although its callers' B is usually a weight
 * matrix that changes once per step; this is the entry point behind blas.PackedTensors.keepB.
 * The caller guarantees: the previous call that used this workspace was a wk_gemm or
 * wk_gemm_packed_b_kept with the same dtype, op_b, M, N, K and B contents (for the complex types also
 * the same alpha, present or absent alike), and nothing else has written the workspace since.  A
 * violated guarantee gives a wrong product, never an access outside the operands.  Problems that
 * do not use the workspace run exactly as under wk_gemm. */
int    wk_gemm_packed_b_kept(wk_stream *s, int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
                             const void *host_alpha, const void *A, uint64_t lda, const void *B, uint64_t ldb,
                             const void *host_beta, void *C, uint64_t ldc, void *workspace, size_t workspace_bytes);

/* ---- around the hot path: what one MLP training step needs besides gemm / axpy -----------------
 * (f32 and f64 only; every tensor is a logical {depth, rows, cols} region with its own pitches) */
enum { WK_ACT_NONE = -1, WK_ACT_SIGMOID = 0, WK_ACT_TANH = 1 };
/* math.dot, the in-place Hadamard product x *= y: src/math/basic.zig:18-77, kernels/dot.cl */
int  wk_hadamard(wk_stream *s, int dtype, const uint64_t shape3[3], void *x, uint64_t x_row_pitch, uint64_t x_slice_pitch,
                 const void *y, uint64_t y_row_pitch, uint64_t y_slice_pitch);
/* Activation.run in place: Sigmoid 1/(1+exp(-x)) (src/nn/activation/kernels/sigmoid.cl:3-19),
 * Tanh (src/nn/activation/tanh.zig:16-31 -> math.tanh, src/math/kernels/trig.cl) */
int  wk_activation(wk_stream *s, int dtype, int kind, const uint64_t shape3[3], void *x, uint64_t row_pitch, uint64_t slice_pitch);
/* Activation.getDerivative from the activation OUTPUT y: sigmoid_dev y(1-y) (sigmoid.cl:21-38),
 * tanh_dev 1-y^2 (src/nn/activation/kernels/tanh.cl) */
int  wk_activation_dev(wk_stream *s, int dtype, int kind, const uint64_t shape3[3], const void *out, uint64_t out_row_pitch,
                       uint64_t out_slice_pitch, void *dev, uint64_t dev_row_pitch, uint64_t dev_slice_pitch);
/* Linear.addBias (src/nn/layer/kernels/bias.cl: out[r][c] += bias[c]) fused with the activation that
 * follows it in Linear.forward (src/nn/layer/linear.zig:480-525).  bias may be NULL, kind WK_ACT_NONE. */
int  wk_bias_activation(wk_stream *s, int dtype, int kind, uint64_t rows, uint64_t cols, void *out, uint64_t out_pitch,
                        const void *bias);
/* One matrix of Linear.forward in one call (src/nn/layer/linear.zig:480-525: blas.gemm, addBias,
 * act.run): C = act(op(A)op(B) + bias[col]), f32 / f64.  For op N, T (x times the transposed weight
 * matrix, what Linear runs) bias and activation are applied in the epilogue of the matrix-core kernel,
 * to the same bits as wk_gemm followed by wk_bias_activation; any other layout runs those two.
 * bias may be NULL, kind WK_ACT_NONE. */
int  wk_gemm_bias_activation(wk_stream *s, int dtype, int op_a, int op_b, uint64_t M, uint64_t N, uint64_t K,
                             const void *A, uint64_t lda, const void *B, uint64_t ldb, void *C, uint64_t ldc,
                             const void *bias, int kind);
/* Linear.getBiasSensitivity: bias_grad[c] = sum_r sens[r][c] (src/nn/layer/kernels/bias_step.cl) */
int  wk_bias_step(wk_stream *s, int dtype, uint64_t rows, uint64_t cols, const void *sens, uint64_t pitch, void *bias_grad);
/* wk_bias_step for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it).  No counterpart in the reference.  Same arguments, same
 * kernels and bit for bit the same result, but the band partials live in an array that is part of the
 * library's code object (WK_BIAS_STEP_STATIC_SCRATCH_BYTES per device, held until the process ends),
 * whose address wk_device_open looks up once per device.  The call itself allocates and frees nothing.
 * Limit: cols * element size <= WK_BIAS_STEP_STATIC_SCRATCH_BYTES / 2 (131072 f32 or 65536 f64 columns),
 * beyond it WK_E_SCRATCH_TOO_SMALL; f32 / f64 only.  Every call on a device uses that device's one
 * array: nothing in it has to start at zero (each partial is written before it is read), but two calls
 * that overlap on one device -- on different streams or from different threads -- race. */
#define WK_BIAS_STEP_STATIC_SCRATCH_BYTES (1u << 20)
int  wk_bias_step_static(wk_stream *s, int dtype, uint64_t rows, uint64_t cols, const void *sens, uint64_t pitch, void *bias_grad);
/* Linear.backward's element-wise half in one pass over the layer's output (src/nn/layer/linear.zig:606-640:
 * act.getDerivative, math.dot, getBiasSensitivity): dev = act'(out), sens *= dev, bias_grad[c] = sum_r sens[r][c]
 * of the new sens (skipped when bias_grad is NULL).  The same values, bit for bit, as wk_activation_dev,
 * wk_hadamard and wk_bias_step one after the other, with half the memory traffic.  kind WK_ACT_NONE: dev is
 * read as it is (the reference multiplies by its cached derivative tensor whatever it holds) and out may be NULL. */
int  wk_sensitivity_step(wk_stream *s, int dtype, int kind, uint64_t rows, uint64_t cols, const void *out, uint64_t out_pitch,
                         void *sens, uint64_t sens_pitch, void *dev, uint64_t dev_pitch, void *bias_grad);
/* loss.mse kernel: err = expected - output; error = err^2; dev = -2*err when dev != NULL
 * (src/nn/loss/kernels/mse.cl:3-35, src/nn/loss/mse.zig:63-132) */
int  wk_mse(wk_stream *s, int dtype, const uint64_t shape3[3], const void *output, uint64_t out_row_pitch, uint64_t out_slice_pitch,
            const void *expected, uint64_t exp_row_pitch, uint64_t exp_slice_pitch, void *error, uint64_t err_row_pitch,
            uint64_t err_slice_pitch, void *dev, uint64_t dev_row_pitch, uint64_t dev_slice_pitch);
/* math.sum / math.mean (src/math/basic.zig:128-244): scale * sum of the logical elements into one
 * element at dev_result; workspace holds wk_sum_workspace_bytes(dtype) bytes of device memory. */
size_t wk_sum_workspace_bytes(int dtype);
int  wk_sum(wk_stream *s, int dtype, const uint64_t shape3[3], const void *x, uint64_t row_pitch, uint64_t slice_pitch,
            void *workspace, void *dev_result, double scale);
/* Adam update.  The reference's Zig tree has no Adam (src/nn/optimizers/adam.zig is empty); this is
 * the textbook rule with the reference's sibling optimizers' epsilon placement (rmsprop.cl:54):
 * m = b1 m + (1-b1) g; v = b2 v + (1-b2) g^2; w -= lr/(1-b1^t) * m / (sqrt(v/(1-b2^t)) + eps).
 * m and v share one layout. */
int  wk_adam_step(wk_stream *s, int dtype, const uint64_t shape3[3], void *w, uint64_t w_row_pitch, uint64_t w_slice_pitch,
                  const void *g, uint64_t g_row_pitch, uint64_t g_slice_pitch, void *m, void *v, uint64_t mv_row_pitch,
                  uint64_t mv_slice_pitch, double lr, double beta1, double beta2, double eps, uint64_t step);
/* The same update of `count` parameter tensors (host array, read before the call returns) in one launch
 * per eight tensors instead of one per tensor; every element gets exactly the arithmetic of wk_adam_step.
 * Tensors that do not allow 16-byte accesses make the call fall back to one wk_adam_step each. */
typedef struct wk_adam_tensor {
    void       *w;
    const void *g;
    void       *m, *v;
    uint64_t    shape3[3];
    uint64_t    w_row_pitch, w_slice_pitch, g_row_pitch, g_slice_pitch, mv_row_pitch, mv_slice_pitch;
} wk_adam_tensor;
int  wk_adam_step_multi(wk_stream *s, int dtype, uint32_t count, const wk_adam_tensor *host_tensors, double lr, double beta1,
                        double beta2, double eps, uint64_t step);

/* ---- tensor support operations (src/tensor) --------------------------------------------------- */
#define WK_MAX_DIMS 8
/* transpose (src/tensor/transpose.zig:14-105, kernels/transpose.cl): swaps dimensions dim0 != dim1 of an
 * ndim-dimensional tensor (ndim <= WK_MAX_DIMS).  `shape` and `src_pitches` describe the source,
 * `dst_pitches` the destination, whose shape is `shape` with the two dimensions exchanged; pitches are
 * element strides per dimension (the last is 1), as Tensor.dimensions.pitches (src/tensor/main.zig:198-220). */
int  wk_transpose(wk_stream *s, int dtype, int ndim, const uint64_t *shape, const uint64_t *src_pitches,
                  const uint64_t *dst_pitches, int dim0, int dim1, const void *src, void *dst);
/* random.uniform (src/tensor/random/uniform.zig:60-135, kernels/uniform.cl).  host_min == NULL: floats
 * hash / 2^64 in [0, 1], integers the low bits of the hash.  Otherwise host_min / host_range point to
 * one value of the real component type and every value is min + hash / 2^64 * range, formed in double.
 * The hash is the reference's; it is keyed on the LOGICAL element index (complex: 2*index, 2*index + 1),
 * where the reference keys it on the index in its padded layout, so the two streams agree exactly when
 * the reference's tensor has no padding. */
int  wk_random_uniform(wk_stream *s, int dtype, const uint64_t shape3[3], void *ptr, uint64_t row_pitch, uint64_t slice_pitch,
                       uint64_t seed, const void *host_min, const void *host_range);
/* The hash random.uniform draws from (kernels/uniform.cl:31-55), on the host. */
uint64_t wk_random_hash(uint64_t index, uint64_t seed);
/* toComplex / toReal (src/tensor/convertions/to_complex.zig:52-98, to_real.zig:51-97): copy a real
 * tensor into the real (space 0) or imaginary (space 1) components of a complex one, or back.
 * real_dtype is the id of the component type (0..9); pitches are in elements of each tensor's own type. */
int  wk_to_complex(wk_stream *s, int real_dtype, const uint64_t shape3[3], const void *src, uint64_t src_row_pitch,
                   uint64_t src_slice_pitch, void *dst, uint64_t dst_row_pitch, uint64_t dst_slice_pitch, int space);
int  wk_to_real(wk_stream *s, int real_dtype, const uint64_t shape3[3], const void *src, uint64_t src_row_pitch,
                uint64_t src_slice_pitch, void *dst, uint64_t dst_row_pitch, uint64_t dst_slice_pitch, int space);

#ifdef __cplusplus
}
#endif
#endif /* WEKUA_HIP_H */
